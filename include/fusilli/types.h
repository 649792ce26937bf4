// Element types of the graph API.
//
// Same enumerators, in the same order, as the reference's DataType
// (attributes/types.h:27-45) — the numeric values double as the C ABI's
// fhip_dtype — plus FP8E4M3 (OCP e4m3fn, the gfx950 hardware fp8), which the
// reference lacks.  The MLIR spellings are kept because the benchmark driver
// uses them as CLI type names (benchmarks/driver.cpp:41).
#ifndef FUSILLI_TYPES_H
#define FUSILLI_TYPES_H

#include <cstdint>
#include <string>

namespace fusilli {

enum class DataType : uint8_t {
  NotSet,
  Half,
  BFloat16,
  Float,
  Double,
  Uint8,
  Int4,
  Int8,
  Int16,
  Int32,
  Int64,
  Boolean,
  FP8E5M2,
  FP8E4M3,
};

inline bool isIntegerType(DataType t) {
  return t == DataType::Uint8 || t == DataType::Int4 || t == DataType::Int8 ||
         t == DataType::Int16 || t == DataType::Int32 || t == DataType::Int64;
}
inline bool isIntegralOrBoolType(DataType t) {
  return isIntegerType(t) || t == DataType::Boolean;
}

inline const char *dataTypeAsm(DataType t) {
  switch (t) {
  case DataType::Half:
    return "f16";
  case DataType::BFloat16:
    return "bf16";
  case DataType::Float:
    return "f32";
  case DataType::Double:
    return "f64";
  case DataType::Uint8:
    return "ui8";
  case DataType::Int4:
    return "si4";
  case DataType::Int8:
    return "si8";
  case DataType::Int16:
    return "si16";
  case DataType::Int32:
    return "si32";
  case DataType::Int64:
    return "si64";
  case DataType::Boolean:
    return "i1";
  case DataType::FP8E5M2:
    return "f8E5M2";
  case DataType::FP8E4M3:
    return "f8E4M3FN";
  default:
    return "notset";
  }
}

inline DataType dataTypeFromAsm(const std::string &s) {
  for (int i = 1; i <= static_cast<int>(DataType::FP8E4M3); ++i)
    if (s == dataTypeAsm(static_cast<DataType>(i)))
      return static_cast<DataType>(i);
  return DataType::NotSet;
}

// Bytes per element in device buffers (Int4 is not executable here).
inline size_t dataTypeSize(DataType t) {
  switch (t) {
  case DataType::Half:
  case DataType::BFloat16:
  case DataType::Int16:
    return 2;
  case DataType::Float:
  case DataType::Int32:
    return 4;
  case DataType::Double:
  case DataType::Int64:
    return 8;
  case DataType::Uint8:
  case DataType::Int8:
  case DataType::Boolean:
  case DataType::FP8E5M2:
  case DataType::FP8E4M3:
    return 1;
  default:
    return 0;
  }
}

// Native 16-bit floats (ROCm clang has both; reference
// support/float_types.h:101-102).
using half = _Float16;
using bf16 = __bf16;

// One-byte storage tags so Buffer::allocate<T> can tell the two fp8 formats
// apart.
struct fp8e4m3 {
  uint8_t bits;
};
struct fp8e5m2 {
  uint8_t bits;
};

template <typename T> struct DataTypeOf;
#define FUSILLI_MAP_TYPE(T, DT)                                                \
  template <> struct DataTypeOf<T> {                                           \
    static constexpr DataType value = DataType::DT;                            \
  };
FUSILLI_MAP_TYPE(half, Half)
FUSILLI_MAP_TYPE(bf16, BFloat16)
FUSILLI_MAP_TYPE(float, Float)
FUSILLI_MAP_TYPE(double, Double)
FUSILLI_MAP_TYPE(uint8_t, Uint8)
FUSILLI_MAP_TYPE(int8_t, Int8)
FUSILLI_MAP_TYPE(int16_t, Int16)
FUSILLI_MAP_TYPE(int32_t, Int32)
FUSILLI_MAP_TYPE(int64_t, Int64)
FUSILLI_MAP_TYPE(bool, Boolean)
FUSILLI_MAP_TYPE(fp8e4m3, FP8E4M3)
FUSILLI_MAP_TYPE(fp8e5m2, FP8E5M2)
#undef FUSILLI_MAP_TYPE

} // namespace fusilli

#endif // FUSILLI_TYPES_H
