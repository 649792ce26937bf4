// What this MI355X sustains, measured with nothing in the way: the yardsticks
// that the kernels' fractions of the published peaks are read against.
//
//   mfma   register-resident MFMA loops (no memory traffic at all), bf16 /
//          int8 / fp8, with random and with constant operand bits: the rate
//          the matrix pipes hold at the clock the chip settles to under that
//          load (operand bits that toggle draw more power than constant ones)
//   copy   16-byte loads and non-temporal stores (one write per read) and
//          read-only passes, over 64 MiB windows of 1 GiB buffers and over
//          the whole buffers
//
// Prints one JSON object.  Usage: peaks [seconds per measurement, default 0.3]
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                               \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                  \
      exit(1);                                                                 \
    }                                                                          \
  } while (0)

enum { K_BF16 = 0, K_I8 = 1, K_FP8 = 2 };

__device__ __forceinline__ uint32_t mix(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// 8 independent accumulators per wavefront, ITERS x 8 MFMAs; operands live in
// registers.  random = 0: all operand registers hold the same constant.
template <int KIND>
__global__ __launch_bounds__(512) void mfma_loop(int iters, int random,
                                                 float *sink) {
  uint32_t a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    const uint32_t h = mix(threadIdx.x * 16 + i + blockIdx.x * 8192);
    if (KIND == K_BF16) { // finite bf16 pairs of moderate magnitude
      a[i] = random ? ((h & 0x807f807fu) | 0x3f003f00u) : 0x3f803f80u;
      b[i] = random ? ((mix(h) & 0x807f807fu) | 0x3f003f00u) : 0x3f803f80u;
    } else if (KIND == K_I8) {
      a[i] = random ? h : 0x01010101u;
      b[i] = random ? mix(h) : 0x01010101u;
    } else { // e4m3 bytes with exponent below the top
      a[i] = random ? (h & 0xb7b7b7b7u) : 0x38383838u;
      b[i] = random ? (mix(h) & 0xb7b7b7b7u) : 0x38383838u;
    }
  }
  float out = 0.f;
  if constexpr (KIND == K_I8) {
    i32x16 acc[8];
    for (int i = 0; i < 8; ++i)
      for (int r = 0; r < 16; ++r)
        acc[i][r] = 0;
    const i32x4 va = {(int)a[0], (int)a[1], (int)a[2], (int)a[3]};
    const i32x4 vb = {(int)b[0], (int)b[1], (int)b[2], (int)b[3]};
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(va, vb, acc[i], 0, 0, 0);
    for (int i = 0; i < 8; ++i)
      out += (float)acc[i][0];
  } else {
    f32x16 acc[8];
    for (int i = 0; i < 8; ++i)
      for (int r = 0; r < 16; ++r)
        acc[i][r] = 0.f;
    if constexpr (KIND == K_BF16) {
      const u32x4 ua = {a[0], a[1], a[2], a[3]}, ub = {b[0], b[1], b[2], b[3]};
      const bf16x8 va = __builtin_bit_cast(bf16x8, ua);
      const bf16x8 vb = __builtin_bit_cast(bf16x8, ub);
      for (int it = 0; it < iters; ++it)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, vb, acc[i], 0, 0, 0);
    } else {
      const i32x8 va = {(int)a[0], (int)a[1], (int)a[2], (int)a[3],
                        (int)a[4], (int)a[5], (int)a[6], (int)a[7]};
      const i32x8 vb = {(int)b[0], (int)b[1], (int)b[2], (int)b[3],
                        (int)b[4], (int)b[5], (int)b[6], (int)b[7]};
      for (int it = 0; it < iters; ++it)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              va, vb, acc[i], 0, 0, 0, 0, 0, 0);
    }
    for (int i = 0; i < 8; ++i)
      out += acc[i][0];
  }
  if (out == 12345.678f) // never true; keeps the loop
    sink[blockIdx.x * blockDim.x + threadIdx.x] = out;
}

// The same with the 16 x 16 MFMA shapes (K = 32 / 64 / 128): 16 independent
// accumulators of four registers per wavefront.
template <int KIND>
__global__ __launch_bounds__(512) void mfma16_loop(int iters, int random, float *sink) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef int i32x4v __attribute__((ext_vector_type(4)));
  uint32_t a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    const uint32_t h = mix(threadIdx.x * 16 + i + blockIdx.x * 8192);
    if (KIND == K_BF16) {
      a[i] = random ? ((h & 0x807f807fu) | 0x3f003f00u) : 0x3f803f80u;
      b[i] = random ? ((mix(h) & 0x807f807fu) | 0x3f003f00u) : 0x3f803f80u;
    } else if (KIND == K_I8) {
      a[i] = random ? h : 0x01010101u;
      b[i] = random ? mix(h) : 0x01010101u;
    } else {
      a[i] = random ? (h & 0xb7b7b7b7u) : 0x38383838u;
      b[i] = random ? (mix(h) & 0xb7b7b7b7u) : 0x38383838u;
    }
  }
  float out = 0.f;
  if constexpr (KIND == K_I8) {
    i32x4v acc[16];
    for (int i = 0; i < 16; ++i)
      for (int r = 0; r < 4; ++r)
        acc[i][r] = 0;
    const i32x4 va = {(int)a[0], (int)a[1], (int)a[2], (int)a[3]};
    const i32x4 vb = {(int)b[0], (int)b[1], (int)b[2], (int)b[3]};
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(va, vb, acc[i], 0, 0, 0);
    for (int i = 0; i < 16; ++i)
      out += (float)acc[i][0];
  } else {
    f32x4 acc[16];
    for (int i = 0; i < 16; ++i)
      for (int r = 0; r < 4; ++r)
        acc[i][r] = 0.f;
    if constexpr (KIND == K_BF16) {
      const u32x4 ua = {a[0], a[1], a[2], a[3]}, ub = {b[0], b[1], b[2], b[3]};
      const bf16x8 va = __builtin_bit_cast(bf16x8, ua);
      const bf16x8 vb = __builtin_bit_cast(bf16x8, ub);
      for (int it = 0; it < iters; ++it)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, vb, acc[i], 0, 0, 0);
    } else {
      const i32x8 va = {(int)a[0], (int)a[1], (int)a[2], (int)a[3],
                        (int)a[4], (int)a[5], (int)a[6], (int)a[7]};
      const i32x8 vb = {(int)b[0], (int)b[1], (int)b[2], (int)b[3],
                        (int)b[4], (int)b[5], (int)b[6], (int)b[7]};
      for (int it = 0; it < iters; ++it)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              va, vb, acc[i], 0, 0, 0, 0, 0, 0);
    }
    for (int i = 0; i < 16; ++i)
      out += acc[i][0];
  }
  if (out == 12345.678f)
    sink[blockIdx.x * blockDim.x + threadIdx.x] = out;
}

// One contiguous chunk of UNROLL x 4 KiB per workgroup: all loads of a lane are
// issued before its first store.
template <int UNROLL>
__global__ __launch_bounds__(256) void copy_chunks(const u32x4 *src, u32x4 *dst) {
  const size_t base = (size_t)blockIdx.x * UNROLL * 256 + threadIdx.x;
  u32x4 v[UNROLL];
#pragma unroll
  for (int i = 0; i < UNROLL; ++i)
    v[i] = src[base + (size_t)i * 256];
#pragma unroll
  for (int i = 0; i < UNROLL; ++i)
    __builtin_nontemporal_store(v[i], dst + base + (size_t)i * 256);
}

template <int UNROLL>
__global__ __launch_bounds__(256) void read_chunks(const u32x4 *src,
                                                   uint32_t *sink) {
  const size_t base = (size_t)blockIdx.x * UNROLL * 256 + threadIdx.x;
  u32x4 v[UNROLL];
#pragma unroll
  for (int i = 0; i < UNROLL; ++i)
    v[i] = src[base + (size_t)i * 256];
  uint32_t acc = 0;
#pragma unroll
  for (int i = 0; i < UNROLL; ++i)
    acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
  if (acc == 0x12345678u)
    sink[0] = acc;
}

// Grid-stride copy of a whole buffer.
__global__ __launch_bounds__(256) void copy_kernel(const u32x4 *src, u32x4 *dst,
                                                   size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const u32x4 v = src[i];
    __builtin_nontemporal_store(v, dst + i);
  }
}

__global__ __launch_bounds__(256) void read_kernel(const u32x4 *src, size_t n,
                                                   uint32_t *sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  u32x4 acc = {0, 0, 0, 0};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const u32x4 v = src[i];
    acc.x ^= v.x, acc.y ^= v.y, acc.z ^= v.z, acc.w ^= v.w;
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u)
    sink[0] = acc.x;
}

// Launches `launch` repeatedly for about `seconds` (after as much warm-up)
// and returns the average milliseconds per launch over the timed part.
template <typename F> double time_launches(double seconds, F &&launch) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  launch();
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(e0));
  launch();
  CHECK(hipEventRecord(e1));
  CHECK(hipDeviceSynchronize());
  float one = 0;
  CHECK(hipEventElapsedTime(&one, e0, e1));
  int reps = (int)(seconds * 1e3 / (one > 1e-3f ? one : 1e-3f));
  reps = reps < 3 ? 3 : reps;
  for (int i = 0; i < reps; ++i) // warm-up: lets the clocks settle
    launch();
  CHECK(hipEventRecord(e0));
  for (int i = 0; i < reps; ++i)
    launch();
  CHECK(hipEventRecord(e1));
  CHECK(hipDeviceSynchronize());
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  CHECK(hipEventDestroy(e0));
  CHECK(hipEventDestroy(e1));
  return ms / reps;
}

template <int KIND>
double mfma_tops(double seconds, int random, int cus, float *sink) {
  const int iters = 2048;
  const double ms = time_launches(seconds, [&] {
    hipLaunchKernelGGL(mfma_loop<KIND>, dim3(cus), dim3(512), 0, 0, iters,
                       random, sink);
  });
  // per MFMA: 32 x 32 x K x 2 operations, K = 16 / 32 / 64
  const double k = KIND == K_BF16 ? 16 : KIND == K_I8 ? 32 : 64;
  const double ops = (double)cus * 8 * iters * 8 * 32 * 32 * k * 2;
  return ops / ms / 1e9;
}

template <int KIND>
double mfma16_tops(double seconds, int random, int cus, float *sink) {
  const int iters = 2048;
  const double ms = time_launches(seconds, [&] {
    hipLaunchKernelGGL(mfma16_loop<KIND>, dim3(cus), dim3(512), 0, 0, iters, random, sink);
  });
  // per MFMA: 16 x 16 x K x 2 operations, K = 32 / 64 / 128
  const double k = KIND == K_BF16 ? 32 : KIND == K_I8 ? 64 : 128;
  const double ops = (double)cus * 8 * iters * 16 * 16 * 16 * k * 2;
  return ops / ms / 1e9;
}

int main(int argc, char **argv) {
  const double seconds = argc > 1 ? atof(argv[1]) : 0.3;
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  float *sink;
  CHECK(hipMalloc(&sink, (size_t)cus * 512 * 4));
  printf("{\"device\": \"%s\", \"compute_units\": %d, \"seconds_per_measurement\": %.2f",
         prop.gcnArchName, cus, seconds);
  const char *names[3] = {"bf16", "int8", "fp8e4m3"};
  for (int random = 1; random >= 0; --random) {
    const double t[3] = {mfma_tops<K_BF16>(seconds, random, cus, sink),
                         mfma_tops<K_I8>(seconds, random, cus, sink),
                         mfma_tops<K_FP8>(seconds, random, cus, sink)};
    for (int i = 0; i < 3; ++i)
      printf(", \"mfma_%s_%s_operands_tops\": %.1f", names[i],
             random ? "random" : "constant", t[i]);
    const double u[3] = {mfma16_tops<K_BF16>(seconds, random, cus, sink),
                         mfma16_tops<K_I8>(seconds, random, cus, sink),
                         mfma16_tops<K_FP8>(seconds, random, cus, sink)};
    for (int i = 0; i < 3; ++i)
      printf(", \"mfma16x16_%s_%s_operands_tops\": %.1f", names[i],
             random ? "random" : "constant", u[i]);
  }
  // 1 GiB source and destination (far beyond the 256 MB Infinity Cache); a
  // launch moves one 64 MiB window (the size of the benchmark's bf16
  // 8192 x 4096 tensors), and consecutive launches walk the windows.
  const size_t bytes = 1024ull << 20, n = bytes / 16;
  const size_t win = 64ull << 20, nwin = bytes / win, wn = win / 16;
  u32x4 *src, *dst;
  CHECK(hipMalloc(&src, bytes));
  CHECK(hipMalloc(&dst, bytes));
  CHECK(hipMemset(src, 1, bytes));
  CHECK(hipMemset(dst, 0, bytes));
  uint32_t *s2 = (uint32_t *)sink;
  size_t turn = 0;
  auto window = [&] { return (turn++ % nwin) * wn; };
  {
    const double ms = time_launches(seconds, [&] {
      const size_t o = window();
      hipLaunchKernelGGL(copy_chunks<1>, dim3(wn / 256), dim3(256), 0, 0, src + o, dst + o);
    });
    printf(", \"copy_64MiB_windows_4KiB_chunks_tbs\": %.3f", 2.0 * win / ms / 1e9);
  }
  {
    const double ms = time_launches(seconds, [&] {
      const size_t o = window();
      hipLaunchKernelGGL(copy_chunks<4>, dim3(wn / 1024), dim3(256), 0, 0, src + o, dst + o);
    });
    printf(", \"copy_64MiB_windows_16KiB_chunks_tbs\": %.3f", 2.0 * win / ms / 1e9);
  }
  {
    const double ms = time_launches(seconds, [&] {
      const size_t o = window();
      hipLaunchKernelGGL(copy_chunks<8>, dim3(wn / 2048), dim3(256), 0, 0, src + o, dst + o);
    });
    printf(", \"copy_64MiB_windows_32KiB_chunks_tbs\": %.3f", 2.0 * win / ms / 1e9);
  }
  {
    const double ms = time_launches(seconds, [&] {
      hipLaunchKernelGGL(copy_kernel, dim3(cus * 16), dim3(256), 0, 0, src, dst, n);
    });
    printf(", \"copy_1GiB_grid_stride_tbs\": %.3f", 2.0 * bytes / ms / 1e9);
  }
  {
    const double ms = time_launches(seconds, [&] {
      const size_t o = window();
      hipLaunchKernelGGL(read_chunks<8>, dim3(wn / 2048), dim3(256), 0, 0, src + o, s2);
    });
    printf(", \"read_64MiB_windows_32KiB_chunks_tbs\": %.3f", (double)win / ms / 1e9);
  }
  {
    const double ms = time_launches(seconds, [&] {
      hipLaunchKernelGGL(read_kernel, dim3(cus * 16), dim3(256), 0, 0, src, n, s2);
    });
    printf(", \"read_1GiB_grid_stride_tbs\": %.3f", (double)bytes / ms / 1e9);
  }
  printf("}\n");
  return 0;
}
