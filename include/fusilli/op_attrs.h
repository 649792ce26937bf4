// Operation attributes: named input/output tensor slots plus op parameters.
//
// Same classes, slot names and setters/getters as the reference's
// attributes/{attributes,conv,matmul,pointwise,reduction,sdpa,rmsnorm,
// layernorm}_attributes.h; the slot accessors are generated from one list per
// class instead of per-slot macros.
#ifndef FUSILLI_OP_ATTRS_H
#define FUSILLI_OP_ATTRS_H

#include <cstdint>
#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

#include "tensor_attr.h"

namespace fusilli {

using TensorPtr = std::shared_ptr<TensorAttr>;

// Shared behaviour of every attribute class (attributes/attributes.h:30-115).
template <typename Derived> class AttributesCRTP {
public:
  DataType computeDataType = DataType::NotSet;

  const std::string &getName() const { return name_; }
  Derived &setName(const std::string &n) {
    name_ = n;
    return self();
  }
  Derived &setComputeDataType(DataType t) {
    computeDataType = t;
    return self();
  }

  template <typename Key> Derived &setInput(Key k, const TensorPtr &t) {
    self().inputs[k] = t;
    return self();
  }
  template <typename Key> Derived &setOutput(Key k, const TensorPtr &t) {
    self().outputs[k] = t;
    return self();
  }
  template <typename Key> TensorPtr getInput(Key k) const {
    auto it = self().inputs.find(k);
    return it == self().inputs.end() ? nullptr : it->second;
  }
  template <typename Key> TensorPtr getOutput(Key k) const {
    auto it = self().outputs.find(k);
    return it == self().outputs.end() ? nullptr : it->second;
  }

  // Unset compute dtype <- context; every attached tensor fills its own dtype.
  void fillFromContext(const Context &ctx) {
    if (computeDataType == DataType::NotSet)
      computeDataType = ctx.getComputeDataType();
    for (auto &kv : self().inputs)
      if (kv.second)
        kv.second->fillFromContext(ctx);
    for (auto &kv : self().outputs)
      if (kv.second)
        kv.second->fillFromContext(ctx);
  }

private:
  Derived &self() { return static_cast<Derived &>(*this); }
  const Derived &self() const { return static_cast<const Derived &>(*this); }
  std::string name_;
};

#define FUSILLI_IN_SLOT(CLASS, NAME)                                           \
  CLASS &set##NAME(const TensorPtr &t) { return setInput(InputNames::NAME, t); } \
  TensorPtr get##NAME() const { return getInput(InputNames::NAME); }
#define FUSILLI_OUT_SLOT(CLASS, NAME)                                          \
  CLASS &set##NAME(const TensorPtr &t) {                                       \
    return setOutput(OutputNames::NAME, t);                                    \
  }                                                                            \
  TensorPtr get##NAME() const { return getOutput(OutputNames::NAME); }
#define FUSILLI_SLOT_MAPS                                                      \
  std::unordered_map<InputNames, TensorPtr> inputs;                            \
  std::unordered_map<OutputNames, TensorPtr> outputs;

enum class NormFwdPhase : uint8_t { NOT_SET, TRAINING, INFERENCE };

// ---- convolution (attributes/conv_attributes.h) -------------------------------
// Padding / stride / dilation setters and getters shared by the three
// convolution attribute classes.
#define FUSILLI_CONV_GEOMETRY(CLASS)                                           \
  CLASS &setPadding(const std::vector<int64_t> &v) {                           \
    padding_ = v;                                                              \
    return *this;                                                              \
  }                                                                            \
  CLASS &setStride(const std::vector<int64_t> &v) {                            \
    stride_ = v;                                                               \
    return *this;                                                              \
  }                                                                            \
  CLASS &setDilation(const std::vector<int64_t> &v) {                          \
    dilation_ = v;                                                             \
    return *this;                                                              \
  }                                                                            \
  template <Int64Range R> CLASS &setPadding(R &&v) {                           \
    padding_.assign(v.begin(), v.end());                                       \
    return *this;                                                              \
  }                                                                            \
  template <Int64Range R> CLASS &setStride(R &&v) {                            \
    stride_.assign(v.begin(), v.end());                                        \
    return *this;                                                              \
  }                                                                            \
  template <Int64Range R> CLASS &setDilation(R &&v) {                          \
    dilation_.assign(v.begin(), v.end());                                      \
    return *this;                                                              \
  }                                                                            \
  const std::vector<int64_t> &getPadding() const { return padding_; }          \
  const std::vector<int64_t> &getStride() const { return stride_; }            \
  const std::vector<int64_t> &getDilation() const { return dilation_; }        \
                                                                               \
private:                                                                       \
  std::vector<int64_t> padding_, stride_, dilation_;                           \
                                                                               \
public:

// forward (conv_attributes.h:20-84)
class ConvFPropAttr : public AttributesCRTP<ConvFPropAttr> {
public:
  enum class InputNames : uint8_t { X, W };
  enum class OutputNames : uint8_t { Y };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(ConvFPropAttr, X)
  FUSILLI_IN_SLOT(ConvFPropAttr, W)
  FUSILLI_OUT_SLOT(ConvFPropAttr, Y)
  FUSILLI_CONV_GEOMETRY(ConvFPropAttr)
};

// weight gradient (conv_attributes.h:86-139)
class ConvWGradAttr : public AttributesCRTP<ConvWGradAttr> {
public:
  enum class InputNames : uint8_t { DY, X };
  enum class OutputNames : uint8_t { DW };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(ConvWGradAttr, DY)
  FUSILLI_IN_SLOT(ConvWGradAttr, X)
  FUSILLI_OUT_SLOT(ConvWGradAttr, DW)
  FUSILLI_CONV_GEOMETRY(ConvWGradAttr)
};

// data gradient (conv_attributes.h:141-191)
class ConvDGradAttr : public AttributesCRTP<ConvDGradAttr> {
public:
  enum class InputNames : uint8_t { DY, W };
  enum class OutputNames : uint8_t { DX };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(ConvDGradAttr, DY)
  FUSILLI_IN_SLOT(ConvDGradAttr, W)
  FUSILLI_OUT_SLOT(ConvDGradAttr, DX)
  FUSILLI_CONV_GEOMETRY(ConvDGradAttr)
};

// ---- matmul (attributes/matmul_attributes.h) --------------------------------
class MatmulAttr : public AttributesCRTP<MatmulAttr> {
public:
  enum class InputNames : uint8_t { A, B };
  enum class OutputNames : uint8_t { C };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(MatmulAttr, A)
  FUSILLI_IN_SLOT(MatmulAttr, B)
  FUSILLI_OUT_SLOT(MatmulAttr, C)
};

// ---- pointwise (attributes/pointwise_attributes.h) --------------------------
class PointwiseAttr : public AttributesCRTP<PointwiseAttr> {
public:
  enum class InputNames : uint8_t { IN_0, IN_1, IN_2 };
  enum class OutputNames : uint8_t { OUT_0 };

  // Enumerator values are the C ABI's fhip_pointwise_mode.
  enum class Mode : uint8_t {
    NOT_SET,
    ABS,
    ADD,
    ADD_SQUARE,
    BINARY_SELECT,
    CEIL,
    CMP_EQ,
    CMP_GE,
    CMP_GT,
    CMP_LE,
    CMP_LT,
    CMP_NEQ,
    DIV,
    ELU_FWD,
    ERF,
    EXP,
    FLOOR,
    GELU_APPROX_TANH_BWD,
    GELU_APPROX_TANH_FWD,
    GELU_BWD,
    GELU_FWD,
    IDENTITY,
    LOG,
    LOGICAL_AND,
    LOGICAL_NOT,
    LOGICAL_OR,
    MAX_OP,
    MIN_OP,
    MUL,
    NEG,
    RECIPROCAL,
    RELU_BWD,
    RELU_FWD,
    RSQRT,
    SIGMOID_FWD,
    SIN,
    SOFTPLUS_FWD,
    SQRT,
    SUB,
    SWISH_BWD,
    SWISH_FWD,
    TAN,
    TANH_BWD,
    TANH_FWD,
  };

  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(PointwiseAttr, IN_0)
  FUSILLI_IN_SLOT(PointwiseAttr, IN_1)
  FUSILLI_IN_SLOT(PointwiseAttr, IN_2)
  FUSILLI_OUT_SLOT(PointwiseAttr, OUT_0)

  PointwiseAttr &setMode(Mode m) {
    mode_ = m;
    return *this;
  }
  PointwiseAttr &setEluAlpha(float v) {
    eluAlpha_ = v;
    return *this;
  }
  PointwiseAttr &setSoftplusBeta(float v) {
    softplusBeta_ = v;
    return *this;
  }
  PointwiseAttr &setSoftplusThreshold(float v) {
    softplusThreshold_ = v;
    return *this;
  }
  PointwiseAttr &setSwishBeta(float v) {
    swishBeta_ = v;
    return *this;
  }
  Mode getMode() const { return mode_; }
  float getEluAlpha() const { return eluAlpha_; }
  float getSoftplusBeta() const { return softplusBeta_; }
  float getSoftplusThreshold() const { return softplusThreshold_; }
  float getSwishBeta() const { return swishBeta_; }

  static const char *modeName(Mode m) {
    static const char *const names[] = {
        "NOT_SET", "ABS", "ADD", "ADD_SQUARE", "BINARY_SELECT", "CEIL",
        "CMP_EQ", "CMP_GE", "CMP_GT", "CMP_LE", "CMP_LT", "CMP_NEQ", "DIV",
        "ELU_FWD", "ERF", "EXP", "FLOOR", "GELU_APPROX_TANH_BWD",
        "GELU_APPROX_TANH_FWD", "GELU_BWD", "GELU_FWD", "IDENTITY", "LOG",
        "LOGICAL_AND", "LOGICAL_NOT", "LOGICAL_OR", "MAX_OP", "MIN_OP", "MUL",
        "NEG", "RECIPROCAL", "RELU_BWD", "RELU_FWD", "RSQRT", "SIGMOID_FWD",
        "SIN", "SOFTPLUS_FWD", "SQRT", "SUB", "SWISH_BWD", "SWISH_FWD", "TAN",
        "TANH_BWD", "TANH_FWD"};
    return names[static_cast<size_t>(m)];
  }

  // Number of tensor inputs a mode takes (pointwise_attributes.h:157-201).
  static int requiredInputCount(Mode m) {
    switch (m) {
    case Mode::BINARY_SELECT:
      return 3;
    case Mode::ADD:
    case Mode::ADD_SQUARE:
    case Mode::CMP_EQ:
    case Mode::CMP_GE:
    case Mode::CMP_GT:
    case Mode::CMP_LE:
    case Mode::CMP_LT:
    case Mode::CMP_NEQ:
    case Mode::DIV:
    case Mode::GELU_APPROX_TANH_BWD:
    case Mode::GELU_BWD:
    case Mode::LOGICAL_AND:
    case Mode::LOGICAL_OR:
    case Mode::MAX_OP:
    case Mode::MIN_OP:
    case Mode::MUL:
    case Mode::RELU_BWD:
    case Mode::SUB:
    case Mode::SWISH_BWD:
    case Mode::TANH_BWD:
      return 2;
    default:
      return 1;
    }
  }

  // Compare and logical modes always produce Boolean
  // (node/pointwise_node.h:31-42).
  static bool forcesBooleanOutput(Mode m) {
    switch (m) {
    case Mode::CMP_EQ:
    case Mode::CMP_NEQ:
    case Mode::CMP_LT:
    case Mode::CMP_LE:
    case Mode::CMP_GT:
    case Mode::CMP_GE:
    case Mode::LOGICAL_AND:
    case Mode::LOGICAL_NOT:
    case Mode::LOGICAL_OR:
      return true;
    default:
      return false;
    }
  }

private:
  Mode mode_ = Mode::NOT_SET;
  float eluAlpha_ = 1.0f;
  float softplusBeta_ = 1.0f;
  float softplusThreshold_ = 20.0f;
  float swishBeta_ = 1.0f;
};

// ---- reduction (attributes/reduction_attributes.h) --------------------------
class ReductionAttr : public AttributesCRTP<ReductionAttr> {
public:
  enum class InputNames : uint8_t { X };
  enum class OutputNames : uint8_t { Y };
  // Enumerator values are the C ABI's fhip_reduction_mode.
  enum class Mode : uint8_t {
    NOT_SET,
    ADD,
    SUM,
    MUL,
    MIN,
    MAX,
    AMAX,
    AVG,
    NORM1,
    NORM2,
    MUL_NO_ZEROS,
  };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(ReductionAttr, X)
  FUSILLI_OUT_SLOT(ReductionAttr, Y)

  ReductionAttr &setMode(Mode m) {
    mode_ = m;
    return *this;
  }
  Mode getMode() const { return mode_; }
  static const char *modeName(Mode m) {
    static const char *const names[] = {"NOT_SET", "ADD",   "SUM",   "MUL",
                                        "MIN",     "MAX",   "AMAX",  "AVG",
                                        "NORM1",   "NORM2", "MUL_NO_ZEROS"};
    return names[static_cast<size_t>(m)];
  }

private:
  Mode mode_ = Mode::NOT_SET;
};

// ---- SDPA (attributes/sdpa_attributes.h) ------------------------------------
class SdpaAttr : public AttributesCRTP<SdpaAttr> {
public:
  enum class InputNames : uint8_t { Q, K, V, MASK };
  enum class OutputNames : uint8_t { O };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(SdpaAttr, Q)
  FUSILLI_IN_SLOT(SdpaAttr, K)
  FUSILLI_IN_SLOT(SdpaAttr, V)
  FUSILLI_IN_SLOT(SdpaAttr, MASK)
  FUSILLI_OUT_SLOT(SdpaAttr, O)

  SdpaAttr &setDropout(float p) {
    dropout_ = p;
    return *this;
  }
  SdpaAttr &setIsCausal(bool v) {
    isCausal_ = v;
    return *this;
  }
  SdpaAttr &setScale(std::optional<float> s) {
    scale_ = s;
    return *this;
  }
  SdpaAttr &setEnableGqa(bool v) {
    enableGqa_ = v;
    return *this;
  }
  float getDropout() const { return dropout_; }
  bool getIsCausal() const { return isCausal_; }
  std::optional<float> getScale() const { return scale_; }
  bool getEnableGqa() const { return enableGqa_; }

private:
  float dropout_ = 0.0f;
  bool isCausal_ = false;
  std::optional<float> scale_;
  bool enableGqa_ = false;
};

// ---- RMSNorm (attributes/rmsnorm_attributes.h) ------------------------------
class RmsnormAttr : public AttributesCRTP<RmsnormAttr> {
public:
  enum class InputNames : uint8_t { X, SCALE, EPSILON };
  enum class OutputNames : uint8_t { Y, INV_RMS };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(RmsnormAttr, X)
  FUSILLI_IN_SLOT(RmsnormAttr, SCALE)
  FUSILLI_OUT_SLOT(RmsnormAttr, Y)
  FUSILLI_OUT_SLOT(RmsnormAttr, INV_RMS)

  RmsnormAttr &setEpsilon(const TensorPtr &eps) {
    return setInput(InputNames::EPSILON, eps);
  }
  TensorPtr getEpsilon() const { return getInput(InputNames::EPSILON); }
  RmsnormAttr &setForwardPhase(NormFwdPhase p) {
    phase_ = p;
    return *this;
  }
  NormFwdPhase getForwardPhase() const { return phase_; }

private:
  NormFwdPhase phase_ = NormFwdPhase::NOT_SET;
};

// ---- LayerNorm (attributes/layernorm_attributes.h) --------------------------
class LayernormAttr : public AttributesCRTP<LayernormAttr> {
public:
  enum class InputNames : uint8_t { X, SCALE, BIAS, EPSILON };
  enum class OutputNames : uint8_t { Y, MEAN, INV_VARIANCE };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(LayernormAttr, X)
  FUSILLI_IN_SLOT(LayernormAttr, SCALE)
  FUSILLI_IN_SLOT(LayernormAttr, BIAS)
  FUSILLI_OUT_SLOT(LayernormAttr, Y)
  FUSILLI_OUT_SLOT(LayernormAttr, MEAN)
  FUSILLI_OUT_SLOT(LayernormAttr, INV_VARIANCE)

  LayernormAttr &setEpsilon(const TensorPtr &eps) {
    return setInput(InputNames::EPSILON, eps);
  }
  TensorPtr getEpsilon() const { return getInput(InputNames::EPSILON); }
  LayernormAttr &setForwardPhase(NormFwdPhase p) {
    phase_ = p;
    return *this;
  }
  NormFwdPhase getForwardPhase() const { return phase_; }

private:
  NormFwdPhase phase_ = NormFwdPhase::NOT_SET;
};

// ---- batch norm (attributes/batchnorm_attributes.h) ------------------------------
class BatchnormAttr : public AttributesCRTP<BatchnormAttr> {
public:
  enum class InputNames : uint8_t { X, SCALE, BIAS, MEAN, VAR, EPSILON, MOMENTUM };
  enum class OutputNames : uint8_t { Y, SAVED_MEAN, SAVED_INV_VARIANCE };
  FUSILLI_SLOT_MAPS
  FUSILLI_IN_SLOT(BatchnormAttr, X)
  FUSILLI_IN_SLOT(BatchnormAttr, SCALE)
  FUSILLI_IN_SLOT(BatchnormAttr, BIAS)
  FUSILLI_IN_SLOT(BatchnormAttr, MEAN)
  FUSILLI_IN_SLOT(BatchnormAttr, VAR)
  FUSILLI_OUT_SLOT(BatchnormAttr, Y)
  FUSILLI_OUT_SLOT(BatchnormAttr, SAVED_MEAN)
  FUSILLI_OUT_SLOT(BatchnormAttr, SAVED_INV_VARIANCE)

  BatchnormAttr &setEpsilon(const TensorPtr &eps) {
    return setInput(InputNames::EPSILON, eps);
  }
  TensorPtr getEpsilon() const { return getInput(InputNames::EPSILON); }
  BatchnormAttr &setMomentum(const TensorPtr &m) {
    return setInput(InputNames::MOMENTUM, m);
  }
  TensorPtr getMomentum() const { return getInput(InputNames::MOMENTUM); }
  BatchnormAttr &setForwardPhase(NormFwdPhase p) {
    phase_ = p;
    return *this;
  }
  NormFwdPhase getForwardPhase() const { return phase_; }

private:
  NormFwdPhase phase_ = NormFwdPhase::NOT_SET;
};

#undef FUSILLI_IN_SLOT
#undef FUSILLI_OUT_SLOT
#undef FUSILLI_SLOT_MAPS

} // namespace fusilli

#endif // FUSILLI_OP_ATTRS_H
