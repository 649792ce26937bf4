// Execution plan: what replaces the reference's "emit torch-MLIR, run
// iree-compile, load the VMFB" pipeline (graph/graph.h:127-203, 407-416;
// backend/runtime.h:242-315).
//
// A plan is a list of steps, one C-ABI kernel call each.  The planner walks the
// validated node list in order and fuses `{conv | matmul | rmsnorm |
// layernorm} -> pointwise -> pointwise ...` chains into the producer's epilogue
// whenever the backend reports the fused descriptor as supported — the same
// fusions the reference expects from IREE (one dispatch for conv + bias +
// relu, tests/lit/test_conv_asm_emitter_nhwc_krsc_with_relu.cpp:103-104).
// Everything else becomes its own step, with virtual tensors between steps
// placed in the workspace.
//
// Kernel arguments are numbered like the reference's compiled function:
// non-virtual outputs sorted by name, then non-scalar inputs sorted by name
// (support/asm_emitter.h:444-492), so a plan serialised by one Graph loads
// into any identically built Graph.
#ifndef FUSILLI_PLAN_H
#define FUSILLI_PLAN_H

#include <cstring>
#include <map>
#include <set>
#include <span>
#include <string>
#include <unordered_map>
#include <vector>

#include "../fusilli_hip.h"
#include "backend.h"
#include "nodes.h"

namespace fusilli::plan {

enum class StepKind : uint32_t {
  Matmul = 1,
  Conv = 2,
  Sdpa = 3,
  Norm = 4,
  Reduce = 5,
  Pointwise = 6,
  ConvDGrad = 7,
  ConvWGrad = 8,
  BatchNorm = 9,
};

constexpr int kMaxSlots = 12;
constexpr int32_t kNoTensor = -1;

// Tensor slot encoding: >= 0 argument index; -1 none; <= -2 workspace tensor
// number (-slot - 2).
inline int32_t workspaceSlot(size_t index) {
  return -static_cast<int32_t>(index) - 2;
}

union StepDesc {
  fhip_matmul_desc matmul;
  fhip_conv_desc conv;
  fhip_sdpa_desc sdpa;
  fhip_norm_desc norm;
  fhip_reduce_desc reduce;
  fhip_pointwise_desc pointwise;
  fhip_batchnorm_desc batchnorm;
};

struct Step {
  uint32_t kind = 0;
  int32_t slot[kMaxSlots];
  StepDesc desc;
  // Steps are hashed and serialised as raw bytes, so every byte (padding
  // included) is defined: zero-filled here, and copied with memcpy.
  Step() {
    std::memset(static_cast<void *>(this), 0, sizeof(*this));
    for (int &s : slot)
      s = kNoTensor;
  }
  Step(const Step &o) { std::memcpy(static_cast<void *>(this), &o, sizeof(o)); }
  Step &operator=(const Step &o) {
    std::memcpy(static_cast<void *>(this), &o, sizeof(o));
    return *this;
  }
};

// Slot positions per step kind.
enum : int { kMmA = 0, kMmB = 1, kMmOut = 2, kMmEpi = 3 };
enum : int { kCvX = 0, kCvW = 1, kCvOut = 2, kCvEpi = 3 };
enum : int { kCbDY = 0, kCbIn = 1, kCbOut = 2, kCbScratch = 3 }; // conv gradients
enum : int { kSdQ = 0, kSdK = 1, kSdV = 2, kSdMask = 3, kSdO = 4 };
enum : int {
  kNmX = 0,
  kNmScale = 1,
  kNmBias = 2,
  kNmOut = 3,
  kNmMean = 4,
  kNmRstd = 5,
  kNmEpi = 6
};
enum : int {
  kBnX = 0,
  kBnScale = 1,
  kBnBias = 2,
  kBnMean = 3,
  kBnVar = 4,
  kBnY = 5,
  kBnSavedMean = 6,
  kBnSavedInvVar = 7
};
enum : int { kRdX = 0, kRdY = 1 };
enum : int { kPwIn0 = 0, kPwIn1 = 1, kPwIn2 = 2, kPwOut = 3 };

struct WorkspaceTensor {
  uint64_t offset = 0;
  uint64_t bytes = 0;
};

struct ArgInfo {
  uint64_t minBytes = 0; // bytes the kernels may touch
  uint32_t dtype = 0;
  uint32_t reserved = 0; // keeps the struct free of undefined padding
};

struct Plan {
  uint32_t backend = 0;
  uint64_t signature = 0;
  uint64_t workspaceBytes = 0;
  std::vector<Step> steps;
  std::vector<WorkspaceTensor> workspaceTensors;
  std::vector<ArgInfo> args;
};

constexpr char kMagic[8] = {'F', 'S', 'L', 'H', 'I', 'P', '0', '1'};
constexpr char kArch[8] = {'g', 'f', 'x', '9', '5', '0', 0, 0};

// ---- serialisation ----------------------------------------------------------
inline std::vector<uint8_t> serialize(const Plan &p) {
  std::vector<uint8_t> out;
  auto put = [&](const void *src, size_t n) {
    const auto *b = static_cast<const uint8_t *>(src);
    out.insert(out.end(), b, b + n);
  };
  auto putU64 = [&](uint64_t v) { put(&v, 8); };
  put(kMagic, 8);
  put(kArch, 8);
  putU64(FHIP_ABI_VERSION);
  putU64(sizeof(Step));
  putU64(p.backend);
  putU64(p.signature);
  putU64(p.workspaceBytes);
  putU64(p.steps.size());
  putU64(p.workspaceTensors.size());
  putU64(p.args.size());
  for (const Step &s : p.steps)
    put(&s, sizeof(Step));
  for (const WorkspaceTensor &w : p.workspaceTensors)
    put(&w, sizeof(w));
  for (const ArgInfo &a : p.args)
    put(&a, sizeof(a));
  // trailing checksum (FNV-1a over everything before it)
  uint64_t h = 1469598103934665603ull;
  for (uint8_t b : out)
    h = (h ^ b) * 1099511628211ull;
  putU64(h);
  return out;
}

inline ErrorOr<Plan> deserialize(std::span<const uint8_t> bytes) {
  constexpr size_t header = 8 + 8 + 8 * 8;
  FUSILLI_RETURN_ERROR_IF(bytes.size() < header + 8, ErrorCode::RuntimeFailure,
                          "Artifact is too small to be a compiled plan");
  FUSILLI_RETURN_ERROR_IF(std::memcmp(bytes.data(), kMagic, 8) != 0,
                          ErrorCode::RuntimeFailure,
                          "Artifact does not start with the plan magic");
  FUSILLI_RETURN_ERROR_IF(std::memcmp(bytes.data() + 8, kArch, 8) != 0,
                          ErrorCode::RuntimeFailure,
                          "Artifact was built for a different GPU architecture");
  uint64_t h = 1469598103934665603ull;
  for (size_t i = 0; i + 8 < bytes.size(); ++i)
    h = (h ^ bytes[i]) * 1099511628211ull;
  uint64_t stored;
  std::memcpy(&stored, bytes.data() + bytes.size() - 8, 8);
  FUSILLI_RETURN_ERROR_IF(h != stored, ErrorCode::RuntimeFailure,
                          "Artifact checksum mismatch (corrupted plan)");
  size_t pos = 16;
  auto getU64 = [&]() {
    uint64_t v;
    std::memcpy(&v, bytes.data() + pos, 8);
    pos += 8;
    return v;
  };
  const uint64_t abi = getU64(), stepSize = getU64();
  FUSILLI_RETURN_ERROR_IF(abi != FHIP_ABI_VERSION || stepSize != sizeof(Step),
                          ErrorCode::RuntimeFailure,
                          "Artifact was produced by an incompatible version");
  Plan p;
  p.backend = static_cast<uint32_t>(getU64());
  p.signature = getU64();
  p.workspaceBytes = getU64();
  const uint64_t nSteps = getU64(), nWs = getU64(), nArgs = getU64();
  // counts are bounded by the byte count first, so the products cannot wrap
  FUSILLI_RETURN_ERROR_IF(nSteps > bytes.size() / sizeof(Step) ||
                              nWs > bytes.size() / sizeof(WorkspaceTensor) ||
                              nArgs > bytes.size() / sizeof(ArgInfo),
                          ErrorCode::RuntimeFailure,
                          "Artifact length does not match its header");
  const uint64_t need = nSteps * sizeof(Step) + nWs * sizeof(WorkspaceTensor) +
                        nArgs * sizeof(ArgInfo);
  FUSILLI_RETURN_ERROR_IF(bytes.size() != header + need + 8,
                          ErrorCode::RuntimeFailure,
                          "Artifact length does not match its header");
  p.steps.resize(nSteps);
  p.workspaceTensors.resize(nWs);
  p.args.resize(nArgs);
  if (nSteps) {
    std::memcpy(static_cast<void *>(p.steps.data()), bytes.data() + pos,
                nSteps * sizeof(Step));
    pos += nSteps * sizeof(Step);
  }
  if (nWs) {
    std::memcpy(p.workspaceTensors.data(), bytes.data() + pos,
                nWs * sizeof(WorkspaceTensor));
    pos += nWs * sizeof(WorkspaceTensor);
  }
  if (nArgs)
    std::memcpy(p.args.data(), bytes.data() + pos, nArgs * sizeof(ArgInfo));
  return ok(std::move(p));
}

// ---- planner ----------------------------------------------------------------
inline ErrorOr<fhip_tensor_desc> toDesc(const TensorPtr &t) {
  fhip_tensor_desc d;
  std::memset(&d, 0, sizeof(d));
  FUSILLI_RETURN_ERROR_IF(t->getDim().size() > FHIP_MAX_RANK,
                          ErrorCode::NotImplemented,
                          "Tensor '" + t->getName() + "' has rank above " +
                              std::to_string(FHIP_MAX_RANK));
  // Dynamic dims are planned at the extents the TensorAttr holds: the graph
  // re-plans with the buffers' extents when they differ (Graph::execute).
  FUSILLI_RETURN_ERROR_IF(dataTypeSize(t->getDataType()) == 0,
                          ErrorCode::NotImplemented,
                          "Tensor '" + t->getName() + "' has element type " +
                              dataTypeAsm(t->getDataType()) +
                              ", which no kernel here executes");
  d.rank = static_cast<int32_t>(t->getDim().size());
  d.dtype = static_cast<int32_t>(t->getDataType());
  for (int i = 0; i < d.rank; ++i) {
    d.dim[i] = t->getDim()[i];
    d.stride[i] = t->getStride()[i];
  }
  return ok(d);
}

// Elements of storage a (dims, strides) view spans.
inline uint64_t storageExtent(const TensorPtr &t) {
  uint64_t e = 1;
  for (size_t i = 0; i < t->getDim().size(); ++i)
    e += static_cast<uint64_t>(t->getDim()[i] - 1) *
         static_cast<uint64_t>(t->getStride()[i]);
  return e;
}

class Planner {
public:
  Planner(const std::vector<std::shared_ptr<INode>> &nodes,
          const std::set<TensorPtr, TensorAttrSortByName> &inputsSorted,
          const std::set<TensorPtr, TensorAttrSortByName> &outputsSorted,
          Backend backend)
      : nodes_(nodes) {
    plan_.backend = static_cast<uint32_t>(backend);
    for (const auto &t : outputsSorted)
      if (!t->isVirtual())
        addArg(t);
    for (const auto &t : inputsSorted)
      if (!t->isScalar())
        addArg(t);
    for (const auto &n : nodes_)
      forEachInput(*n, [&](const TensorPtr &t) { consumers_[t.get()]++; });
  }

  ErrorOr<Plan> run() {
    size_t i = 0;
    while (i < nodes_.size()) {
      const INode &node = *nodes_[i];
      switch (node.getType()) {
      case INode::Type::Matmul: {
        FUSILLI_ASSIGN_OR_RETURN(size_t next, planMatmul(i));
        i = next;
        break;
      }
      case INode::Type::Convolution: {
        FUSILLI_ASSIGN_OR_RETURN(size_t next, planConv(i));
        i = next;
        break;
      }
      case INode::Type::WGrad:
      case INode::Type::DGrad:
        FUSILLI_CHECK_ERROR(planConvBackward(i));
        ++i;
        break;
      case INode::Type::BatchNorm:
        FUSILLI_CHECK_ERROR(planBatchNorm(i));
        ++i;
        break;
      case INode::Type::RmsNorm:
      case INode::Type::LayerNorm: {
        FUSILLI_ASSIGN_OR_RETURN(size_t next, planNorm(i));
        i = next;
        break;
      }
      case INode::Type::Sdpa:
        FUSILLI_CHECK_ERROR(planSdpa(i));
        ++i;
        break;
      case INode::Type::Reduction:
        FUSILLI_CHECK_ERROR(planReduction(i));
        ++i;
        break;
      case INode::Type::Pointwise:
        FUSILLI_CHECK_ERROR(planPointwise(i));
        ++i;
        break;
      default:
        return error(ErrorCode::NotImplemented,
                     "Node '" + node.getName() +
                         "' has a type this backend does not execute");
      }
    }
    plan_.workspaceBytes = workspaceCursor_;
    plan_.signature = signature();
    return ok(std::move(plan_));
  }

private:
  // -- bookkeeping ----------------------------------------------------------
  void addArg(const TensorPtr &t) {
    argIndex_[t.get()] = static_cast<int32_t>(plan_.args.size());
    ArgInfo a;
    a.minBytes = storageExtent(t) * dataTypeSize(t->getDataType());
    a.dtype = static_cast<uint32_t>(t->getDataType());
    plan_.args.push_back(a);
    argTensors_.push_back(t);
  }

  template <typename F> static void forEachInput(const INode &n, F &&f) {
    auto each = [&](const auto &attr) {
      for (const auto &kv : attr.inputs)
        if (kv.second)
          f(kv.second);
    };
    switch (n.getType()) {
    case INode::Type::Convolution:
      each(static_cast<const ConvFPropNode &>(n).convFPropAttr);
      break;
    case INode::Type::BatchNorm:
      each(static_cast<const BatchNormNode &>(n).batchnormAttr);
      break;
    case INode::Type::WGrad:
      each(static_cast<const ConvWGradNode &>(n).convWGradAttr);
      break;
    case INode::Type::DGrad:
      each(static_cast<const ConvDGradNode &>(n).convDGradAttr);
      break;
    case INode::Type::Matmul:
      each(static_cast<const MatmulNode &>(n).matmulAttr);
      break;
    case INode::Type::Pointwise:
      each(static_cast<const PointwiseNode &>(n).pointwiseAttr);
      break;
    case INode::Type::Reduction:
      each(static_cast<const ReductionNode &>(n).reductionAttr);
      break;
    case INode::Type::Sdpa:
      each(static_cast<const SdpaNode &>(n).sdpaAttr);
      break;
    case INode::Type::RmsNorm:
      each(static_cast<const RmsNormNode &>(n).rmsnormAttr);
      break;
    case INode::Type::LayerNorm:
      each(static_cast<const LayerNormNode &>(n).layernormAttr);
      break;
    default:
      break;
    }
  }

  // Slot of a tensor a step reads.
  ErrorOr<int32_t> readSlot(const TensorPtr &t) {
    FUSILLI_RETURN_ERROR_IF(t->isScalar(), ErrorCode::NotImplemented,
                            "Tensor '" + t->getName() +
                                "' is a scalar constant where a buffer operand "
                                "is required");
    if (auto it = argIndex_.find(t.get()); it != argIndex_.end())
      return ok(it->second);
    if (auto it = workspaceIndex_.find(t.get()); it != workspaceIndex_.end())
      return ok(workspaceSlot(it->second));
    return error(ErrorCode::InternalError,
                 "Tensor '" + t->getName() +
                     "' is read before any node produces it");
  }

  // Slot of a tensor a step writes: its argument, or fresh workspace when it
  // is virtual.
  ErrorOr<int32_t> writeSlot(const TensorPtr &t) {
    if (auto it = argIndex_.find(t.get()); it != argIndex_.end())
      return ok(it->second);
    FUSILLI_RETURN_ERROR_IF(!t->isVirtual(), ErrorCode::InternalError,
                            "Output tensor '" + t->getName() +
                                "' is neither an argument nor virtual");
    WorkspaceTensor w;
    w.offset = workspaceCursor_;
    w.bytes = storageExtent(t) * dataTypeSize(t->getDataType());
    workspaceCursor_ += (w.bytes + 255) / 256 * 256;
    workspaceIndex_[t.get()] = plan_.workspaceTensors.size();
    plan_.workspaceTensors.push_back(w);
    return ok(workspaceSlot(plan_.workspaceTensors.size() - 1));
  }

  static fhip_pointwise_params paramsOf(const PointwiseAttr &a) {
    fhip_pointwise_params p;
    p.elu_alpha = a.getEluAlpha();
    p.softplus_beta = a.getSoftplusBeta();
    p.softplus_threshold = a.getSoftplusThreshold();
    p.swish_beta = a.getSwishBeta();
    return p;
  }

  // -- epilogue fusion ---------------------------------------------------------
  // Tries to absorb pointwise nodes that directly follow node `i` and consume
  // `cur`.  `accept(epilogue, outTensor)` installs the candidate chain into the
  // producer's descriptor and asks the backend whether it is supported.
  template <typename Accept>
  ErrorOr<size_t> fuseFollowers(size_t i, TensorPtr &cur, fhip_epilogue &epi,
                                std::vector<TensorPtr> &operands,
                                Accept &&accept) {
    size_t j = i + 1;
    while (j < nodes_.size() && epi.count < FHIP_MAX_EPILOGUE &&
           nodes_[j]->getType() == INode::Type::Pointwise) {
      const auto &pw = static_cast<const PointwiseNode &>(*nodes_[j]).pointwiseAttr;
      const int arity = PointwiseAttr::requiredInputCount(pw.getMode());
      if (arity > 2)
        break;
      const TensorPtr in0 = pw.getIN_0(), in1 = pw.getIN_1(),
                      out = pw.getOUT_0();
      const bool curIsIn0 = in0 == cur, curIsIn1 = arity == 2 && in1 == cur;
      if (!curIsIn0 && !curIsIn1)
        break;
      if (curIsIn0 && curIsIn1)
        break; // x op x: keep it a separate node
      if (!cur->isVirtual() || consumers_[cur.get()] != 1)
        break;
      if (out->getDim() != cur->getDim())
        break;
      fhip_epilogue_op op;
      std::memset(&op, 0, sizeof(op));
      op.mode = static_cast<int32_t>(pw.getMode());
      op.acc_is_in1 = curIsIn1 ? 1 : 0;
      op.result_dtype = static_cast<int32_t>(out->getDataType());
      op.params = paramsOf(pw);
      op.operand_kind = FHIP_OPERAND_NONE;
      TensorPtr other;
      if (arity == 2) {
        other = curIsIn0 ? in1 : in0;
        if (other->isScalar()) {
          op.operand_kind = FHIP_OPERAND_SCALAR;
          op.scalar = static_cast<float>(scalarAsDouble(*other));
        } else {
          if (!argIndex_.count(other.get()))
            break; // produced by another node: not a plain operand
          op.operand_kind = FHIP_OPERAND_TENSOR;
          op.operand_index = static_cast<int32_t>(operands.size());
          auto d = toDesc(other);
          if (isError(d))
            break;
          op.operand = *d;
        }
      }
      fhip_epilogue trial;
      std::memcpy(&trial, &epi, sizeof(epi));
      std::memcpy(&trial.op[trial.count++], &op, sizeof(op));
      if (!accept(trial, out))
        break;
      std::memcpy(&epi, &trial, sizeof(epi));
      if (op.operand_kind == FHIP_OPERAND_TENSOR)
        operands.push_back(other);
      cur = out;
      ++j;
    }
    return ok(j);
  }

  // -- per-op planning ---------------------------------------------------------
  ErrorOr<size_t> planMatmul(size_t i) {
    const auto &attr = static_cast<const MatmulNode &>(*nodes_[i]).matmulAttr;
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::Matmul);
    fhip_matmul_desc &d = s.desc.matmul;
    FUSILLI_ASSIGN_OR_RETURN(d.a, toDesc(attr.getA()));
    FUSILLI_ASSIGN_OR_RETURN(d.b, toDesc(attr.getB()));
    FUSILLI_ASSIGN_OR_RETURN(d.c, toDesc(attr.getC()));
    d.out = d.c;
    d.out_dtype = d.c.dtype;
    TensorPtr cur = attr.getC();
    std::vector<TensorPtr> operands;
    FUSILLI_ASSIGN_OR_RETURN(
        size_t next,
        fuseFollowers(i, cur, d.epilogue, operands,
                      [&](const fhip_epilogue &e, const TensorPtr &out) {
                        fhip_matmul_desc t;
                        std::memcpy(&t, &d, sizeof(d));
                        std::memcpy(&t.epilogue, &e, sizeof(e));
                        auto od = toDesc(out);
                        if (isError(od))
                          return false;
                        std::memcpy(&t.out, &*od, sizeof(t.out));
                        t.out_dtype = od->dtype;
                        if (fhip_matmul_supported(&t) == 0)
                          return false;
                        std::memcpy(&d, &t, sizeof(d));
                        return true;
                      }));
    FUSILLI_RETURN_ERROR_IF(fhip_matmul_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "Matmul node '" + attr.getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kMmA], readSlot(attr.getA()));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kMmB], readSlot(attr.getB()));
    for (size_t k = 0; k < operands.size(); ++k) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kMmEpi + k], readSlot(operands[k]));
    }
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kMmOut], writeSlot(cur));
    plan_.steps.push_back(s);
    return ok(next);
  }

  ErrorOr<size_t> planConv(size_t i) {
    const auto &attr =
        static_cast<const ConvFPropNode &>(*nodes_[i]).convFPropAttr;
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::Conv);
    fhip_conv_desc &d = s.desc.conv;
    FUSILLI_ASSIGN_OR_RETURN(d.x, toDesc(attr.getX()));
    FUSILLI_ASSIGN_OR_RETURN(d.w, toDesc(attr.getW()));
    FUSILLI_ASSIGN_OR_RETURN(d.y, toDesc(attr.getY()));
    d.spatial_rank = static_cast<int32_t>(attr.getPadding().size());
    FUSILLI_RETURN_ERROR_IF(d.spatial_rank > 3, ErrorCode::NotImplemented,
                            "Convolutions above 3 spatial dims are not "
                            "supported");
    for (int k = 0; k < d.spatial_rank; ++k) {
      d.padding[k] = attr.getPadding()[k];
      d.stride[k] = attr.getStride()[k];
      d.dilation[k] = attr.getDilation()[k];
    }
    d.out = d.y;
    d.out_dtype = d.y.dtype;
    TensorPtr cur = attr.getY();
    std::vector<TensorPtr> operands;
    FUSILLI_ASSIGN_OR_RETURN(
        size_t next,
        fuseFollowers(i, cur, d.epilogue, operands,
                      [&](const fhip_epilogue &e, const TensorPtr &out) {
                        fhip_conv_desc t;
                        std::memcpy(&t, &d, sizeof(d));
                        std::memcpy(&t.epilogue, &e, sizeof(e));
                        auto od = toDesc(out);
                        if (isError(od))
                          return false;
                        std::memcpy(&t.out, &*od, sizeof(t.out));
                        t.out_dtype = od->dtype;
                        if (fhip_conv_fprop_supported(&t) == 0)
                          return false;
                        std::memcpy(&d, &t, sizeof(d));
                        return true;
                      }));
    FUSILLI_RETURN_ERROR_IF(fhip_conv_fprop_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "Conv node '" + attr.getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kCvX], readSlot(attr.getX()));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kCvW], readSlot(attr.getW()));
    for (size_t k = 0; k < operands.size(); ++k) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kCvEpi + k], readSlot(operands[k]));
    }
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kCvOut], writeSlot(cur));
    plan_.steps.push_back(s);
    return ok(next);
  }

  ErrorOr<size_t> planNorm(size_t i) {
    const bool layer = nodes_[i]->getType() == INode::Type::LayerNorm;
    TensorPtr x, scale, bias, y, eps, mean, rstd;
    std::string name;
    bool training = false;
    if (layer) {
      const auto &a =
          static_cast<const LayerNormNode &>(*nodes_[i]).layernormAttr;
      x = a.getX(), scale = a.getSCALE(), bias = a.getBIAS(), y = a.getY();
      eps = a.getEpsilon(), mean = a.getMEAN(), rstd = a.getINV_VARIANCE();
      training = a.getForwardPhase() == NormFwdPhase::TRAINING;
      name = a.getName();
    } else {
      const auto &a = static_cast<const RmsNormNode &>(*nodes_[i]).rmsnormAttr;
      x = a.getX(), scale = a.getSCALE(), y = a.getY(), eps = a.getEpsilon();
      name = a.getName();
    }
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::Norm);
    fhip_norm_desc &d = s.desc.norm;
    FUSILLI_ASSIGN_OR_RETURN(d.x, toDesc(x));
    if (scale) {
      FUSILLI_ASSIGN_OR_RETURN(d.scale, toDesc(scale));
    }
    if (bias) {
      FUSILLI_ASSIGN_OR_RETURN(d.bias, toDesc(bias));
    }
    FUSILLI_ASSIGN_OR_RETURN(d.y, toDesc(y));
    d.epsilon = static_cast<float>(scalarAsDouble(*eps));
    d.is_layernorm = layer ? 1 : 0;
    d.emit_stats = training ? 1 : 0;
    if (training) {
      FUSILLI_RETURN_ERROR_IF(mean->getDataType() != rstd->getDataType(),
                              ErrorCode::NotImplemented,
                              "LayerNorm MEAN and INV_VARIANCE must share an "
                              "element type");
      d.stats_dtype = static_cast<int32_t>(mean->getDataType());
    }
    d.out = d.y;
    d.out_dtype = d.y.dtype;
    TensorPtr cur = y;
    std::vector<TensorPtr> operands;
    FUSILLI_ASSIGN_OR_RETURN(
        size_t next,
        fuseFollowers(i, cur, d.epilogue, operands,
                      [&](const fhip_epilogue &e, const TensorPtr &out) {
                        fhip_norm_desc t;
                        std::memcpy(&t, &d, sizeof(d));
                        std::memcpy(&t.epilogue, &e, sizeof(e));
                        auto od = toDesc(out);
                        if (isError(od))
                          return false;
                        std::memcpy(&t.out, &*od, sizeof(t.out));
                        t.out_dtype = od->dtype;
                        if (fhip_norm_fwd_supported(&t) == 0)
                          return false;
                        std::memcpy(&d, &t, sizeof(d));
                        return true;
                      }));
    FUSILLI_RETURN_ERROR_IF(fhip_norm_fwd_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "Norm node '" + name +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmX], readSlot(x));
    if (scale) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmScale], readSlot(scale));
    }
    if (bias) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmBias], readSlot(bias));
    }
    for (size_t k = 0; k < operands.size(); ++k) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmEpi + k], readSlot(operands[k]));
    }
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmOut], writeSlot(cur));
    if (training) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmMean], writeSlot(mean));
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kNmRstd], writeSlot(rstd));
    }
    plan_.steps.push_back(s);
    return ok(next);
  }

  ErrorObject planSdpa(size_t i) {
    const auto &attr = static_cast<const SdpaNode &>(*nodes_[i]).sdpaAttr;
    FUSILLI_RETURN_ERROR_IF(attr.getDropout() != 0.0f,
                            ErrorCode::NotImplemented,
                            "SDPA dropout is not executable (only p = 0)");
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::Sdpa);
    fhip_sdpa_desc &d = s.desc.sdpa;
    FUSILLI_ASSIGN_OR_RETURN(d.q, toDesc(attr.getQ()));
    FUSILLI_ASSIGN_OR_RETURN(d.k, toDesc(attr.getK()));
    FUSILLI_ASSIGN_OR_RETURN(d.v, toDesc(attr.getV()));
    FUSILLI_ASSIGN_OR_RETURN(d.o, toDesc(attr.getO()));
    if (attr.getMASK()) {
      FUSILLI_ASSIGN_OR_RETURN(d.mask, toDesc(attr.getMASK()));
    }
    d.is_causal = attr.getIsCausal() ? 1 : 0;
    d.has_scale = attr.getScale().has_value() ? 1 : 0;
    d.scale = attr.getScale().value_or(0.0f);
    FUSILLI_RETURN_ERROR_IF(fhip_sdpa_fwd_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "SDPA node '" + attr.getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kSdQ], readSlot(attr.getQ()));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kSdK], readSlot(attr.getK()));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kSdV], readSlot(attr.getV()));
    if (attr.getMASK()) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kSdMask], readSlot(attr.getMASK()));
    }
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kSdO], writeSlot(attr.getO()));
    plan_.steps.push_back(s);
    return ok();
  }

  ErrorObject planReduction(size_t i) {
    const auto &attr =
        static_cast<const ReductionNode &>(*nodes_[i]).reductionAttr;
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::Reduce);
    fhip_reduce_desc &d = s.desc.reduce;
    FUSILLI_ASSIGN_OR_RETURN(d.x, toDesc(attr.getX()));
    FUSILLI_ASSIGN_OR_RETURN(d.y, toDesc(attr.getY()));
    d.mode = static_cast<int32_t>(attr.getMode());
    FUSILLI_RETURN_ERROR_IF(fhip_reduce_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "Reduction node '" + attr.getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kRdX], readSlot(attr.getX()));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kRdY], writeSlot(attr.getY()));
    plan_.steps.push_back(s);
    return ok();
  }

  ErrorObject planPointwise(size_t i) {
    const auto &attr =
        static_cast<const PointwiseNode &>(*nodes_[i]).pointwiseAttr;
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::Pointwise);
    fhip_pointwise_desc &d = s.desc.pointwise;
    d.mode = static_cast<int32_t>(attr.getMode());
    d.num_inputs = PointwiseAttr::requiredInputCount(attr.getMode());
    d.params = paramsOf(attr);
    const TensorPtr ins[3] = {attr.getIN_0(), attr.getIN_1(), attr.getIN_2()};
    for (int k = 0; k < d.num_inputs; ++k) {
      if (ins[k]->isScalar()) {
        d.in_is_scalar[k] = 1;
        d.in_scalar[k] = scalarAsDouble(*ins[k]);
      } else {
        FUSILLI_ASSIGN_OR_RETURN(d.in[k], toDesc(ins[k]));
        FUSILLI_ASSIGN_OR_RETURN(s.slot[kPwIn0 + k], readSlot(ins[k]));
      }
    }
    FUSILLI_ASSIGN_OR_RETURN(d.out, toDesc(attr.getOUT_0()));
    FUSILLI_RETURN_ERROR_IF(fhip_pointwise_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "Pointwise node '" + attr.getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kPwOut], writeSlot(attr.getOUT_0()));
    plan_.steps.push_back(s);
    return ok();
  }

  // FNV-1a over the plan's step descriptors, slots and argument table: two
  // graphs built the same way hash the same.
  uint64_t signature() const {
    uint64_t h = 1469598103934665603ull;
    auto mix = [&](const void *p, size_t n) {
      const auto *b = static_cast<const uint8_t *>(p);
      for (size_t k = 0; k < n; ++k)
        h = (h ^ b[k]) * 1099511628211ull;
    };
    mix(&plan_.backend, sizeof(plan_.backend));
    for (const Step &s : plan_.steps)
      mix(&s, sizeof(Step));
    for (const ArgInfo &a : plan_.args)
      mix(&a, sizeof(a));
    for (const auto &t : argTensors_)
      mix(t->getName().data(), t->getName().size());
    return h;
  }

  const std::vector<std::shared_ptr<INode>> &nodes_;
  Plan plan_;
  // Batch norm: one step, nothing fused.  MOMENTUM is validated by the node
  // and has no effect on the outputs.
  ErrorObject planBatchNorm(size_t i) {
    const auto &a = static_cast<const BatchNormNode &>(*nodes_[i]).batchnormAttr;
    const bool training = a.getForwardPhase() == NormFwdPhase::TRAINING;
    Step s;
    s.kind = static_cast<uint32_t>(StepKind::BatchNorm);
    fhip_batchnorm_desc &d = s.desc.batchnorm;
    FUSILLI_ASSIGN_OR_RETURN(d.x, toDesc(a.getX()));
    FUSILLI_ASSIGN_OR_RETURN(d.y, toDesc(a.getY()));
    d.training = training ? 1 : 0;
    d.epsilon = static_cast<float>(scalarAsDouble(*a.getEpsilon()));
    const int32_t f32 = static_cast<int32_t>(DataType::Float);
    d.scale_dtype = d.bias_dtype = d.running_dtype = d.stats_dtype = f32;
    if (const TensorPtr t = a.getSCALE()) {
      d.has_scale = 1;
      d.scale_dtype = static_cast<int32_t>(t->getDataType());
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnScale], readSlot(t));
    }
    if (const TensorPtr t = a.getBIAS()) {
      d.has_bias = 1;
      d.bias_dtype = static_cast<int32_t>(t->getDataType());
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnBias], readSlot(t));
    }
    if (!training) {
      const TensorPtr m = a.getMEAN(), v = a.getVAR();
      FUSILLI_RETURN_ERROR_IF(m->getDataType() != v->getDataType(),
                              ErrorCode::NotImplemented,
                              "BatchNorm MEAN and VAR must share an element "
                              "type");
      d.running_dtype = static_cast<int32_t>(m->getDataType());
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnMean], readSlot(m));
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnVar], readSlot(v));
    } else {
      const TensorPtr m = a.getSAVED_MEAN(), v = a.getSAVED_INV_VARIANCE();
      FUSILLI_RETURN_ERROR_IF(m->getDataType() != v->getDataType(),
                              ErrorCode::NotImplemented,
                              "BatchNorm SAVED_MEAN and SAVED_INV_VARIANCE must "
                              "share an element type");
      d.stats_dtype = static_cast<int32_t>(m->getDataType());
    }
    FUSILLI_RETURN_ERROR_IF(fhip_batchnorm_fwd_supported(&d) == 0,
                            ErrorCode::NotImplemented,
                            "BatchNorm node '" + a.getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnX], readSlot(a.getX()));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnY], writeSlot(a.getY()));
    if (training) {
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnSavedMean],
                               writeSlot(a.getSAVED_MEAN()));
      FUSILLI_ASSIGN_OR_RETURN(s.slot[kBnSavedInvVar],
                               writeSlot(a.getSAVED_INV_VARIANCE()));
    }
    plan_.steps.push_back(s);
    return ok();
  }

  // Conv gradients: one step each, nothing fused (the descriptor names the
  // forward problem: x = X / DX, w = W / DW, y = DY).
  ErrorObject planConvBackward(size_t i) {
    const bool dgrad = nodes_[i]->getType() == INode::Type::DGrad;
    TensorPtr x, w, dy;
    const std::vector<int64_t> *pad, *str, *dil;
    if (dgrad) {
      const auto &a = static_cast<const ConvDGradNode &>(*nodes_[i]).convDGradAttr;
      x = a.getDX(), w = a.getW(), dy = a.getDY();
      pad = &a.getPadding(), str = &a.getStride(), dil = &a.getDilation();
    } else {
      const auto &a = static_cast<const ConvWGradNode &>(*nodes_[i]).convWGradAttr;
      x = a.getX(), w = a.getDW(), dy = a.getDY();
      pad = &a.getPadding(), str = &a.getStride(), dil = &a.getDilation();
    }
    Step s;
    s.kind = static_cast<uint32_t>(dgrad ? StepKind::ConvDGrad
                                         : StepKind::ConvWGrad);
    fhip_conv_desc &d = s.desc.conv;
    FUSILLI_ASSIGN_OR_RETURN(d.x, toDesc(x));
    FUSILLI_ASSIGN_OR_RETURN(d.w, toDesc(w));
    FUSILLI_ASSIGN_OR_RETURN(d.y, toDesc(dy));
    d.spatial_rank = static_cast<int32_t>(pad->size());
    FUSILLI_RETURN_ERROR_IF(d.spatial_rank > 3, ErrorCode::NotImplemented,
                            "Convolutions above 3 spatial dims are not "
                            "supported");
    for (int k = 0; k < d.spatial_rank; ++k) {
      d.padding[k] = (*pad)[k];
      d.stride[k] = (*str)[k];
      d.dilation[k] = (*dil)[k];
    }
    const int supported =
        dgrad ? fhip_conv_dgrad_supported(&d) : fhip_conv_wgrad_supported(&d);
    FUSILLI_RETURN_ERROR_IF(supported == 0, ErrorCode::NotImplemented,
                            "Conv gradient node '" + nodes_[i]->getName() +
                                "' is not executable by this backend: " +
                                fhip_last_error(nullptr));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kCbDY], readSlot(dy));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kCbIn], readSlot(dgrad ? w : x));
    FUSILLI_ASSIGN_OR_RETURN(s.slot[kCbOut], writeSlot(dgrad ? x : w));
    // kernel scratch (the data gradient's mirrored filter): a workspace
    // region of its own, like a virtual tensor
    size_t scratch = 0;
    const int rc = dgrad ? fhip_conv_dgrad_workspace_size(&d, &scratch)
                         : fhip_conv_wgrad_workspace_size(&d, &scratch);
    FUSILLI_RETURN_ERROR_IF(rc != 0, ErrorCode::InternalError,
                            std::string(fhip_last_error(nullptr)));
    if (scratch > 0) {
      WorkspaceTensor t;
      t.offset = workspaceCursor_;
      t.bytes = scratch;
      workspaceCursor_ += (t.bytes + 255) / 256 * 256;
      plan_.workspaceTensors.push_back(t);
      s.slot[kCbScratch] = workspaceSlot(plan_.workspaceTensors.size() - 1);
    }
    plan_.steps.push_back(s);
    return ok();
  }

  std::unordered_map<const TensorAttr *, int32_t> argIndex_;
  std::vector<TensorPtr> argTensors_;
  std::unordered_map<const TensorAttr *, size_t> workspaceIndex_;
  std::unordered_map<const TensorAttr *, int> consumers_;
  uint64_t workspaceCursor_ = 0;
};

// ---- execution ----------------------------------------------------------------
// Runs every step of `p` on `ctx`.  `args[i]` is the device pointer of
// argument i; `workspace` backs the plan's workspace tensors.
inline ErrorObject execute(fhip_ctx *ctx, const Plan &p,
                           const std::vector<void *> &args, void *workspace) {
  auto ptr = [&](int32_t slot) -> void * {
    if (slot >= 0)
      return args[static_cast<size_t>(slot)];
    if (slot == kNoTensor)
      return nullptr;
    const WorkspaceTensor &w =
        p.workspaceTensors[static_cast<size_t>(-slot - 2)];
    return static_cast<char *>(workspace) + w.offset;
  };
  auto bytesOf = [&](int32_t slot) -> size_t { // of a workspace region
    return slot <= -2
               ? p.workspaceTensors[static_cast<size_t>(-slot - 2)].bytes
               : 0;
  };
  for (const Step &s : p.steps) {
    int rc = 0;
    const void *epi[FHIP_MAX_EPILOGUE] = {nullptr, nullptr, nullptr, nullptr};
    switch (static_cast<StepKind>(s.kind)) {
    case StepKind::Matmul:
      for (int k = 0; k < FHIP_MAX_EPILOGUE; ++k)
        epi[k] = ptr(s.slot[kMmEpi + k]);
      rc = fhip_matmul(ctx, &s.desc.matmul, ptr(s.slot[kMmA]),
                       ptr(s.slot[kMmB]), epi, ptr(s.slot[kMmOut]), nullptr, 0);
      break;
    case StepKind::Conv:
      for (int k = 0; k < FHIP_MAX_EPILOGUE; ++k)
        epi[k] = ptr(s.slot[kCvEpi + k]);
      rc = fhip_conv_fprop(ctx, &s.desc.conv, ptr(s.slot[kCvX]),
                           ptr(s.slot[kCvW]), epi, ptr(s.slot[kCvOut]), nullptr,
                           0);
      break;
    case StepKind::ConvDGrad:
      rc = fhip_conv_dgrad(ctx, &s.desc.conv, ptr(s.slot[kCbDY]),
                           ptr(s.slot[kCbIn]), ptr(s.slot[kCbOut]),
                           ptr(s.slot[kCbScratch]), bytesOf(s.slot[kCbScratch]));
      break;
    case StepKind::ConvWGrad:
      rc = fhip_conv_wgrad(ctx, &s.desc.conv, ptr(s.slot[kCbDY]),
                           ptr(s.slot[kCbIn]), ptr(s.slot[kCbOut]),
                           ptr(s.slot[kCbScratch]), bytesOf(s.slot[kCbScratch]));
      break;
    case StepKind::BatchNorm:
      rc = fhip_batchnorm_fwd(ctx, &s.desc.batchnorm, ptr(s.slot[kBnX]),
                              ptr(s.slot[kBnScale]), ptr(s.slot[kBnBias]),
                              ptr(s.slot[kBnMean]), ptr(s.slot[kBnVar]),
                              ptr(s.slot[kBnY]), ptr(s.slot[kBnSavedMean]),
                              ptr(s.slot[kBnSavedInvVar]), nullptr, 0);
      break;
    case StepKind::Sdpa:
      rc = fhip_sdpa_fwd(ctx, &s.desc.sdpa, ptr(s.slot[kSdQ]),
                         ptr(s.slot[kSdK]), ptr(s.slot[kSdV]),
                         ptr(s.slot[kSdMask]), ptr(s.slot[kSdO]), nullptr, 0);
      break;
    case StepKind::Norm:
      for (int k = 0; k < FHIP_MAX_EPILOGUE; ++k)
        epi[k] = ptr(s.slot[kNmEpi + k]);
      rc = fhip_norm_fwd(ctx, &s.desc.norm, ptr(s.slot[kNmX]),
                         ptr(s.slot[kNmScale]), ptr(s.slot[kNmBias]), epi,
                         ptr(s.slot[kNmOut]), ptr(s.slot[kNmMean]),
                         ptr(s.slot[kNmRstd]), nullptr, 0);
      break;
    case StepKind::Reduce:
      rc = fhip_reduce(ctx, &s.desc.reduce, ptr(s.slot[kRdX]),
                       ptr(s.slot[kRdY]), nullptr, 0);
      break;
    case StepKind::Pointwise:
      rc = fhip_pointwise(ctx, &s.desc.pointwise, ptr(s.slot[kPwIn0]),
                          ptr(s.slot[kPwIn1]), ptr(s.slot[kPwIn2]),
                          ptr(s.slot[kPwOut]));
      break;
    default:
      return error(ErrorCode::InternalError, "Plan holds an unknown step kind");
    }
    FUSILLI_RETURN_ERROR_IF(rc != 0, ErrorCode::RuntimeFailure,
                            std::string(fhip_last_error(ctx)));
  }
  return ok();
}

} // namespace fusilli::plan

#endif // FUSILLI_PLAN_H
