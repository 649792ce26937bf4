// Graph nodes: one class per operation, each with the reference's three-phase
// validation (preValidateNode -> inferPropertiesNode -> postValidateNode) and
// the same error codes and messages (reference node/{node,conv_node,
// matmul_node,pointwise_node,reduction_node,sdpa_node,rmsnorm_node,
// layernorm_node,norm_utils}.h).  There is no MLIR emission here: a planner
// (plan.h) reads the validated nodes instead.
#ifndef FUSILLI_NODES_H
#define FUSILLI_NODES_H

#include <memory>
#include <string>
#include <unordered_set>
#include <vector>

#include "op_attrs.h"

namespace fusilli {

class INode {
public:
  enum class Type : uint8_t {
    Composite,
    Convolution,
    Pointwise,
    WGrad,
    DGrad,
    LayerNorm,
    BatchNorm,
    RmsNorm,
    Matmul,
    Reduction,
    Custom,
    Sdpa,
  };

  explicit INode(const Context &ctx) : context(ctx) {}
  virtual ~INode() = default;
  virtual const std::string &getName() const = 0;
  virtual Type getType() const = 0;

  Context context;

protected:
  std::vector<std::shared_ptr<INode>> subNodes_;

  virtual ErrorObject preValidateNode() const { return ok(); }
  virtual ErrorObject inferPropertiesNode() = 0;
  virtual ErrorObject postValidateNode() const { return ok(); }

  // pre -> infer -> children -> post (node/node.h:84-91).
  ErrorObject validateSubtree() {
    FUSILLI_CHECK_ERROR(preValidateNode());
    FUSILLI_CHECK_ERROR(inferPropertiesNode());
    for (const auto &child : subNodes_)
      FUSILLI_CHECK_ERROR(child->validateSubtree());
    FUSILLI_CHECK_ERROR(postValidateNode());
    return ok();
  }

  ErrorObject
  checkNodeNamesAreUnique(std::unordered_set<std::string> &used) const {
    for (const auto &child : subNodes_) {
      FUSILLI_RETURN_ERROR_IF(used.contains(child->getName()),
                              ErrorCode::InvalidAttribute,
                              "Symbol name '" + child->getName() +
                                  "' already in use");
      used.insert(child->getName());
      FUSILLI_CHECK_ERROR(child->checkNodeNamesAreUnique(used));
    }
    return ok();
  }
};

template <typename Derived> class NodeCRTP : public INode {
protected:
  using INode::INode;
};

namespace detail {
inline bool contiguousOrChannelsLast(const TensorPtr &t) {
  return t->isContiguous() || t->isChannelsLast();
}
inline std::string layoutMessage(const TensorPtr &t) {
  return "Tensor '" + t->getName() +
         "' is neither contiguous nor channels-last as defined by its stride";
}
} // namespace detail

// ---- convolution forward ---------------------------------------------------
// Output extent 1 + (H + 2p - d(R-1) - 1)/s per spatial dim
// (node/conv_node.h:38-56).
inline std::vector<int64_t>
getConvInferredOutputShape(const std::vector<int64_t> &xDim,
                           const std::vector<int64_t> &wDim,
                           const std::vector<int64_t> &dilation,
                           const std::vector<int64_t> &padding,
                           const std::vector<int64_t> &stride) {
  std::vector<int64_t> y(xDim.size());
  y[0] = xDim[0];
  y[1] = wDim[0];
  for (size_t i = 2; i < xDim.size(); ++i) {
    const size_t s = i - 2;
    y[i] = 1 + (xDim[i] + 2 * padding[s] - dilation[s] * (wDim[i] - 1) - 1) /
                   stride[s];
  }
  return y;
}

class ConvFPropNode : public NodeCRTP<ConvFPropNode> {
public:
  ConvFPropAttr convFPropAttr;
  ConvFPropNode(ConvFPropAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), convFPropAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return convFPropAttr.getName();
  }
  Type getType() const override final { return Type::Convolution; }

  ErrorObject preValidateNode() const override final {
    FUSILLI_LOG_LABEL_ENDL("INFO: Pre-Validating ConvFPropNode '" << getName()
                                                                  << "'");
    const auto &pad = convFPropAttr.getPadding();
    const auto &str = convFPropAttr.getStride();
    const auto &dil = convFPropAttr.getDilation();
    FUSILLI_RETURN_ERROR_IF(pad.empty(), ErrorCode::AttributeNotSet,
                            "Conv padding not set");
    FUSILLI_RETURN_ERROR_IF(str.empty(), ErrorCode::AttributeNotSet,
                            "Conv stride not set");
    FUSILLI_RETURN_ERROR_IF(dil.empty(), ErrorCode::AttributeNotSet,
                            "Conv dilation not set");
    const TensorPtr x = convFPropAttr.getX(), w = convFPropAttr.getW(),
                    y = convFPropAttr.getY();
    FUSILLI_RETURN_ERROR_IF(!x, ErrorCode::AttributeNotSet,
                            "Conv input tensor X not set");
    FUSILLI_RETURN_ERROR_IF(!w, ErrorCode::AttributeNotSet,
                            "Conv weight tensor W not set");
    FUSILLI_RETURN_ERROR_IF(!y, ErrorCode::AttributeNotSet,
                            "Conv output tensor Y not set");
    const size_t xRank = x->getDim().size(), wRank = w->getDim().size();
    FUSILLI_RETURN_ERROR_IF(
        xRank < 3, ErrorCode::InvalidAttribute,
        "Conv input tensor X must have a rank of at least 3");
    FUSILLI_RETURN_ERROR_IF(
        xRank != wRank, ErrorCode::InvalidAttribute,
        "Conv input tensor X and weight tensor W have different ranks");
    const size_t spatial = xRank - 2;
    FUSILLI_RETURN_ERROR_IF(
        pad.size() != spatial, ErrorCode::InvalidAttribute,
        "Conv padding size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(
        str.size() != spatial, ErrorCode::InvalidAttribute,
        "Conv stride size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(
        dil.size() != spatial, ErrorCode::InvalidAttribute,
        "Conv dilation size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(x),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(x));
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(w),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(w));
    const int64_t inC = x->getDim()[1], outC = w->getDim()[0],
                  filterC = w->getDim()[1];
    FUSILLI_RETURN_ERROR_IF(
        inC % filterC != 0, ErrorCode::InvalidAttribute,
        "Conv input channels must be divisible by the filter channels");
    const int64_t groups = inC / filterC;
    FUSILLI_RETURN_ERROR_IF(
        groups <= 0 || groups > inC || groups > outC,
        ErrorCode::InvalidAttribute,
        "Conv group count must be greater than 0 and less than or equal to the "
        "numbers of input and outputs channels");
    FUSILLI_RETURN_ERROR_IF(
        outC % groups != 0, ErrorCode::InvalidAttribute,
        "Conv output channels must be divisible by the group count");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    convFPropAttr.fillFromContext(context);
    const TensorPtr x = convFPropAttr.getX(), w = convFPropAttr.getW(),
                    y = convFPropAttr.getY();
    if (y->getDim().empty())
      y->setDim(getConvInferredOutputShape(
          x->getDim(), w->getDim(), convFPropAttr.getDilation(),
          convFPropAttr.getPadding(), convFPropAttr.getStride()));
    if (y->getStride().empty()) {
      const size_t rank = y->getDim().size();
      y->setStride(generateStrideFromDim(
          y->getDim(), x->isContiguous() ? getContiguousStrideOrder(rank)
                                         : getChannelsLastStrideOrder(rank)));
    }
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr x = convFPropAttr.getX(), w = convFPropAttr.getW(),
                    y = convFPropAttr.getY();
    FUSILLI_RETURN_ERROR_IF(
        y->getDim().size() < 3, ErrorCode::InvalidAttribute,
        "Conv output tensor Y must have a rank of at least 3");
    FUSILLI_RETURN_ERROR_IF(
        x->getDim().size() != y->getDim().size(), ErrorCode::InvalidAttribute,
        "Conv input tensor X and output tensor Y have different ranks");
    FUSILLI_RETURN_ERROR_IF(
        y->getDim() != getConvInferredOutputShape(
                           x->getDim(), w->getDim(), convFPropAttr.getDilation(),
                           convFPropAttr.getPadding(), convFPropAttr.getStride()),
        ErrorCode::InvalidAttribute,
        "Conv output tensor Y dimensions do not match the expected shapes "
        "inferred based on the input and weight dimensions");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(y),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(y));
    return ok();
  }
};

// ---- convolution weight gradient (node/conv_node.h:255-426) --------------------
class ConvWGradNode : public NodeCRTP<ConvWGradNode> {
public:
  ConvWGradAttr convWGradAttr;
  ConvWGradNode(ConvWGradAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), convWGradAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return convWGradAttr.getName();
  }
  Type getType() const override final { return Type::WGrad; }

  ErrorObject preValidateNode() const override final {
    FUSILLI_LOG_LABEL_ENDL("INFO: Pre-Validating ConvWGradNode '" << getName()
                                                                  << "'");
    const auto &pad = convWGradAttr.getPadding();
    const auto &str = convWGradAttr.getStride();
    const auto &dil = convWGradAttr.getDilation();
    FUSILLI_RETURN_ERROR_IF(pad.empty(), ErrorCode::AttributeNotSet,
                            "ConvWGrad padding not set");
    FUSILLI_RETURN_ERROR_IF(str.empty(), ErrorCode::AttributeNotSet,
                            "ConvWGrad stride not set");
    FUSILLI_RETURN_ERROR_IF(dil.empty(), ErrorCode::AttributeNotSet,
                            "ConvWGrad dilation not set");
    const TensorPtr dy = convWGradAttr.getDY(), x = convWGradAttr.getX(),
                    dw = convWGradAttr.getDW();
    FUSILLI_RETURN_ERROR_IF(!dy, ErrorCode::AttributeNotSet,
                            "ConvWGrad gradient tensor DY not set");
    FUSILLI_RETURN_ERROR_IF(!x, ErrorCode::AttributeNotSet,
                            "ConvWGrad input tensor X not set");
    FUSILLI_RETURN_ERROR_IF(!dw, ErrorCode::AttributeNotSet,
                            "ConvWGrad output tensor DW not set");
    const size_t dyRank = dy->getDim().size(), xRank = x->getDim().size();
    FUSILLI_RETURN_ERROR_IF(
        dyRank < 3 || xRank < 3, ErrorCode::InvalidAttribute,
        "ConvWGrad input tensors DY/X must have a rank of at least 3");
    FUSILLI_RETURN_ERROR_IF(dyRank != xRank, ErrorCode::InvalidAttribute,
                            "ConvWGrad tensors DY and X have different ranks");
    const size_t spatial = dyRank - 2;
    FUSILLI_RETURN_ERROR_IF(
        pad.size() != spatial, ErrorCode::InvalidAttribute,
        "ConvWGrad padding size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(
        str.size() != spatial, ErrorCode::InvalidAttribute,
        "ConvWGrad stride size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(
        dil.size() != spatial, ErrorCode::InvalidAttribute,
        "ConvWGrad dilation size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(dy),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(dy));
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(x),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(x));
    // The filter's channel extent gives the group count, so DW's dims are the
    // caller's to set (conv_node.h:372-375).
    FUSILLI_RETURN_ERROR_IF(dw->getDim().size() < 2,
                            ErrorCode::InvalidAttribute,
                            "ConvWGrad weight gradient tensor DW must have a "
                            "rank of at least 3");
    const int64_t inC = x->getDim()[1], outC = dy->getDim()[1],
                  filterC = dw->getDim()[1];
    FUSILLI_RETURN_ERROR_IF(filterC <= 0 || inC % filterC != 0,
                            ErrorCode::InvalidAttribute,
                            "ConvWGrad input (X) channels must be divisible by "
                            "the filter (W) channels");
    const int64_t groups = inC / filterC;
    FUSILLI_RETURN_ERROR_IF(
        groups <= 0 || groups > inC || groups > outC,
        ErrorCode::InvalidAttribute,
        "ConvWGrad group count must be greater than 0 and less than or equal "
        "to the numbers of input and outputs channels");
    FUSILLI_RETURN_ERROR_IF(
        outC % groups != 0, ErrorCode::InvalidAttribute,
        "ConvWGrad output (DY) channels must be divisible by the group count");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    convWGradAttr.fillFromContext(context);
    const TensorPtr dy = convWGradAttr.getDY(), dw = convWGradAttr.getDW();
    if (dw->getStride().empty()) {
      // follows the gradient's layout (conv_node.h:376-386)
      const size_t rank = dw->getDim().size();
      dw->setStride(generateStrideFromDim(
          dw->getDim(), dy->isContiguous() ? getContiguousStrideOrder(rank)
                                           : getChannelsLastStrideOrder(rank)));
    }
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr dy = convWGradAttr.getDY(), x = convWGradAttr.getX(),
                    dw = convWGradAttr.getDW();
    FUSILLI_RETURN_ERROR_IF(
        dw->getDim().size() < 3, ErrorCode::InvalidAttribute,
        "ConvWGrad weight gradient tensor DW must have a rank of at least 3");
    FUSILLI_RETURN_ERROR_IF(
        dw->getDim().size() != x->getDim().size() ||
            dy->getDim() != getConvInferredOutputShape(
                                x->getDim(), dw->getDim(),
                                convWGradAttr.getDilation(),
                                convWGradAttr.getPadding(),
                                convWGradAttr.getStride()),
        ErrorCode::InvalidAttribute,
        "ConvWGrad output DW dimensions do not match the expected shapes "
        "inferred based on input dimensions");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(dw),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(dw));
    return ok();
  }
};

// ---- convolution data gradient (node/conv_node.h:428-598) ----------------------
class ConvDGradNode : public NodeCRTP<ConvDGradNode> {
public:
  ConvDGradAttr convDGradAttr;
  ConvDGradNode(ConvDGradAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), convDGradAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return convDGradAttr.getName();
  }
  Type getType() const override final { return Type::DGrad; }

  ErrorObject preValidateNode() const override final {
    FUSILLI_LOG_LABEL_ENDL("INFO: Pre-Validating ConvDGradNode '" << getName()
                                                                  << "'");
    const auto &pad = convDGradAttr.getPadding();
    const auto &str = convDGradAttr.getStride();
    const auto &dil = convDGradAttr.getDilation();
    FUSILLI_RETURN_ERROR_IF(pad.empty(), ErrorCode::AttributeNotSet,
                            "ConvDGrad padding not set");
    FUSILLI_RETURN_ERROR_IF(str.empty(), ErrorCode::AttributeNotSet,
                            "ConvDGrad stride not set");
    FUSILLI_RETURN_ERROR_IF(dil.empty(), ErrorCode::AttributeNotSet,
                            "ConvDGrad dilation not set");
    const TensorPtr dy = convDGradAttr.getDY(), w = convDGradAttr.getW(),
                    dx = convDGradAttr.getDX();
    FUSILLI_RETURN_ERROR_IF(!dy, ErrorCode::AttributeNotSet,
                            "ConvDGrad gradient tensor DY not set");
    FUSILLI_RETURN_ERROR_IF(!w, ErrorCode::AttributeNotSet,
                            "ConvDGrad input tensor W not set");
    FUSILLI_RETURN_ERROR_IF(!dx, ErrorCode::AttributeNotSet,
                            "ConvDGrad output tensor DX not set");
    const size_t dyRank = dy->getDim().size(), wRank = w->getDim().size();
    FUSILLI_RETURN_ERROR_IF(
        dyRank < 3 || wRank < 3, ErrorCode::InvalidAttribute,
        "ConvDGrad input tensors DY/W must have a rank of at least 3");
    const size_t spatial = dyRank - 2;
    FUSILLI_RETURN_ERROR_IF(
        pad.size() != spatial, ErrorCode::InvalidAttribute,
        "ConvDGrad padding size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(
        str.size() != spatial, ErrorCode::InvalidAttribute,
        "ConvDGrad stride size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(
        dil.size() != spatial, ErrorCode::InvalidAttribute,
        "ConvDGrad dilation size does not match number of spatial dimensions");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(dy),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(dy));
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(w),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(w));
    // DX's dims are the caller's to set: padding and stride do not determine
    // the input extent uniquely.
    FUSILLI_RETURN_ERROR_IF(
        dx->getDim().size() < 2, ErrorCode::InvalidAttribute,
        "ConvDGrad input gradient DX must have a rank of at least 3");
    const int64_t inC = dx->getDim()[1], outC = w->getDim()[0],
                  filterC = w->getDim()[1];
    FUSILLI_RETURN_ERROR_IF(filterC <= 0 || inC % filterC != 0,
                            ErrorCode::InvalidAttribute,
                            "ConvDGrad input (DX) channels must be divisible "
                            "by the filter (W) channels");
    const int64_t groups = inC / filterC;
    FUSILLI_RETURN_ERROR_IF(
        groups <= 0 || groups > inC || groups > outC,
        ErrorCode::InvalidAttribute,
        "ConvDGrad group count must be greater than 0 and less than or equal "
        "to the numbers of input and outputs channels");
    FUSILLI_RETURN_ERROR_IF(
        outC % groups != 0, ErrorCode::InvalidAttribute,
        "ConvDGrad output (DY) channels must be divisible by the group count");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    convDGradAttr.fillFromContext(context);
    const TensorPtr dy = convDGradAttr.getDY(), dx = convDGradAttr.getDX();
    if (dx->getStride().empty()) {
      const size_t rank = dx->getDim().size();
      dx->setStride(generateStrideFromDim(
          dx->getDim(), dy->isContiguous() ? getContiguousStrideOrder(rank)
                                           : getChannelsLastStrideOrder(rank)));
    }
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr dy = convDGradAttr.getDY(), w = convDGradAttr.getW(),
                    dx = convDGradAttr.getDX();
    FUSILLI_RETURN_ERROR_IF(
        dx->getDim().size() < 3, ErrorCode::InvalidAttribute,
        "ConvDGrad input gradient DX must have a rank of at least 3");
    FUSILLI_RETURN_ERROR_IF(dy->getDim().size() != dx->getDim().size(),
                            ErrorCode::InvalidAttribute,
                            "ConvDGrad tensors DY and DX have different ranks");
    FUSILLI_RETURN_ERROR_IF(
        w->getDim().size() != dx->getDim().size() ||
            dy->getDim() != getConvInferredOutputShape(
                                dx->getDim(), w->getDim(),
                                convDGradAttr.getDilation(),
                                convDGradAttr.getPadding(),
                                convDGradAttr.getStride()),
        ErrorCode::InvalidAttribute,
        "ConvDGrad DY dimensions do not match the expected shapes inferred "
        "based on DX and W");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(dx),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(dx));
    return ok();
  }
};

// ---- matmul -------------------------------------------------------------------
// Batch dims take the larger extent; last two dims are M x N
// (node/matmul_node.h:40-66).
inline std::vector<int64_t>
getMatmulInferredOutputShape(const std::vector<int64_t> &aDim,
                             const std::vector<int64_t> &bDim) {
  const size_t rank = aDim.size();
  std::vector<int64_t> c(rank);
  for (size_t i = 0; i + 2 < rank; ++i)
    c[i] = std::max(aDim[i], bDim[i]);
  c[rank - 2] = aDim[rank - 2];
  c[rank - 1] = bDim[rank - 1];
  return c;
}

class MatmulNode : public NodeCRTP<MatmulNode> {
public:
  MatmulAttr matmulAttr;
  MatmulNode(MatmulAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), matmulAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return matmulAttr.getName();
  }
  Type getType() const override final { return Type::Matmul; }

  ErrorObject preValidateNode() const override final {
    const TensorPtr a = matmulAttr.getA(), b = matmulAttr.getB(),
                    c = matmulAttr.getC();
    FUSILLI_RETURN_ERROR_IF(!a, ErrorCode::AttributeNotSet,
                            "Matmul input tensor A not set");
    FUSILLI_RETURN_ERROR_IF(!b, ErrorCode::AttributeNotSet,
                            "Matmul input tensor B not set");
    FUSILLI_RETURN_ERROR_IF(!c, ErrorCode::AttributeNotSet,
                            "Matmul output tensor C not set");
    const auto &aDim = a->getDim(), &bDim = b->getDim();
    const size_t aRank = aDim.size(), bRank = bDim.size();
    FUSILLI_RETURN_ERROR_IF(
        aRank < 2, ErrorCode::InvalidAttribute,
        "Matmul input tensor A must have a rank of at least 2");
    FUSILLI_RETURN_ERROR_IF(
        bRank < 2, ErrorCode::InvalidAttribute,
        "Matmul input tensor B must have a rank of at least 2");
    FUSILLI_RETURN_ERROR_IF(
        aRank != bRank, ErrorCode::InvalidAttribute,
        "Matmul input tensors A and B must have the same rank: A has rank=" +
            std::to_string(aRank) + ", B has rank=" + std::to_string(bRank));
    const int64_t aK = aDim[aRank - 1], bK = bDim[bRank - 2];
    FUSILLI_RETURN_ERROR_IF(
        aK != bK, ErrorCode::InvalidAttribute,
        "Matmul input tensors A and B have incompatible inner dimensions (K): "
        "A has K=" +
            std::to_string(aK) + ", B has K=" + std::to_string(bK));
    for (size_t i = 0; i + 2 < aRank; ++i) {
      FUSILLI_RETURN_ERROR_IF(
          !(aDim[i] % bDim[i] == 0 || bDim[i] % aDim[i] == 0),
          ErrorCode::InvalidAttribute,
          "Matmul input tensors A and B have incompatible batch dimensions for "
          "broadcasting at index " +
              std::to_string(i) + ": A has dim=" + std::to_string(aDim[i]) +
              ", B has dim=" + std::to_string(bDim[i]));
    }
    FUSILLI_CHECK_ERROR(batchDimsOutermost(a, "A"));
    FUSILLI_CHECK_ERROR(batchDimsOutermost(b, "B"));
    if (a->getDataType() != b->getDataType()) {
      FUSILLI_RETURN_ERROR_IF(
          aRank != 3, ErrorCode::InvalidAttribute,
          "Mixed precision matmul is only supported when input tensors A and B "
          "are of rank 3 (single batch dim): A and B have rank=" +
              std::to_string(aRank));
      FUSILLI_RETURN_ERROR_IF(
          aDim[0] != bDim[0], ErrorCode::InvalidAttribute,
          "Mixed precision matmul input tensors A and B must have exactly "
          "equal batch dimensions (no broadcast): A has batch dim=" +
              std::to_string(aDim[0]) +
              ", B has batch dim=" + std::to_string(bDim[0]));
    }
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    matmulAttr.fillFromContext(context);
    const TensorPtr a = matmulAttr.getA(), b = matmulAttr.getB(),
                    c = matmulAttr.getC();
    if (c->getDim().empty())
      c->setDim(getMatmulInferredOutputShape(a->getDim(), b->getDim()));
    if (c->getStride().empty())
      c->setStride(generateStrideFromDim(
          c->getDim(), getContiguousStrideOrder(c->getDim().size())));
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr a = matmulAttr.getA(), b = matmulAttr.getB(),
                    c = matmulAttr.getC();
    FUSILLI_RETURN_ERROR_IF(
        c->getDim().size() < 2, ErrorCode::InvalidAttribute,
        "Matmul output tensor C must have a rank of at least 2");
    FUSILLI_RETURN_ERROR_IF(
        c->getDim() != getMatmulInferredOutputShape(a->getDim(), b->getDim()),
        ErrorCode::InvalidAttribute,
        "Matmul output tensor C dimensions do not match the expected shapes "
        "inferred based on the input dimensions");
    FUSILLI_CHECK_ERROR(batchDimsOutermost(c, "C"));
    return ok();
  }

private:
  // Batch dims must stay the outermost physical dims, in order
  // (node/matmul_node.h:240-252).
  static ErrorObject batchDimsOutermost(const TensorPtr &t,
                                        const std::string &which) {
    const auto perm = t->getLogicalToPhysicalPermuteOrder();
    for (size_t i = 0; i + 2 < t->getDim().size(); ++i)
      FUSILLI_RETURN_ERROR_IF(
          perm[i] != static_cast<int64_t>(i), ErrorCode::InvalidAttribute,
          "Matmul tensor " + which +
              " has batch dimensions that are not outermost or are transposed");
    return ok();
  }
};

// ---- pointwise ----------------------------------------------------------------
class PointwiseNode : public NodeCRTP<PointwiseNode> {
public:
  PointwiseAttr pointwiseAttr;
  PointwiseNode(PointwiseAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), pointwiseAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return pointwiseAttr.getName();
  }
  Type getType() const override final { return Type::Pointwise; }

  ErrorObject preValidateNode() const override final {
    const auto mode = pointwiseAttr.getMode();
    FUSILLI_RETURN_ERROR_IF(mode == PointwiseAttr::Mode::NOT_SET,
                            ErrorCode::AttributeNotSet,
                            "Pointwise mode not set");
    const int required = PointwiseAttr::requiredInputCount(mode);
    const TensorPtr ins[3] = {pointwiseAttr.getIN_0(), pointwiseAttr.getIN_1(),
                              pointwiseAttr.getIN_2()};
    for (int i = 0; i < 3; ++i) {
      if (i < required) {
        FUSILLI_RETURN_ERROR_IF(!ins[i], ErrorCode::AttributeNotSet,
                                std::string(PointwiseAttr::modeName(mode)) +
                                    " mode requires IN_" + std::to_string(i) +
                                    " input");
      } else {
        FUSILLI_RETURN_ERROR_IF(ins[i] != nullptr, ErrorCode::InvalidAttribute,
                                std::string(PointwiseAttr::modeName(mode)) +
                                    " mode should not have IN_" +
                                    std::to_string(i) + " input set");
      }
    }
    FUSILLI_RETURN_ERROR_IF(!pointwiseAttr.getOUT_0(),
                            ErrorCode::AttributeNotSet,
                            "Pointwise operation requires output");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    const TensorPtr out = pointwiseAttr.getOUT_0();
    if (PointwiseAttr::forcesBooleanOutput(pointwiseAttr.getMode()))
      out->setDataType(DataType::Boolean);
    pointwiseAttr.fillFromContext(context);
    const TensorPtr ins[3] = {pointwiseAttr.getIN_0(), pointwiseAttr.getIN_1(),
                              pointwiseAttr.getIN_2()};
    if (out->getDim().empty()) {
      std::vector<std::vector<int64_t>> shapes;
      for (const auto &t : ins)
        if (t)
          shapes.push_back(t->getDim());
      FUSILLI_ASSIGN_OR_RETURN(auto shape, computeBroadcastShape(shapes));
      out->setDim(std::move(shape));
    }
    if (out->getStride().empty()) {
      // Inherit the strides of the first input with the output's shape.
      for (const auto &t : ins)
        if (t && t->getDim() == out->getDim()) {
          out->setStride(t->getStride());
          break;
        }
      // A virtual output whose shape no input has follows IN_0's format.
      if (out->getStride().empty() && out->isVirtual())
        out->setStride(generateStrideFromDim(
            out->getDim(), generateStrideOrderPreservingFormat(
                               ins[0]->getStride(), out->getDim().size())));
      FUSILLI_RETURN_ERROR_IF(out->getStride().empty(),
                              ErrorCode::InvalidAttribute,
                              "Pointwise output strides could not be computed");
    }
    return ok();
  }
};

// ---- reduction ----------------------------------------------------------------
class ReductionNode : public NodeCRTP<ReductionNode> {
public:
  ReductionAttr reductionAttr;
  ReductionNode(ReductionAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), reductionAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return reductionAttr.getName();
  }
  Type getType() const override final { return Type::Reduction; }

  // Dims reduced: Y == 1 where X > 1 (node/reduction_node.h:47-56).
  std::vector<int64_t> getReductionDims() const {
    std::vector<int64_t> dims;
    const auto &x = reductionAttr.getX()->getDim();
    const auto &y = reductionAttr.getY()->getDim();
    for (size_t i = 0; i < x.size(); ++i)
      if (y[i] == 1 && x[i] > 1)
        dims.push_back(static_cast<int64_t>(i));
    return dims;
  }

  ErrorObject preValidateNode() const override final {
    FUSILLI_RETURN_ERROR_IF(reductionAttr.getMode() ==
                                ReductionAttr::Mode::NOT_SET,
                            ErrorCode::AttributeNotSet,
                            "Reduction mode not set");
    FUSILLI_RETURN_ERROR_IF(!reductionAttr.getX(), ErrorCode::AttributeNotSet,
                            "Reduction operation requires X input");
    FUSILLI_RETURN_ERROR_IF(!reductionAttr.getY(), ErrorCode::AttributeNotSet,
                            "Reduction operation requires Y output");
    FUSILLI_RETURN_ERROR_IF(reductionAttr.getX()->getDim().empty(),
                            ErrorCode::AttributeNotSet,
                            "Reduction input X dimensions not set");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    reductionAttr.fillFromContext(context);
    const TensorPtr x = reductionAttr.getX(), y = reductionAttr.getY();
    if (y->getDim().empty())
      y->setDim(x->getDim());
    if (y->getStride().empty())
      y->setStride(generateStrideFromDim(
          y->getDim(), getContiguousStrideOrder(y->getDim().size())));
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr x = reductionAttr.getX(), y = reductionAttr.getY();
    FUSILLI_RETURN_ERROR_IF(
        x->getDim().size() != y->getDim().size(), ErrorCode::InvalidAttribute,
        "Reduction input and output must have the same rank");
    FUSILLI_RETURN_ERROR_IF(
        reductionAttr.getMode() == ReductionAttr::Mode::AVG &&
            (isIntegralOrBoolType(x->getDataType()) ||
             isIntegralOrBoolType(y->getDataType())),
        ErrorCode::InvalidAttribute,
        "Reduction AVG is not supported for integral or boolean tensors");
    for (size_t i = 0; i < x->getDim().size(); ++i)
      FUSILLI_RETURN_ERROR_IF(
          y->getDim()[i] != 1 && y->getDim()[i] != x->getDim()[i],
          ErrorCode::InvalidAttribute,
          "Reduction output dimension " + std::to_string(i) +
              " must be 1 or match input dimension");
    FUSILLI_RETURN_ERROR_IF(getReductionDims().empty(),
                            ErrorCode::InvalidAttribute,
                            "Reduction requires at least one dimension to "
                            "reduce (Y[i] == 1 where X[i] > 1)");
    return ok();
  }
};

// ---- SDPA -------------------------------------------------------------------
class SdpaNode : public NodeCRTP<SdpaNode> {
public:
  SdpaAttr sdpaAttr;
  SdpaNode(SdpaAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), sdpaAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return sdpaAttr.getName();
  }
  Type getType() const override final { return Type::Sdpa; }

  ErrorObject preValidateNode() const override final {
    const TensorPtr q = sdpaAttr.getQ(), k = sdpaAttr.getK(),
                    v = sdpaAttr.getV(), o = sdpaAttr.getO(),
                    mask = sdpaAttr.getMASK();
    FUSILLI_RETURN_ERROR_IF(!q, ErrorCode::AttributeNotSet,
                            "SDPA input tensor Q not set");
    FUSILLI_RETURN_ERROR_IF(!k, ErrorCode::AttributeNotSet,
                            "SDPA input tensor K not set");
    FUSILLI_RETURN_ERROR_IF(!v, ErrorCode::AttributeNotSet,
                            "SDPA input tensor V not set");
    FUSILLI_RETURN_ERROR_IF(!o, ErrorCode::AttributeNotSet,
                            "SDPA output tensor O not set");
    FUSILLI_RETURN_ERROR_IF(q->getDim().size() != 4,
                            ErrorCode::InvalidAttribute,
                            "SDPA input tensor Q must be rank 4 "
                            "[batch, heads_q, seq_q, head_dim]");
    FUSILLI_RETURN_ERROR_IF(k->getDim().size() != 4,
                            ErrorCode::InvalidAttribute,
                            "SDPA input tensor K must be rank 4 "
                            "[batch, heads_kv, seq_kv, head_dim]");
    FUSILLI_RETURN_ERROR_IF(v->getDim().size() != 4,
                            ErrorCode::InvalidAttribute,
                            "SDPA input tensor V must be rank 4 "
                            "[batch, heads_kv, seq_kv, head_dim]");
    const auto &qd = q->getDim(), &kd = k->getDim(), &vd = v->getDim();
    FUSILLI_RETURN_ERROR_IF(
        qd[0] != kd[0] || qd[0] != vd[0], ErrorCode::InvalidAttribute,
        "SDPA input tensors Q, K, V must have matching batch dimension");
    FUSILLI_RETURN_ERROR_IF(
        qd[3] != kd[3], ErrorCode::InvalidAttribute,
        "SDPA input tensors Q and K must have matching head_dim");
    FUSILLI_RETURN_ERROR_IF(
        kd[2] != vd[2], ErrorCode::InvalidAttribute,
        "SDPA input tensors K and V must have matching sequence length");
    const int64_t hq = qd[1], hk = kd[1], hv = vd[1];
    const auto n = [](int64_t x) { return std::to_string(x); };
    if (sdpaAttr.getEnableGqa()) {
      FUSILLI_RETURN_ERROR_IF(hq % hk != 0, ErrorCode::InvalidAttribute,
                              "SDPA with GQA requires Q heads (" + n(hq) +
                                  ") to be a multiple of K heads (" + n(hk) +
                                  ")");
      FUSILLI_RETURN_ERROR_IF(hq % hv != 0, ErrorCode::InvalidAttribute,
                              "SDPA with GQA requires Q heads (" + n(hq) +
                                  ") to be a multiple of V heads (" + n(hv) +
                                  ")");
    } else {
      FUSILLI_RETURN_ERROR_IF(hq != hk, ErrorCode::InvalidAttribute,
                              "SDPA without GQA requires Q heads (" + n(hq) +
                                  ") to equal K heads (" + n(hk) + ")");
      FUSILLI_RETURN_ERROR_IF(hq != hv, ErrorCode::InvalidAttribute,
                              "SDPA without GQA requires Q heads (" + n(hq) +
                                  ") to equal V heads (" + n(hv) + ")");
    }
    FUSILLI_RETURN_ERROR_IF(
        mask && sdpaAttr.getIsCausal(), ErrorCode::InvalidAttribute,
        "SDPA attention mask and is_causal are mutually exclusive");
    if (mask) {
      const auto &md = mask->getDim();
      FUSILLI_RETURN_ERROR_IF(md.size() != 4, ErrorCode::InvalidAttribute,
                              "SDPA attention mask must be rank 4");
      FUSILLI_RETURN_ERROR_IF(md[0] != 1 && md[0] != qd[0],
                              ErrorCode::InvalidAttribute,
                              "SDPA attention mask batch dim (" + n(md[0]) +
                                  ") must be 1 or match input batch (" +
                                  n(qd[0]) + ")");
      FUSILLI_RETURN_ERROR_IF(md[1] != 1 && md[1] != hq,
                              ErrorCode::InvalidAttribute,
                              "SDPA attention mask heads dim (" + n(md[1]) +
                                  ") must be 1 or match Q heads (" + n(hq) +
                                  ")");
      FUSILLI_RETURN_ERROR_IF(
          md[2] != 1 && md[2] != qd[2], ErrorCode::InvalidAttribute,
          "SDPA attention mask seq_q dim (" + n(md[2]) +
              ") must be 1 or match Q sequence length (" + n(qd[2]) + ")");
      FUSILLI_RETURN_ERROR_IF(
          md[3] != 1 && md[3] != kd[2], ErrorCode::InvalidAttribute,
          "SDPA attention mask seq_kv dim (" + n(md[3]) +
              ") must be 1 or match KV sequence length (" + n(kd[2]) + ")");
    }
    const float p = sdpaAttr.getDropout();
    FUSILLI_RETURN_ERROR_IF(p < 0.0f || p >= 1.0f, ErrorCode::InvalidAttribute,
                            "SDPA dropout probability must be in [0, 1)");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    sdpaAttr.fillFromContext(context);
    const TensorPtr o = sdpaAttr.getO();
    const std::vector<int64_t> dim = expectedOutputDim();
    if (o->getDim().empty())
      o->setDim(dim);
    if (o->getStride().empty())
      o->setStride(generateStrideFromDim(dim, getContiguousStrideOrder(4)));
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    FUSILLI_RETURN_ERROR_IF(
        sdpaAttr.getO()->getDim() != expectedOutputDim(),
        ErrorCode::InvalidAttribute,
        "SDPA output tensor O dimensions do not match expected shape "
        "[batch, headsQ, seqQ, headDim]");
    return ok();
  }

private:
  std::vector<int64_t> expectedOutputDim() const {
    const auto &qd = sdpaAttr.getQ()->getDim();
    return {qd[0], qd[1], qd[2], sdpaAttr.getV()->getDim()[3]};
  }
};

// ---- norms ------------------------------------------------------------------
namespace norm_utils {
// Dims normalised over: all but the batch dim (node/norm_utils.h:27-36).
inline std::vector<int64_t> getNormalizedShape(const std::vector<int64_t> &xDim) {
  return std::vector<int64_t>(xDim.begin() + 1, xDim.end());
}
// [B, 1, ..., 1] contiguous: shape of the per-row statistics.
inline std::pair<std::vector<int64_t>, std::vector<int64_t>>
getTrainingForwardOutputDimAndStride(const std::vector<int64_t> &xDim) {
  std::vector<int64_t> dim(xDim.size(), 1);
  dim[0] = xDim[0];
  return {dim, generateStrideFromDim(dim, getContiguousStrideOrder(dim.size()))};
}
// X's dims with the batch dim set to 1.
inline std::vector<int64_t> getScaleBiasDim(const std::vector<int64_t> &xDim) {
  std::vector<int64_t> d = xDim;
  d[0] = 1;
  return d;
}
inline std::vector<int64_t>
getScaleBiasStride(const std::vector<int64_t> &dim,
                   const std::vector<int64_t> &xStride) {
  return generateStrideFromDim(
      dim, generateStrideOrderPreservingFormat(xStride, dim.size()));
}
inline void inferDimAndStride(const TensorPtr &t, const std::vector<int64_t> &d,
                              const std::vector<int64_t> &s) {
  if (t->getDim().empty())
    t->setDim(d);
  if (t->getStride().empty())
    t->setStride(s);
}
inline void inferScaleBias(const TensorPtr &t, const TensorPtr &x) {
  if (t->getDim().empty())
    t->setDim(getScaleBiasDim(x->getDim()));
  if (t->getStride().empty())
    t->setStride(getScaleBiasStride(t->getDim(), x->getStride()));
}
// Shared checks on an optional SCALE / BIAS operand.
inline ErrorObject checkScaleBias(const TensorPtr &t, const TensorPtr &x,
                                  const std::string &op,
                                  const std::string &which) {
  if (!t)
    return ok();
  if (!t->getDim().empty())
    FUSILLI_RETURN_ERROR_IF(t->getDim() != getScaleBiasDim(x->getDim()),
                            ErrorCode::InvalidAttribute,
                            op + " input tensor " + which +
                                " must have shape as tensor X with single "
                                "batch");
  if (!t->getStride().empty())
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(t),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(t));
  return ok();
}
} // namespace norm_utils

class RmsNormNode : public NodeCRTP<RmsNormNode> {
public:
  RmsnormAttr rmsnormAttr;
  RmsNormNode(RmsnormAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), rmsnormAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return rmsnormAttr.getName();
  }
  Type getType() const override final { return Type::RmsNorm; }

  ErrorObject preValidateNode() const override final {
    FUSILLI_RETURN_ERROR_IF(rmsnormAttr.getForwardPhase() ==
                                NormFwdPhase::NOT_SET,
                            ErrorCode::AttributeNotSet,
                            "RmsNorm forward phase not set");
    const TensorPtr x = rmsnormAttr.getX(), y = rmsnormAttr.getY(),
                    r = rmsnormAttr.getINV_RMS();
    FUSILLI_RETURN_ERROR_IF(!x, ErrorCode::AttributeNotSet,
                            "RmsNorm input tensor X not set");
    FUSILLI_RETURN_ERROR_IF(!y, ErrorCode::AttributeNotSet,
                            "RmsNorm output tensor Y not set");
    FUSILLI_RETURN_ERROR_IF(
        x->getDim().size() < 2, ErrorCode::InvalidAttribute,
        "RmsNorm input tensor X must have a rank of at least 2");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(x),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(x));
    FUSILLI_CHECK_ERROR(norm_utils::checkScaleBias(rmsnormAttr.getSCALE(), x,
                                                   "RmsNorm", "SCALE"));
    if (training()) {
      FUSILLI_RETURN_ERROR_IF(!r, ErrorCode::AttributeNotSet,
                              "RmsNorm output tensor INV_RMS not set");
    } else {
      FUSILLI_RETURN_ERROR_IF(r != nullptr, ErrorCode::InvalidAttribute,
                              "RmsNorm output tensor INV_RMS should not be set");
    }
    const TensorPtr eps = rmsnormAttr.getEpsilon();
    FUSILLI_RETURN_ERROR_IF(!eps, ErrorCode::AttributeNotSet,
                            "RmsNorm epsilon not set");
    FUSILLI_RETURN_ERROR_IF(!eps->isScalar(), ErrorCode::InvalidAttribute,
                            "RmsNorm epsilon must be a scalar constant");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    rmsnormAttr.fillFromContext(context);
    const TensorPtr x = rmsnormAttr.getX();
    if (const TensorPtr s = rmsnormAttr.getSCALE())
      norm_utils::inferScaleBias(s, x);
    norm_utils::inferDimAndStride(rmsnormAttr.getY(), x->getDim(),
                                  x->getStride());
    if (training()) {
      const auto [dim, stride] =
          norm_utils::getTrainingForwardOutputDimAndStride(x->getDim());
      norm_utils::inferDimAndStride(rmsnormAttr.getINV_RMS(), dim, stride);
    }
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr x = rmsnormAttr.getX(), y = rmsnormAttr.getY();
    FUSILLI_RETURN_ERROR_IF(
        x->getDim() != y->getDim(), ErrorCode::InvalidAttribute,
        "RmsNorm output Y tensor must have the same shape as input X tensor");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(y),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(y));
    if (training()) {
      const auto [dim, stride] =
          norm_utils::getTrainingForwardOutputDimAndStride(x->getDim());
      const TensorPtr r = rmsnormAttr.getINV_RMS();
      FUSILLI_RETURN_ERROR_IF(
          dim != r->getDim(), ErrorCode::InvalidAttribute,
          "RmsNorm output INV_RMS tensor must have shape [B, 1, ..., 1] with "
          "rank equal to input X tensor's rank, and batch dimension equal "
          "to input X tensor's batch dimension");
      FUSILLI_RETURN_ERROR_IF(
          stride != r->getStride(), ErrorCode::InvalidAttribute,
          "RmsNorm output INV_RMS tensor must have unit strides");
    }
    // The reference rejects the training phase (rmsnorm_node.h:203-206).
    FUSILLI_RETURN_ERROR_IF(
        training(), ErrorCode::NotImplemented,
        "RmsNorm training mode is not yet supported: torch-mlir does not "
        "lower the training variant");
    return ok();
  }

private:
  bool training() const {
    return rmsnormAttr.getForwardPhase() == NormFwdPhase::TRAINING;
  }
};

class LayerNormNode : public NodeCRTP<LayerNormNode> {
public:
  LayernormAttr layernormAttr;
  LayerNormNode(LayernormAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), layernormAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return layernormAttr.getName();
  }
  Type getType() const override final { return Type::LayerNorm; }

  ErrorObject preValidateNode() const override final {
    FUSILLI_RETURN_ERROR_IF(layernormAttr.getForwardPhase() ==
                                NormFwdPhase::NOT_SET,
                            ErrorCode::AttributeNotSet,
                            "LayerNorm forward phase not set");
    const TensorPtr x = layernormAttr.getX(), y = layernormAttr.getY(),
                    m = layernormAttr.getMEAN(),
                    v = layernormAttr.getINV_VARIANCE();
    FUSILLI_RETURN_ERROR_IF(!x, ErrorCode::AttributeNotSet,
                            "LayerNorm input tensor X not set");
    FUSILLI_RETURN_ERROR_IF(!y, ErrorCode::AttributeNotSet,
                            "LayerNorm output tensor Y not set");
    FUSILLI_RETURN_ERROR_IF(
        x->getDim().size() < 2, ErrorCode::InvalidAttribute,
        "LayerNorm input tensor X must have a rank of at least 2");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(x),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(x));
    FUSILLI_CHECK_ERROR(norm_utils::checkScaleBias(layernormAttr.getSCALE(), x,
                                                   "LayerNorm", "SCALE"));
    FUSILLI_CHECK_ERROR(norm_utils::checkScaleBias(layernormAttr.getBIAS(), x,
                                                   "LayerNorm", "BIAS"));
    if (training()) {
      FUSILLI_RETURN_ERROR_IF(!m, ErrorCode::AttributeNotSet,
                              "LayerNorm output tensor MEAN not set");
      FUSILLI_RETURN_ERROR_IF(!v, ErrorCode::AttributeNotSet,
                              "LayerNorm output tensor INV_VARIANCE not set");
    } else {
      FUSILLI_RETURN_ERROR_IF(m != nullptr, ErrorCode::InvalidAttribute,
                              "LayerNorm output tensor MEAN should not be set");
      FUSILLI_RETURN_ERROR_IF(
          v != nullptr, ErrorCode::InvalidAttribute,
          "LayerNorm output tensor INV_VARIANCE should not be set");
    }
    const TensorPtr eps = layernormAttr.getEpsilon();
    FUSILLI_RETURN_ERROR_IF(!eps, ErrorCode::AttributeNotSet,
                            "LayerNorm epsilon not set");
    FUSILLI_RETURN_ERROR_IF(!eps->isScalar(), ErrorCode::InvalidAttribute,
                            "LayerNorm epsilon must be a scalar constant");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    layernormAttr.fillFromContext(context);
    const TensorPtr x = layernormAttr.getX();
    if (const TensorPtr s = layernormAttr.getSCALE())
      norm_utils::inferScaleBias(s, x);
    if (const TensorPtr b = layernormAttr.getBIAS())
      norm_utils::inferScaleBias(b, x);
    norm_utils::inferDimAndStride(layernormAttr.getY(), x->getDim(),
                                  x->getStride());
    if (training()) {
      const auto [dim, stride] =
          norm_utils::getTrainingForwardOutputDimAndStride(x->getDim());
      norm_utils::inferDimAndStride(layernormAttr.getMEAN(), dim, stride);
      norm_utils::inferDimAndStride(layernormAttr.getINV_VARIANCE(), dim,
                                    stride);
    }
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr x = layernormAttr.getX(), y = layernormAttr.getY();
    FUSILLI_RETURN_ERROR_IF(
        x->getDim() != y->getDim(), ErrorCode::InvalidAttribute,
        "LayerNorm output Y tensor must have the same shape as input X tensor");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(y),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(y));
    if (training()) {
      const auto [dim, stride] =
          norm_utils::getTrainingForwardOutputDimAndStride(x->getDim());
      const TensorPtr m = layernormAttr.getMEAN(),
                      v = layernormAttr.getINV_VARIANCE();
      FUSILLI_RETURN_ERROR_IF(
          dim != m->getDim(), ErrorCode::InvalidAttribute,
          "Layernorm output MEAN tensor must have shape [B, 1, ..., 1] with "
          "rank equal to input X tensor's rank, and batch dimension equal "
          "to input X tensor's batch dimension");
      FUSILLI_RETURN_ERROR_IF(
          dim != v->getDim(), ErrorCode::InvalidAttribute,
          "LayerNorm output INV_VARIANCE tensor must have "
          "shape [B, 1, ..., 1] with  rank equal to "
          "input X tensor's rank, and batch dimension equal "
          "to input X tensor's batch dimension");
      FUSILLI_RETURN_ERROR_IF(
          stride != m->getStride(), ErrorCode::InvalidAttribute,
          "LayerNorm output MEAN tensor must have unit strides");
      FUSILLI_RETURN_ERROR_IF(
          stride != v->getStride(), ErrorCode::InvalidAttribute,
          "LayerNorm output INV_VARIANCE tensor must have unit strides");
    }
    return ok();
  }

private:
  bool training() const {
    return layernormAttr.getForwardPhase() == NormFwdPhase::TRAINING;
  }
};

// ---- batch norm (node/batchnorm_node.h:33-245) -----------------------------------
class BatchNormNode : public NodeCRTP<BatchNormNode> {
public:
  BatchnormAttr batchnormAttr;
  BatchNormNode(BatchnormAttr &&attr, const Context &ctx)
      : NodeCRTP(ctx), batchnormAttr(std::move(attr)) {}
  const std::string &getName() const override final {
    return batchnormAttr.getName();
  }
  Type getType() const override final { return Type::BatchNorm; }

  ErrorObject preValidateNode() const override final {
    FUSILLI_LOG_LABEL_ENDL("INFO: Pre-Validating BatchNormNode '" << getName()
                                                                  << "'");
    FUSILLI_RETURN_ERROR_IF(batchnormAttr.getForwardPhase() ==
                                NormFwdPhase::NOT_SET,
                            ErrorCode::AttributeNotSet,
                            "BatchNorm forward phase not set");
    const TensorPtr x = batchnormAttr.getX(), y = batchnormAttr.getY();
    FUSILLI_RETURN_ERROR_IF(!x, ErrorCode::AttributeNotSet,
                            "BatchNorm input tensor X not set");
    FUSILLI_RETURN_ERROR_IF(!y, ErrorCode::AttributeNotSet,
                            "BatchNorm output tensor Y not set");
    FUSILLI_RETURN_ERROR_IF(
        x->getDim().size() < 2, ErrorCode::InvalidAttribute,
        "BatchNorm input tensor X must have a rank of at least 2");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(x),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(x));
    if (!training()) {
      FUSILLI_RETURN_ERROR_IF(!batchnormAttr.getMEAN(),
                              ErrorCode::AttributeNotSet,
                              "BatchNorm inference requires running MEAN");
      FUSILLI_RETURN_ERROR_IF(!batchnormAttr.getVAR(),
                              ErrorCode::AttributeNotSet,
                              "BatchNorm inference requires running VAR");
      FUSILLI_RETURN_ERROR_IF(
          batchnormAttr.getSAVED_MEAN() != nullptr, ErrorCode::InvalidAttribute,
          "BatchNorm SAVED_MEAN should not be set in inference mode");
      FUSILLI_RETURN_ERROR_IF(
          batchnormAttr.getSAVED_INV_VARIANCE() != nullptr,
          ErrorCode::InvalidAttribute,
          "BatchNorm SAVED_INV_VARIANCE should not be set in inference mode");
    } else {
      FUSILLI_RETURN_ERROR_IF(!batchnormAttr.getSAVED_MEAN(),
                              ErrorCode::AttributeNotSet,
                              "BatchNorm training requires SAVED_MEAN output");
      FUSILLI_RETURN_ERROR_IF(
          !batchnormAttr.getSAVED_INV_VARIANCE(), ErrorCode::AttributeNotSet,
          "BatchNorm training requires SAVED_INV_VARIANCE output");
    }
    const TensorPtr eps = batchnormAttr.getEpsilon();
    FUSILLI_RETURN_ERROR_IF(!eps, ErrorCode::AttributeNotSet,
                            "BatchNorm epsilon not set");
    FUSILLI_RETURN_ERROR_IF(!eps->isScalar(), ErrorCode::InvalidAttribute,
                            "BatchNorm epsilon must be a scalar constant");
    const TensorPtr mom = batchnormAttr.getMomentum();
    FUSILLI_RETURN_ERROR_IF(!mom, ErrorCode::AttributeNotSet,
                            "BatchNorm momentum not set");
    FUSILLI_RETURN_ERROR_IF(!mom->isScalar(), ErrorCode::InvalidAttribute,
                            "BatchNorm momentum must be a scalar constant");
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    batchnormAttr.fillFromContext(context);
    const TensorPtr x = batchnormAttr.getX(), y = batchnormAttr.getY();
    const std::vector<int64_t> cDim = {x->getDim()[1]};
    auto infer1D = [&](const TensorPtr &t) {
      if (!t)
        return;
      if (t->getDim().empty())
        t->setDim(cDim);
      if (t->getStride().empty())
        t->setStride(std::vector<int64_t>{1});
    };
    infer1D(batchnormAttr.getSCALE());
    infer1D(batchnormAttr.getBIAS());
    infer1D(batchnormAttr.getMEAN());
    infer1D(batchnormAttr.getVAR());
    if (y->getDim().empty())
      y->setDim(x->getDim());
    if (y->getStride().empty())
      y->setStride(x->getStride());
    if (training()) {
      infer1D(batchnormAttr.getSAVED_MEAN());
      infer1D(batchnormAttr.getSAVED_INV_VARIANCE());
    }
    return ok();
  }

  ErrorObject postValidateNode() const override final {
    const TensorPtr x = batchnormAttr.getX(), y = batchnormAttr.getY();
    const std::vector<int64_t> cDim = {x->getDim()[1]};
    FUSILLI_RETURN_ERROR_IF(
        x->getDim() != y->getDim(), ErrorCode::InvalidAttribute,
        "BatchNorm output Y tensor must have the same shape as input X tensor");
    FUSILLI_RETURN_ERROR_IF(!detail::contiguousOrChannelsLast(y),
                            ErrorCode::NotImplemented,
                            detail::layoutMessage(y));
    auto check1D = [&](const TensorPtr &t, const std::string &name) {
      if (!t)
        return ok();
      FUSILLI_RETURN_ERROR_IF(
          t->getDim() != cDim, ErrorCode::InvalidAttribute,
          "BatchNorm tensor " + name +
              " must be 1D with size equal to channel dimension C");
      FUSILLI_RETURN_ERROR_IF(t->getStride() != std::vector<int64_t>{1},
                              ErrorCode::InvalidAttribute,
                              "BatchNorm tensor " + name +
                                  " must have unit stride");
      return ok();
    };
    FUSILLI_CHECK_ERROR(check1D(batchnormAttr.getSCALE(), "SCALE"));
    FUSILLI_CHECK_ERROR(check1D(batchnormAttr.getBIAS(), "BIAS"));
    FUSILLI_CHECK_ERROR(check1D(batchnormAttr.getMEAN(), "MEAN"));
    FUSILLI_CHECK_ERROR(check1D(batchnormAttr.getVAR(), "VAR"));
    if (training()) {
      FUSILLI_CHECK_ERROR(check1D(batchnormAttr.getSAVED_MEAN(), "SAVED_MEAN"));
      FUSILLI_CHECK_ERROR(check1D(batchnormAttr.getSAVED_INV_VARIANCE(),
                                  "SAVED_INV_VARIANCE"));
    }
    return ok();
  }

private:
  bool training() const {
    return batchnormAttr.getForwardPhase() == NormFwdPhase::TRAINING;
  }
};

} // namespace fusilli

#endif // FUSILLI_NODES_H
