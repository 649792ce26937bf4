// Validation expectations of the reference's node and attribute tests
// (tests/test_conv_node.cpp, test_matmul_node.cpp, test_pointwise_node.cpp,
// test_reduction_node.cpp, test_sdpa_node.cpp, test_rmsnorm_node.cpp,
// test_layernorm_node.cpp, test_tensor_attributes.cpp, test_ssa_validation.cpp,
// test_buffer.cpp, test_logging.cpp), transcribed as (set-up, stage, error code,
// exact message) over this repository's node classes.  Several cases hold two
// violations at once and expect the one the reference reports first: they pin
// the ORDER of the checks, not only their wording.  Needs no GPU.
#include <fusilli.h>

#include "mini_test.h"

#include <memory>
#include <string>
#include <vector>

using namespace fusilli;
using Dims = std::vector<int64_t>;
using TensorPtr = std::shared_ptr<TensorAttr>;

// a tensor with dims and strides (and a name, where the message quotes it)
static TensorPtr T(Dims dim, Dims stride, const char *name = nullptr) {
  auto t = std::make_shared<TensorAttr>(TensorAttr().setDim(dim).setStride(stride));
  if (name)
    t->setName(name);
  return t;
}
static TensorPtr blank() { return std::make_shared<TensorAttr>(); }
static TensorPtr scalar(float v) { return std::make_shared<TensorAttr>(v); }
static Dims contig(const Dims &d) {
  return generateStrideFromDim(d, getContiguousStrideOrder(d.size()));
}
static TensorPtr TC(Dims dim, const char *name = nullptr) { return T(dim, contig(dim), name); }

// pre-validation only
template <class Node> static ErrorObject pre(Node &&n) { return n.preValidateNode(); }
// pre-validation and inference must pass; the post-validation result is returned
template <class Node> static ErrorObject post(Node &&n) {
  ErrorObject e = n.preValidateNode();
  if (e.isError())
    return e;
  e = n.inferPropertiesNode();
  if (e.isError())
    return e;
  return n.postValidateNode();
}

// ---- convolution forward (tests/test_conv_node.cpp) -------------------------------
static ConvFPropAttr convAttr(Dims pad = {0, 0}, Dims str = {1, 1}, Dims dil = {1, 1}) {
  ConvFPropAttr a;
  if (!pad.empty())
    a.setPadding(pad);
  if (!str.empty())
    a.setStride(str);
  if (!dil.empty())
    a.setDilation(dil);
  return a;
}

TEST("ConvFPropNode: missing attributes, in the reference's order") {
  Context ctx;
  // nothing set at all: padding is asked for first
  CHECK_ERROR(pre(ConvFPropNode(ConvFPropAttr(), ctx)), ErrorCode::AttributeNotSet,
              "Conv padding not set");
  CHECK_ERROR(pre(ConvFPropNode(convAttr({0, 0}, {}, {}), ctx)), ErrorCode::AttributeNotSet,
              "Conv stride not set");
  CHECK_ERROR(pre(ConvFPropNode(convAttr({0, 0}, {1, 1}, {}), ctx)),
              ErrorCode::AttributeNotSet, "Conv dilation not set");
  // stride missing AND dilation missing: stride first
  CHECK_ERROR(pre(ConvFPropNode(ConvFPropAttr(ConvFPropAttr().setPadding(Dims{0, 0})), ctx)),
              ErrorCode::AttributeNotSet, "Conv stride not set");
  CHECK_ERROR(pre(ConvFPropNode(convAttr(), ctx)), ErrorCode::AttributeNotSet,
              "Conv input tensor X not set");
  {
    auto a = convAttr();
    a.setX(TC({1, 8, 4, 4}));
    CHECK_ERROR(pre(ConvFPropNode(std::move(a), ctx)), ErrorCode::AttributeNotSet,
                "Conv weight tensor W not set");
  }
  {
    auto a = convAttr();
    a.setX(TC({1, 8, 4, 4})).setW(TC({4, 8, 1, 1}));
    CHECK_ERROR(pre(ConvFPropNode(std::move(a), ctx)), ErrorCode::AttributeNotSet,
                "Conv output tensor Y not set");
  }
  {
    // W missing and Y missing: W first
    auto a = convAttr();
    a.setX(TC({1, 8, 4, 4}));
    CHECK_ERROR(pre(ConvFPropNode(std::move(a), ctx)), ErrorCode::AttributeNotSet,
                "Conv weight tensor W not set");
  }
}

TEST("ConvFPropNode: ranks, geometry sizes, layouts, groups") {
  Context ctx;
  auto with = [&](TensorPtr x, TensorPtr w, TensorPtr y, Dims pad = {0, 0}, Dims str = {1, 1},
                  Dims dil = {1, 1}) {
    auto a = convAttr(pad, str, dil);
    a.setX(x).setW(w).setY(y);
    return ConvFPropNode(std::move(a), ctx);
  };
  CHECK_ERROR(pre(with(TC({2, 8}), TC({4, 8}), blank())), ErrorCode::InvalidAttribute,
              "Conv input tensor X must have a rank of at least 3");
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 8, 1}), blank())), ErrorCode::InvalidAttribute,
              "Conv input tensor X and weight tensor W have different ranks");
  // rank too small AND ranks differ: the rank of X is checked first
  CHECK_ERROR(pre(with(TC({2, 8}), TC({4, 8, 1}), blank())), ErrorCode::InvalidAttribute,
              "Conv input tensor X must have a rank of at least 3");
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), blank(), {0})),
              ErrorCode::InvalidAttribute,
              "Conv padding size does not match number of spatial dimensions");
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), blank(), {0, 0}, {1})),
              ErrorCode::InvalidAttribute,
              "Conv stride size does not match number of spatial dimensions");
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), blank(), {0, 0}, {1, 1}, {1})),
              ErrorCode::InvalidAttribute,
              "Conv dilation size does not match number of spatial dimensions");
  // padding and stride both of the wrong size: padding first
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), blank(), {0}, {1})),
              ErrorCode::InvalidAttribute,
              "Conv padding size does not match number of spatial dimensions");
  // layouts: neither contiguous nor channels-last (W and H swapped)
  const Dims xd = {1, 8, 4, 6};
  CHECK_ERROR(pre(with(T(xd, {192, 24, 1, 4}, "X_invalid_layout"), TC({4, 8, 1, 1}), blank())),
              ErrorCode::NotImplemented,
              "Tensor 'X_invalid_layout' is neither contiguous nor channels-last as "
              "defined by its stride");
  CHECK_ERROR(pre(with(TC(xd), T({4, 8, 2, 3}, {48, 6, 1, 2}, "W_invalid_layout"), blank())),
              ErrorCode::NotImplemented,
              "Tensor 'W_invalid_layout' is neither contiguous nor channels-last as "
              "defined by its stride");
  // both X and W badly laid out: X is reported
  CHECK_ERROR(pre(with(T(xd, {192, 24, 1, 4}, "X_invalid_layout"),
                       T({4, 8, 2, 3}, {48, 6, 1, 2}, "W_invalid_layout"), blank())),
              ErrorCode::NotImplemented,
              "Tensor 'X_invalid_layout' is neither contiguous nor channels-last as "
              "defined by its stride");
  // groups
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 3, 1, 1}), blank())), ErrorCode::InvalidAttribute,
              "Conv input channels must be divisible by the filter channels");
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({4, 1, 1, 1}), blank())), ErrorCode::InvalidAttribute,
              "Conv group count must be greater than 0 and less than or equal to the "
              "numbers of input and outputs channels");
  CHECK_ERROR(pre(with(TC({1, 8, 4, 4}), TC({6, 2, 1, 1}), blank())), ErrorCode::InvalidAttribute,
              "Conv output channels must be divisible by the group count");
  // post-validation
  CHECK_ERROR(post(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), TC({4, 4}))),
              ErrorCode::InvalidAttribute,
              "Conv output tensor Y must have a rank of at least 3");
  CHECK_ERROR(post(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), TC({1, 4, 16}))),
              ErrorCode::InvalidAttribute,
              "Conv input tensor X and output tensor Y have different ranks");
  CHECK_ERROR(post(with(TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), TC({1, 4, 4, 5}))),
              ErrorCode::InvalidAttribute,
              "Conv output tensor Y dimensions do not match the expected shapes inferred "
              "based on the input and weight dimensions");
  CHECK_ERROR(post(with(TC({1, 8, 4, 6}), TC({4, 8, 1, 1}),
                        T({1, 4, 4, 6}, {96, 24, 1, 4}, "Y_invalid_layout"))),
              ErrorCode::NotImplemented,
              "Tensor 'Y_invalid_layout' is neither contiguous nor channels-last as "
              "defined by its stride");
  // inference fills dims and strides of an empty Y in X's format
  {
    auto y = blank();
    auto n = with(T({2, 8, 6, 6}, {288, 1, 48, 8}), TC({4, 8, 3, 3}), y, {1, 1});
    CHECK(post(std::move(n)).isOk());
    CHECK((y->getDim() == Dims{2, 4, 6, 6}));
    CHECK((y->getStride() == Dims{144, 1, 24, 4}));
  }
}

// ---- convolution gradients ---------------------------------------------------------
TEST("ConvWGradNode / ConvDGradNode: messages and their order") {
  Context ctx;
  auto wg = [&](TensorPtr dy, TensorPtr x, TensorPtr dw, Dims pad = {0, 0}, Dims str = {1, 1},
                Dims dil = {1, 1}) {
    ConvWGradAttr a;
    if (!pad.empty())
      a.setPadding(pad);
    if (!str.empty())
      a.setStride(str);
    if (!dil.empty())
      a.setDilation(dil);
    if (dy)
      a.setDY(dy);
    if (x)
      a.setX(x);
    if (dw)
      a.setDW(dw);
    return ConvWGradNode(std::move(a), ctx);
  };
  CHECK_ERROR(pre(wg(nullptr, nullptr, nullptr, {})), ErrorCode::AttributeNotSet,
              "ConvWGrad padding not set");
  CHECK_ERROR(pre(wg(nullptr, nullptr, nullptr, {0, 0}, {})), ErrorCode::AttributeNotSet,
              "ConvWGrad stride not set");
  CHECK_ERROR(pre(wg(nullptr, nullptr, nullptr, {0, 0}, {1, 1}, {})),
              ErrorCode::AttributeNotSet, "ConvWGrad dilation not set");
  CHECK_ERROR(pre(wg(nullptr, TC({1, 8, 4, 4}), TC({4, 8, 1, 1}))), ErrorCode::AttributeNotSet,
              "ConvWGrad gradient tensor DY not set");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), nullptr, TC({4, 8, 1, 1}))), ErrorCode::AttributeNotSet,
              "ConvWGrad input tensor X not set");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), nullptr)), ErrorCode::AttributeNotSet,
              "ConvWGrad output tensor DW not set");
  CHECK_ERROR(pre(wg(TC({1, 4}), TC({1, 8}), TC({4, 8}))), ErrorCode::InvalidAttribute,
              "ConvWGrad input tensors DY/X must have a rank of at least 3");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4}), TC({4, 8, 1, 1}))),
              ErrorCode::InvalidAttribute, "ConvWGrad tensors DY and X have different ranks");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), {0})),
              ErrorCode::InvalidAttribute,
              "ConvWGrad padding size does not match number of spatial dimensions");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), {0, 0}, {1})),
              ErrorCode::InvalidAttribute,
              "ConvWGrad stride size does not match number of spatial dimensions");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), TC({4, 8, 1, 1}), {0, 0}, {1, 1}, {1})),
              ErrorCode::InvalidAttribute,
              "ConvWGrad dilation size does not match number of spatial dimensions");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), TC({4, 3, 1, 1}))),
              ErrorCode::InvalidAttribute,
              "ConvWGrad input (X) channels must be divisible by the filter (W) channels");
  CHECK_ERROR(pre(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), TC({4, 1, 1, 1}))),
              ErrorCode::InvalidAttribute,
              "ConvWGrad group count must be greater than 0 and less than or equal to the "
              "numbers of input and outputs channels");
  CHECK_ERROR(pre(wg(TC({1, 6, 4, 4}), TC({1, 8, 4, 4}), TC({6, 2, 1, 1}))),
              ErrorCode::InvalidAttribute,
              "ConvWGrad output (DY) channels must be divisible by the group count");
  CHECK_ERROR(post(wg(TC({1, 4, 4, 4}), TC({1, 8, 4, 4}), TC({4, 8, 2, 2}))),
              ErrorCode::InvalidAttribute,
              "ConvWGrad output DW dimensions do not match the expected shapes inferred "
              "based on input dimensions");

  auto dg = [&](TensorPtr dy, TensorPtr w, TensorPtr dx, Dims pad = {0, 0}, Dims str = {1, 1},
                Dims dil = {1, 1}) {
    ConvDGradAttr a;
    if (!pad.empty())
      a.setPadding(pad);
    if (!str.empty())
      a.setStride(str);
    if (!dil.empty())
      a.setDilation(dil);
    if (dy)
      a.setDY(dy);
    if (w)
      a.setW(w);
    if (dx)
      a.setDX(dx);
    return ConvDGradNode(std::move(a), ctx);
  };
  CHECK_ERROR(pre(dg(nullptr, nullptr, nullptr, {})), ErrorCode::AttributeNotSet,
              "ConvDGrad padding not set");
  CHECK_ERROR(pre(dg(nullptr, nullptr, nullptr, {0, 0}, {})), ErrorCode::AttributeNotSet,
              "ConvDGrad stride not set");
  CHECK_ERROR(pre(dg(nullptr, nullptr, nullptr, {0, 0}, {1, 1}, {})),
              ErrorCode::AttributeNotSet, "ConvDGrad dilation not set");
  CHECK_ERROR(pre(dg(nullptr, TC({4, 8, 1, 1}), TC({1, 8, 4, 4}))), ErrorCode::AttributeNotSet,
              "ConvDGrad gradient tensor DY not set");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), nullptr, TC({1, 8, 4, 4}))), ErrorCode::AttributeNotSet,
              "ConvDGrad input tensor W not set");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), TC({4, 8, 1, 1}), nullptr)), ErrorCode::AttributeNotSet,
              "ConvDGrad output tensor DX not set");
  CHECK_ERROR(pre(dg(TC({1, 4}), TC({4, 8}), TC({1, 8, 4, 4}))), ErrorCode::InvalidAttribute,
              "ConvDGrad input tensors DY/W must have a rank of at least 3");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), TC({4, 8, 1, 1}), TC({1, 8, 4, 4}), {0})),
              ErrorCode::InvalidAttribute,
              "ConvDGrad padding size does not match number of spatial dimensions");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), TC({4, 8, 1, 1}), TC({1, 8, 4, 4}), {0, 0}, {1})),
              ErrorCode::InvalidAttribute,
              "ConvDGrad stride size does not match number of spatial dimensions");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), TC({4, 8, 1, 1}), TC({1, 8, 4, 4}), {0, 0}, {1, 1}, {1})),
              ErrorCode::InvalidAttribute,
              "ConvDGrad dilation size does not match number of spatial dimensions");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), TC({4, 3, 1, 1}), TC({1, 8, 4, 4}))),
              ErrorCode::InvalidAttribute,
              "ConvDGrad input (DX) channels must be divisible by the filter (W) channels");
  CHECK_ERROR(pre(dg(TC({1, 4, 4, 4}), TC({4, 1, 1, 1}), TC({1, 8, 4, 4}))),
              ErrorCode::InvalidAttribute,
              "ConvDGrad group count must be greater than 0 and less than or equal to the "
              "numbers of input and outputs channels");
  CHECK_ERROR(pre(dg(TC({1, 6, 4, 4}), TC({6, 2, 1, 1}), TC({1, 8, 4, 4}))),
              ErrorCode::InvalidAttribute,
              "ConvDGrad output (DY) channels must be divisible by the group count");
  CHECK_ERROR(post(dg(TC({1, 4, 4, 4}), TC({4, 8, 1, 1}), TC({1, 8, 4}))),
              ErrorCode::InvalidAttribute, "ConvDGrad tensors DY and DX have different ranks");
  CHECK_ERROR(post(dg(TC({1, 4, 4, 4}), TC({4, 8, 2, 2}), TC({1, 8, 4, 4}))),
              ErrorCode::InvalidAttribute,
              "ConvDGrad DY dimensions do not match the expected shapes inferred based on "
              "DX and W");
}

// ---- matmul (tests/test_matmul_node.cpp) ------------------------------------------
TEST("MatmulNode: messages with their formatted values, and their order") {
  Context ctx;
  auto mm = [&](TensorPtr a, TensorPtr b, TensorPtr c) {
    MatmulAttr m;
    if (a)
      m.setA(a);
    if (b)
      m.setB(b);
    if (c)
      m.setC(c);
    return MatmulNode(std::move(m), ctx);
  };
  CHECK_ERROR(pre(mm(nullptr, nullptr, nullptr)), ErrorCode::AttributeNotSet,
              "Matmul input tensor A not set");
  CHECK_ERROR(pre(mm(TC({4, 8}), nullptr, nullptr)), ErrorCode::AttributeNotSet,
              "Matmul input tensor B not set");
  CHECK_ERROR(pre(mm(TC({4, 8}), TC({8, 4}), nullptr)), ErrorCode::AttributeNotSet,
              "Matmul output tensor C not set");
  CHECK_ERROR(pre(mm(TC({8}), TC({8, 4}), blank())), ErrorCode::InvalidAttribute,
              "Matmul input tensor A must have a rank of at least 2");
  CHECK_ERROR(pre(mm(TC({4, 8}), TC({8}), blank())), ErrorCode::InvalidAttribute,
              "Matmul input tensor B must have a rank of at least 2");
  CHECK_ERROR(pre(mm(TC({16, 32}), TC({2, 32, 8}), blank())), ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B must have the same rank: A has rank=2, B has "
              "rank=3");
  CHECK_ERROR(pre(mm(TC({16, 32}), TC({48, 8}), blank())), ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B have incompatible inner dimensions (K): A has "
              "K=32, B has K=48");
  // rank mismatch and K mismatch together: the rank comes first
  CHECK_ERROR(pre(mm(TC({16, 32}), TC({2, 48, 8}), blank())), ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B must have the same rank: A has rank=2, B has "
              "rank=3");
  CHECK_ERROR(pre(mm(TC({3, 16, 32}), TC({5, 32, 8}), blank())), ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B have incompatible batch dimensions for "
              "broadcasting at index 0: A has dim=3, B has dim=5");
  CHECK_ERROR(pre(mm(TC({2, 3, 16, 32}), TC({2, 5, 32, 8}), blank())),
              ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B have incompatible batch dimensions for "
              "broadcasting at index 1: A has dim=3, B has dim=5");
  // a batch dim that is not outermost in memory
  CHECK_ERROR(pre(mm(T({2, 16, 32}, {32, 64, 1}), TC({2, 32, 8}), blank())),
              ErrorCode::InvalidAttribute,
              "Matmul tensor A has batch dimensions that are not outermost or are "
              "transposed");
  CHECK_ERROR(pre(mm(TC({2, 16, 32}), T({2, 32, 8}, {8, 16, 1}), blank())),
              ErrorCode::InvalidAttribute,
              "Matmul tensor B has batch dimensions that are not outermost or are "
              "transposed");
  {
    // mixed precision: rank 3 only, equal batch extents
    auto a = TC({2, 2, 16, 32}), b = TC({2, 2, 32, 8});
    a->setDataType(DataType::Half);
    b->setDataType(DataType::Int8);
    CHECK_ERROR(pre(mm(a, b, blank())), ErrorCode::InvalidAttribute,
                "Mixed precision matmul is only supported when input tensors A and B are of "
                "rank 3 (single batch dim): A and B have rank=4");
    auto a3 = TC({1, 16, 32}), b3 = TC({8, 32, 8});
    a3->setDataType(DataType::Half);
    b3->setDataType(DataType::Int8);
    CHECK_ERROR(pre(mm(a3, b3, blank())), ErrorCode::InvalidAttribute,
                "Mixed precision matmul input tensors A and B must have exactly equal batch "
                "dimensions (no broadcast): A has batch dim=1, B has batch dim=8");
  }
  CHECK_ERROR(post(mm(TC({16, 32}), TC({32, 8}), TC({16}))), ErrorCode::InvalidAttribute,
              "Matmul output tensor C must have a rank of at least 2");
  CHECK_ERROR(post(mm(TC({16, 32}), TC({32, 8}), TC({16, 9}))), ErrorCode::InvalidAttribute,
              "Matmul output tensor C dimensions do not match the expected shapes inferred "
              "based on the input dimensions");
  CHECK_ERROR(post(mm(TC({2, 16, 32}), TC({2, 32, 8}), T({2, 16, 8}, {8, 16, 1}))),
              ErrorCode::InvalidAttribute,
              "Matmul tensor C has batch dimensions that are not outermost or are "
              "transposed");
  {
    // inference: broadcast batch, contiguous C
    auto c = blank();
    CHECK(post(mm(TC({16, 16, 8, 32}), TC({1, 1, 32, 4}), c)).isOk());
    CHECK((c->getDim() == Dims{16, 16, 8, 4}));
    CHECK((c->getStride() == Dims{512, 32, 4, 1}));
  }
}

// ---- pointwise / reduction ----------------------------------------------------------
TEST("PointwiseNode / ReductionNode: messages and their order") {
  Context ctx;
  auto pw = [&](PointwiseAttr::Mode mode, TensorPtr i0, TensorPtr i1, TensorPtr i2,
                TensorPtr out) {
    PointwiseAttr a;
    a.setMode(mode);
    if (i0)
      a.setIN_0(i0);
    if (i1)
      a.setIN_1(i1);
    if (i2)
      a.setIN_2(i2);
    if (out)
      a.setOUT_0(out);
    return PointwiseNode(std::move(a), ctx);
  };
  using PM = PointwiseAttr::Mode;
  CHECK_ERROR(pre(PointwiseNode(PointwiseAttr(), ctx)), ErrorCode::AttributeNotSet,
              "Pointwise mode not set");
  CHECK_ERROR(pre(pw(PM::RELU_FWD, nullptr, nullptr, nullptr, blank())),
              ErrorCode::AttributeNotSet, "RELU_FWD mode requires IN_0 input");
  CHECK_ERROR(pre(pw(PM::ADD, TC({2, 3}), nullptr, nullptr, blank())),
              ErrorCode::AttributeNotSet, "ADD mode requires IN_1 input");
  CHECK_ERROR(pre(pw(PM::RELU_FWD, TC({2, 3}), TC({2, 3}), nullptr, blank())),
              ErrorCode::InvalidAttribute, "RELU_FWD mode should not have IN_1 input set");
  CHECK_ERROR(pre(pw(PM::ADD, TC({2, 3}), TC({2, 3}), TC({2, 3}), blank())),
              ErrorCode::InvalidAttribute, "ADD mode should not have IN_2 input set");
  // missing IN_1 and missing output: the inputs are checked first
  CHECK_ERROR(pre(pw(PM::ADD, TC({2, 3}), nullptr, nullptr, nullptr)),
              ErrorCode::AttributeNotSet, "ADD mode requires IN_1 input");
  CHECK_ERROR(pre(pw(PM::ADD, TC({2, 3}), TC({2, 3}), nullptr, nullptr)),
              ErrorCode::AttributeNotSet, "Pointwise operation requires output");
  {
    // inference: right-aligned broadcast, strides of the first input of that shape
    auto out = blank();
    auto n = pw(PM::ADD, T({2, 3, 4}, {12, 1, 3}), TC({1, 1, 4}), nullptr, out);
    CHECK(n.preValidateNode().isOk());
    CHECK(n.inferPropertiesNode().isOk());
    CHECK((out->getDim() == Dims{2, 3, 4}));
    CHECK((out->getStride() == Dims{12, 1, 3}));
  }

  auto red = [&](ReductionAttr::Mode mode, TensorPtr x, TensorPtr y) {
    ReductionAttr a;
    a.setMode(mode);
    if (x)
      a.setX(x);
    if (y)
      a.setY(y);
    return ReductionNode(std::move(a), ctx);
  };
  using RM = ReductionAttr::Mode;
  CHECK_ERROR(pre(ReductionNode(ReductionAttr(), ctx)), ErrorCode::AttributeNotSet,
              "Reduction mode not set");
  CHECK_ERROR(pre(red(RM::SUM, nullptr, blank())), ErrorCode::AttributeNotSet,
              "Reduction operation requires X input");
  CHECK_ERROR(pre(red(RM::SUM, TC({2, 3}), nullptr)), ErrorCode::AttributeNotSet,
              "Reduction operation requires Y output");
  // neither X nor Y: X first
  CHECK_ERROR(pre(red(RM::SUM, nullptr, nullptr)), ErrorCode::AttributeNotSet,
              "Reduction operation requires X input");
  CHECK_ERROR(pre(red(RM::SUM, blank(), blank())), ErrorCode::AttributeNotSet,
              "Reduction input X dimensions not set");
  CHECK_ERROR(post(red(RM::SUM, TC({2, 3, 4}), TC({2, 1}))), ErrorCode::InvalidAttribute,
              "Reduction input and output must have the same rank");
  CHECK_ERROR(post(red(RM::SUM, TC({2, 3, 4}), TC({2, 2, 1}))), ErrorCode::InvalidAttribute,
              "Reduction output dimension 1 must be 1 or match input dimension");
  CHECK_ERROR(post(red(RM::SUM, TC({2, 3, 4}), TC({2, 3, 4}))), ErrorCode::InvalidAttribute,
              "Reduction requires at least one dimension to reduce (Y[i] == 1 where X[i] > "
              "1)");
  {
    auto x = TC({2, 3, 4}), y = TC({2, 1, 1});
    x->setDataType(DataType::Int32);
    y->setDataType(DataType::Int32);
    CHECK_ERROR(post(red(RM::AVG, x, y)), ErrorCode::InvalidAttribute,
                "Reduction AVG is not supported for integral or boolean tensors");
  }
}

// ---- SDPA (tests/test_sdpa_node.cpp) -----------------------------------------------
TEST("SdpaNode: messages with their formatted values, and their order") {
  Context ctx;
  struct Opt {
    bool gqa = false, causal = false;
    float dropout = 0.0f;
    TensorPtr mask;
  };
  auto sd = [&](TensorPtr q, TensorPtr k, TensorPtr v, TensorPtr o, Opt opt = {}) {
    SdpaAttr a;
    if (q)
      a.setQ(q);
    if (k)
      a.setK(k);
    if (v)
      a.setV(v);
    if (o)
      a.setO(o);
    if (opt.mask)
      a.setMASK(opt.mask);
    a.setEnableGqa(opt.gqa).setIsCausal(opt.causal).setDropout(opt.dropout);
    return SdpaNode(std::move(a), ctx);
  };
  auto Q = [] { return TC({2, 8, 64, 32}); };
  auto KV = [] { return TC({2, 8, 128, 32}); };
  CHECK_ERROR(pre(sd(nullptr, KV(), KV(), blank())), ErrorCode::AttributeNotSet,
              "SDPA input tensor Q not set");
  CHECK_ERROR(pre(sd(Q(), nullptr, KV(), blank())), ErrorCode::AttributeNotSet,
              "SDPA input tensor K not set");
  CHECK_ERROR(pre(sd(Q(), KV(), nullptr, blank())), ErrorCode::AttributeNotSet,
              "SDPA input tensor V not set");
  CHECK_ERROR(pre(sd(Q(), KV(), KV(), nullptr)), ErrorCode::AttributeNotSet,
              "SDPA output tensor O not set");
  // nothing set: Q first
  CHECK_ERROR(pre(sd(nullptr, nullptr, nullptr, nullptr)), ErrorCode::AttributeNotSet,
              "SDPA input tensor Q not set");
  CHECK_ERROR(pre(sd(TC({2, 64, 32}), KV(), KV(), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensor Q must be rank 4 [batch, heads_q, seq_q, head_dim]");
  CHECK_ERROR(pre(sd(Q(), TC({2, 128, 32}), KV(), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensor K must be rank 4 [batch, heads_kv, seq_kv, head_dim]");
  CHECK_ERROR(pre(sd(Q(), KV(), TC({2, 128, 32}), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensor V must be rank 4 [batch, heads_kv, seq_kv, head_dim]");
  CHECK_ERROR(pre(sd(Q(), TC({3, 8, 128, 32}), KV(), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensors Q, K, V must have matching batch dimension");
  CHECK_ERROR(pre(sd(Q(), TC({2, 8, 128, 48}), KV(), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensors Q and K must have matching head_dim");
  CHECK_ERROR(pre(sd(Q(), KV(), TC({2, 8, 96, 32}), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensors K and V must have matching sequence length");
  // batch and head_dim both wrong: the batch comes first
  CHECK_ERROR(pre(sd(Q(), TC({3, 8, 128, 48}), KV(), blank())), ErrorCode::InvalidAttribute,
              "SDPA input tensors Q, K, V must have matching batch dimension");
  CHECK_ERROR(pre(sd(Q(), TC({2, 4, 128, 32}), KV(), blank())), ErrorCode::InvalidAttribute,
              "SDPA without GQA requires Q heads (8) to equal K heads (4)");
  CHECK_ERROR(pre(sd(Q(), KV(), TC({2, 4, 128, 32}), blank())), ErrorCode::InvalidAttribute,
              "SDPA without GQA requires Q heads (8) to equal V heads (4)");
  {
    Opt gqa;
    gqa.gqa = true;
    CHECK_ERROR(pre(sd(TC({2, 7, 64, 32}), TC({2, 2, 128, 32}), TC({2, 2, 128, 32}), blank(), gqa)),
                ErrorCode::InvalidAttribute,
                "SDPA with GQA requires Q heads (7) to be a multiple of K heads (2)");
    CHECK_ERROR(pre(sd(Q(), TC({2, 2, 128, 32}), TC({2, 3, 128, 32}), blank(), gqa)),
                ErrorCode::InvalidAttribute,
                "SDPA with GQA requires Q heads (8) to be a multiple of V heads (3)");
  }
  {
    Opt m;
    m.mask = TC({2, 8, 64, 128});
    m.causal = true;
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask and is_causal are mutually exclusive");
    m.causal = false;
    m.mask = TC({8, 64, 128});
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask must be rank 4");
    m.mask = TC({3, 8, 64, 128});
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask batch dim (3) must be 1 or match input batch (2)");
    m.mask = TC({2, 3, 64, 128});
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask heads dim (3) must be 1 or match Q heads (8)");
    m.mask = TC({2, 8, 32, 128});
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask seq_q dim (32) must be 1 or match Q sequence length "
                "(64)");
    m.mask = TC({2, 8, 64, 64});
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask seq_kv dim (64) must be 1 or match KV sequence length "
                "(128)");
    // batch and seq_kv both wrong: the batch is reported
    m.mask = TC({3, 8, 64, 64});
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), m)), ErrorCode::InvalidAttribute,
                "SDPA attention mask batch dim (3) must be 1 or match input batch (2)");
    m.mask = TC({1, 1, 64, 128}); // broadcast over batch and heads is fine
    CHECK(pre(sd(Q(), KV(), KV(), blank(), m)).isOk());
  }
  {
    Opt d;
    d.dropout = 1.0f;
    CHECK_ERROR(pre(sd(Q(), KV(), KV(), blank(), d)), ErrorCode::InvalidAttribute,
                "SDPA dropout probability must be in [0, 1)");
  }
  CHECK_ERROR(post(sd(Q(), KV(), KV(), TC({2, 8, 64, 48}))), ErrorCode::InvalidAttribute,
              "SDPA output tensor O dimensions do not match expected shape [batch, headsQ, "
              "seqQ, headDim]");
  {
    auto o = blank();
    CHECK(post(sd(Q(), KV(), KV(), o)).isOk());
    CHECK((o->getDim() == Dims{2, 8, 64, 32}));
  }
}

// ---- RMSNorm / LayerNorm (tests/test_rmsnorm_node.cpp, test_layernorm_node.cpp) --------
TEST("RmsNormNode: messages and their order") {
  Context ctx;
  struct Slots {
    TensorPtr x, scale, y, inv_rms, eps;
  };
  auto rms = [&](NormFwdPhase ph, Slots s) {
    RmsnormAttr a;
    a.setForwardPhase(ph);
    if (s.eps)
      a.setEpsilon(s.eps);
    if (s.x)
      a.setX(s.x);
    if (s.scale)
      a.setSCALE(s.scale);
    if (s.y)
      a.setY(s.y);
    if (s.inv_rms)
      a.setINV_RMS(s.inv_rms);
    return RmsNormNode(std::move(a), ctx);
  };
  const auto INF = NormFwdPhase::INFERENCE, TRAIN = NormFwdPhase::TRAINING;
  CHECK_ERROR(pre(RmsNormNode(RmsnormAttr(), ctx)), ErrorCode::AttributeNotSet,
              "RmsNorm forward phase not set");
  CHECK_ERROR(pre(rms(INF, {})), ErrorCode::AttributeNotSet, "RmsNorm input tensor X not set");
  CHECK_ERROR(pre(rms(INF, {.x = TC({2, 3}), .eps = scalar(1e-5f)})),
              ErrorCode::AttributeNotSet, "RmsNorm output tensor Y not set");
  CHECK_ERROR(pre(rms(INF, {.x = TC({2, 3}), .y = TC({2, 3})})), ErrorCode::AttributeNotSet,
              "RmsNorm epsilon not set");
  // Y missing and epsilon missing: Y first
  CHECK_ERROR(pre(rms(INF, {.x = TC({2, 3})})), ErrorCode::AttributeNotSet,
              "RmsNorm output tensor Y not set");
  CHECK_ERROR(pre(rms(INF, {.x = TC({6}), .y = TC({6}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "RmsNorm input tensor X must have a rank of at least 2");
  CHECK_ERROR(pre(rms(INF, {.x = TC({2, 3}), .y = TC({2, 3}), .inv_rms = T({2, 1}, {1, 1}),
                            .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute, "RmsNorm output tensor INV_RMS should not be set");
  CHECK_ERROR(pre(rms(TRAIN, {.x = TC({2, 3}), .y = TC({2, 3}), .eps = scalar(1e-5f)})),
              ErrorCode::AttributeNotSet, "RmsNorm output tensor INV_RMS not set");
  CHECK_ERROR(pre(rms(INF, {.x = TC({2, 3, 4}), .scale = TC({2, 3, 4}), .y = blank(),
                            .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "RmsNorm input tensor SCALE must have shape as tensor X with single batch");
  CHECK_ERROR(pre(rms(INF, {.x = TC({2, 3}), .y = TC({2, 3}), .eps = TC({1})})),
              ErrorCode::InvalidAttribute, "RmsNorm epsilon must be a scalar constant");
  CHECK_ERROR(post(rms(INF, {.x = TC({2, 3, 4}), .y = TC({3, 3, 4}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "RmsNorm output Y tensor must have the same shape as input X tensor");
  CHECK_ERROR(post(rms(INF, {.x = TC({2, 3, 4}), .y = T({2, 3, 4}, {4, 8, 1}, "Y_invalid_layout"),
                             .eps = scalar(1e-5f)})),
              ErrorCode::NotImplemented,
              "Tensor 'Y_invalid_layout' is neither contiguous nor channels-last as defined "
              "by its stride");
  CHECK_ERROR(post(rms(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}), .inv_rms = TC({2, 3, 4}),
                               .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "RmsNorm output INV_RMS tensor must have shape [B, 1, ..., 1] with rank equal "
              "to input X tensor's rank, and batch dimension equal to input X tensor's batch "
              "dimension");
  CHECK_ERROR(post(rms(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}),
                               .inv_rms = T({2, 1, 1}, {2, 1, 1}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute, "RmsNorm output INV_RMS tensor must have unit strides");
  {
    // inference of an unset SCALE: X's shape with one batch entry, X's format
    auto s = blank();
    auto n = rms(INF, {.x = T({2, 5, 10}, {50, 1, 5}), .scale = s, .y = blank(),
                       .eps = scalar(1e-5f)});
    CHECK(n.preValidateNode().isOk());
    CHECK(n.inferPropertiesNode().isOk());
    CHECK((s->getDim() == Dims{1, 5, 10}));
    CHECK((s->getStride() == Dims{50, 1, 5}));
  }
}

TEST("LayerNormNode: messages and their order") {
  Context ctx;
  struct Slots {
    TensorPtr x, scale, bias, y, mean, inv_var, eps;
  };
  auto ln = [&](NormFwdPhase ph, Slots s) {
    LayernormAttr a;
    a.setForwardPhase(ph);
    if (s.eps)
      a.setEpsilon(s.eps);
    if (s.x)
      a.setX(s.x);
    if (s.scale)
      a.setSCALE(s.scale);
    if (s.bias)
      a.setBIAS(s.bias);
    if (s.y)
      a.setY(s.y);
    if (s.mean)
      a.setMEAN(s.mean);
    if (s.inv_var)
      a.setINV_VARIANCE(s.inv_var);
    return LayerNormNode(std::move(a), ctx);
  };
  const auto INF = NormFwdPhase::INFERENCE, TRAIN = NormFwdPhase::TRAINING;
  auto stat = [] { return T({2, 1}, {1, 1}); };
  CHECK_ERROR(pre(LayerNormNode(LayernormAttr(), ctx)), ErrorCode::AttributeNotSet,
              "LayerNorm forward phase not set");
  CHECK_ERROR(pre(ln(INF, {})), ErrorCode::AttributeNotSet, "LayerNorm input tensor X not set");
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3}), .eps = scalar(1e-5f)})), ErrorCode::AttributeNotSet,
              "LayerNorm output tensor Y not set");
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3}), .y = TC({2, 3})})), ErrorCode::AttributeNotSet,
              "LayerNorm epsilon not set");
  CHECK_ERROR(pre(ln(INF, {.x = TC({6}), .y = TC({6}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm input tensor X must have a rank of at least 2");
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3}), .y = TC({2, 3}), .mean = stat(), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute, "LayerNorm output tensor MEAN should not be set");
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3}), .y = TC({2, 3}), .inv_var = stat(),
                           .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm output tensor INV_VARIANCE should not be set");
  // both statistics set in inference: MEAN is reported
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3}), .y = TC({2, 3}), .mean = stat(), .inv_var = stat(),
                           .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute, "LayerNorm output tensor MEAN should not be set");
  CHECK_ERROR(pre(ln(TRAIN, {.x = TC({2, 3}), .y = TC({2, 3}), .eps = scalar(1e-5f)})),
              ErrorCode::AttributeNotSet, "LayerNorm output tensor MEAN not set");
  CHECK_ERROR(pre(ln(TRAIN, {.x = TC({2, 3}), .y = TC({2, 3}), .mean = stat(),
                             .eps = scalar(1e-5f)})),
              ErrorCode::AttributeNotSet, "LayerNorm output tensor INV_VARIANCE not set");
  CHECK(pre(ln(TRAIN, {.x = TC({2, 3}), .scale = TC({1, 3}), .bias = TC({1, 3}), .y = TC({2, 3}),
                       .mean = stat(), .inv_var = stat(), .eps = scalar(1e-5f)}))
            .isOk());
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3, 4}), .scale = TC({2, 3, 4}), .y = blank(),
                           .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm input tensor SCALE must have shape as tensor X with single batch");
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3, 4}), .bias = TC({2, 3, 4}), .y = blank(),
                           .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm input tensor BIAS must have shape as tensor X with single batch");
  // SCALE and BIAS both wrong: SCALE is reported
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3, 4}), .scale = TC({2, 3, 4}), .bias = TC({2, 3, 4}),
                           .y = blank(), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm input tensor SCALE must have shape as tensor X with single batch");
  CHECK_ERROR(pre(ln(INF, {.x = TC({2, 3}), .y = TC({2, 3}), .eps = TC({1})})),
              ErrorCode::InvalidAttribute, "LayerNorm epsilon must be a scalar constant");
  CHECK_ERROR(post(ln(INF, {.x = TC({2, 3, 4}), .y = TC({3, 3, 4}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm output Y tensor must have the same shape as input X tensor");
  CHECK_ERROR(post(ln(INF, {.x = TC({2, 3, 4}), .y = T({2, 3, 4}, {4, 8, 1}, "Y_invalid_layout"),
                            .eps = scalar(1e-5f)})),
              ErrorCode::NotImplemented,
              "Tensor 'Y_invalid_layout' is neither contiguous nor channels-last as defined "
              "by its stride");
  auto unit3 = [] { return T({2, 1, 1}, {1, 1, 1}); };
  CHECK_ERROR(post(ln(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}), .mean = TC({2, 3, 4}),
                              .inv_var = unit3(), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "Layernorm output MEAN tensor must have shape [B, 1, ..., 1] with rank equal to "
              "input X tensor's rank, and batch dimension equal to input X tensor's batch "
              "dimension");
  CHECK_ERROR(post(ln(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}), .mean = unit3(),
                              .inv_var = TC({2, 3, 4}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm output INV_VARIANCE tensor must have shape [B, 1, ..., 1] with  rank "
              "equal to input X tensor's rank, and batch dimension equal to input X tensor's "
              "batch dimension");
  CHECK_ERROR(post(ln(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}),
                              .mean = T({2, 1, 1}, {2, 1, 1}, "MEAN_invalid_layout"),
                              .inv_var = unit3(), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute, "LayerNorm output MEAN tensor must have unit strides");
  CHECK_ERROR(post(ln(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}), .mean = unit3(),
                              .inv_var = T({2, 1, 1}, {2, 1, 1}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "LayerNorm output INV_VARIANCE tensor must have unit strides");
  // MEAN's shape and INV_VARIANCE's stride both wrong: shapes are checked first
  CHECK_ERROR(post(ln(TRAIN, {.x = TC({2, 3, 4}), .y = TC({2, 3, 4}), .mean = TC({2, 3, 4}),
                              .inv_var = T({2, 1, 1}, {2, 1, 1}), .eps = scalar(1e-5f)})),
              ErrorCode::InvalidAttribute,
              "Layernorm output MEAN tensor must have shape [B, 1, ..., 1] with rank equal to "
              "input X tensor's rank, and batch dimension equal to input X tensor's batch "
              "dimension");
  {
    // under-specified outputs are inferred (training): Y like X, statistics [B, 1] unit
    auto y = blank(), m = blank(), v = blank();
    auto n = ln(TRAIN, {.x = TC({2, 5}), .y = y, .mean = m, .inv_var = v, .eps = scalar(1e-5f)});
    CHECK(n.inferPropertiesNode().isOk());
    CHECK((y->getDim() == Dims{2, 5}) && (y->getStride() == Dims{5, 1}));
    CHECK((m->getDim() == Dims{2, 1}) && (m->getStride() == Dims{1, 1}));
    CHECK((v->getDim() == Dims{2, 1}) && (v->getStride() == Dims{1, 1}));
    // partially specified BIAS keeps its dims and takes X's format
    auto b = std::make_shared<TensorAttr>(TensorAttr().setDim({1, 5, 10}));
    auto n2 = ln(INF, {.x = T({2, 5, 10}, {50, 1, 5}), .bias = b, .y = blank(), .eps = scalar(1e-5f)});
    CHECK(n2.preValidateNode().isOk());
    CHECK(n2.inferPropertiesNode().isOk());
    CHECK((b->getStride() == Dims{50, 1, 5}));
  }
}

// ---- TensorAttr (tests/test_tensor_attributes.cpp) -----------------------------------
TEST("TensorAttr: the reference's validation messages by tensor name, and their order") {
  auto named = [](const char *name) {
    TensorAttr t;
    t.setName(name);
    return t;
  };
  CHECK_ERROR(named("nodim").validate(), ErrorCode::AttributeNotSet, "Tensor 'nodim' dims not set");
  CHECK_ERROR(named("nostride").setDim({2}).validate(), ErrorCode::AttributeNotSet,
              "Tensor 'nostride' strides not set");
  CHECK_ERROR(named("nostride").setDim({2}).setStride({1}).validate(), ErrorCode::AttributeNotSet,
              "Tensor 'nostride' data type not set");
  CHECK_ERROR(named("diffrank").setDim({2, 3}).setStride({1}).setDataType(DataType::Float).validate(),
              ErrorCode::InvalidAttribute,
              "Tensor 'diffrank' uses dim and stride of different dimensionality");
  // different rank AND no data type: the rank is reported
  CHECK_ERROR(named("diffrank").setDim({2, 3}).setStride({1}).validate(),
              ErrorCode::InvalidAttribute,
              "Tensor 'diffrank' uses dim and stride of different dimensionality");
  CHECK_ERROR(named("zero").setDim({2, 0, 3}).setStride({6, 3, 1}).setDataType(DataType::Float).validate(),
              ErrorCode::InvalidAttribute,
              "Tensor 'zero' has invalid physical representation. It must be a valid "
              "permutation of the logical dimensions");
  {
    TensorAttr v(1.0f);
    v.setName("invalid").setIsVirtual(true);
    CHECK_ERROR(v.validate(), ErrorCode::InvalidAttribute,
                "Tensor 'invalid' cannot be both virtual (intermediate) and a scalar constant");
    TensorAttr n(1.0f);
    n.setName("nonscalar").setIsScalar(false);
    CHECK_ERROR(n.validate(), ErrorCode::InvalidAttribute,
                "Tensor 'nonscalar' has a scalar value set but is not marked as a scalar");
    TensorAttr m = named("nonscalar");
    m.setDim({1}).setStride({1}).setDataType(DataType::Float).setIsScalar(true);
    CHECK_ERROR(m.validate(), ErrorCode::InvalidAttribute,
                "Tensor 'nonscalar' is marked as a scalar but does not have a scalar value set");
  }
  auto dyn = [&](const char *name, Dims d, Dims s, std::initializer_list<size_t> idx) {
    TensorAttr t = named(name);
    t.setDim(d).setStride(s).setDataType(DataType::Float).setDynamicDims(idx);
    return t.validate();
  };
  CHECK_ERROR(dyn("bad_dynamic", {4, 8}, {8, 1}, {2}), ErrorCode::InvalidAttribute,
              "Tensor 'bad_dynamic' has dynamic dim index 2 out of range for rank 2");
  CHECK_ERROR(dyn("unit_dynamic", {1, 8}, {8, 1}, {0}), ErrorCode::InvalidAttribute,
              "Tensor 'unit_dynamic' has dynamic dim at index 0 with representative size 1, "
              "which is not supported");
  CHECK_ERROR(dyn("dynamic_broadcast", {4, 8}, {0, 1}, {0}), ErrorCode::InvalidAttribute,
              "Tensor 'dynamic_broadcast' has dynamic dim at index 0 with stride 0 (broadcast "
              "stride), which is not supported");
  // size 1 AND stride 0 on the dynamic dim: the stride is reported
  CHECK_ERROR(dyn("dynamic_unit_zero_stride", {1, 8}, {0, 1}, {0}), ErrorCode::InvalidAttribute,
              "Tensor 'dynamic_unit_zero_stride' has dynamic dim at index 0 with stride 0 "
              "(broadcast stride), which is not supported");
  CHECK_ERROR(dyn("dynamic_on_broadcast_stride_tensor", {4, 8}, {1, 0}, {0}),
              ErrorCode::InvalidAttribute,
              "Tensor 'dynamic_on_broadcast_stride_tensor' has dynamic dimensions on a tensor "
              "with broadcast strides, which is not supported");
  CHECK(dyn("fine", {4, 8}, {8, 1}, {0}).isOk());
  {
    auto bad = generateStrideFromLayout({1, 2, 3, 4}, "WXYZ");
    CHECK_ERROR(ErrorObject(bad), ErrorCode::InvalidArgument, "Invalid layout string: WXYZ");
    auto rank = generateStrideFromLayout({1, 2, 3}, "NCHW");
    CHECK_ERROR(ErrorObject(rank), ErrorCode::InvalidArgument,
                "Invalid input dimensions and layout: they must have the same rank");
    auto good = generateStrideFromLayout({2, 3, 4, 5}, "NHWC");
    CHECK(isOk(good) && (*good == Dims{60, 1, 15, 3}));
  }
}

// ---- symbol names (tests/test_ssa_validation.cpp) ------------------------------------
TEST("Graph: symbol names of inputs, outputs and nodes share one namespace") {
  // The reference's six graphs: two 1-D convolutions in a row, with names that
  // clash in different places.
  auto build = [](const char *graph, const char *in0, const char *in1, const char *node1,
                  const char *y_name, const char *node2, const char *z_name) {
    Graph g;
    g.setName(graph);
    g.setIODataType(DataType::Half)
        .setComputeDataType(DataType::Float)
        .setIntermediateDataType(DataType::Float);
    auto x = g.tensor(TensorAttr().setName(in0).setDim({1}).setStride({1}));
    auto w = g.tensor(TensorAttr().setName(in1).setDim({1}).setStride({1}));
    auto y = g.convFProp(
        x, w, ConvFPropAttr().setPadding({0}).setStride({1}).setDilation({1}).setName(node1));
    y->setDim({1}).setStride({1});
    if (y_name)
      y->setName(y_name);
    auto z = g.convFProp(
        y, w, ConvFPropAttr().setPadding({0}).setStride({1}).setDilation({1}).setName(node2));
    z->setDim({1}).setStride({1});
    if (z_name)
      z->setName(z_name);
    z->setOutput(true);
    return g.validate();
  };
  CHECK_ERROR(build("multiple_inputs_same_name", "arg0", "arg0", "conv1", nullptr, "conv2", nullptr),
              ErrorCode::InvalidAttribute, "Symbol name 'arg0' already in use");
  CHECK_ERROR(build("multiple_outputs_same_name", "arg0", "arg1", "conv1", "result", "conv2", "result"),
              ErrorCode::InvalidAttribute, "Symbol name 'result' already in use");
  CHECK_ERROR(build("multiple_outputs_same_inferred_name", "arg0", "arg1", "conv", nullptr, "conv",
                    nullptr),
              ErrorCode::InvalidAttribute, "Symbol name 'conv_Y' already in use");
  CHECK_ERROR(build("multiple_nodes_same_name", "arg0", "arg1", "conv", nullptr, "conv", "result"),
              ErrorCode::InvalidAttribute, "Symbol name 'conv' already in use");
  CHECK_ERROR(build("input_and_outputs_same_name", "arg0", "arg1", "conv", nullptr, "conv", "arg0"),
              ErrorCode::InvalidAttribute, "Symbol name 'arg0' already in use");
  CHECK_ERROR(build("input_and_nodes_same_name", "arg0", "arg1", "arg0", nullptr, "conv", nullptr),
              ErrorCode::InvalidAttribute, "Symbol name 'arg0' already in use");
}

// ---- ErrorObject (tests/test_logging.cpp) -------------------------------------------------
TEST("ErrorObject: codes, messages and their printed form") {
  const ErrorObject fine = ok();
  CHECK(fine.isOk() && !fine.isError() && fine.getCode() == ErrorCode::OK);
  const ErrorObject e1 = error(ErrorCode::AttributeNotSet, "missing attribute");
  CHECK(e1.isError() && e1.getCode() == ErrorCode::AttributeNotSet &&
        e1.getMessage() == "missing attribute");
  const ErrorObject e2 = error(ErrorCode::VariantPackError, "variant pack error");
  CHECK(e2.getCode() == ErrorCode::VariantPackError && e2.getMessage() == "variant pack error");
  const ErrorObject e3 = error(ErrorCode::NotImplemented, "not implemented");
  CHECK(e3.getCode() == ErrorCode::NotImplemented && e3.getMessage() == "not implemented");
  auto fails = []() -> ErrorObject {
    FUSILLI_RETURN_ERROR_IF(true, ErrorCode::InvalidAttribute, "test case");
    return ok();
  };
  CHECK_ERROR(fails(), ErrorCode::InvalidAttribute, "test case");
  auto passes_on = [&]() -> ErrorObject {
    FUSILLI_CHECK_ERROR(fails());
    return error(ErrorCode::RuntimeFailure, "not reached");
  };
  CHECK_ERROR(passes_on(), ErrorCode::InvalidAttribute, "test case");
}

int main(int argc, char **argv) { return mini::run(argc, argv); }
