// Host-only tests of the graph API: layout math against the reference's known
// answers, per-node validation (codes and messages as in the reference's
// tests/test_*_node.cpp), the Graph state machine and the artifact contract
// (tests/test_graph.cpp:373-510), Handle / Buffer rules (tests/test_handle.cpp,
// tests/test_buffer.cpp).  Needs no GPU.
#include <fusilli.h>

#include <sstream>
#include <thread>

#include "mini_test.h"

using namespace fusilli;
#include "layout_vectors.inc"

using Dims = std::vector<int64_t>;

// ---- layout -----------------------------------------------------------------
TEST("layout: reference known answers") {
  TensorAttr t;
  for (const auto &c : k_physical_dim) {
    t.setDim(c.dim).setStride(c.stride);
    CHECK(t.getPhysicalDim() == c.expect);
  }
  for (const auto &c : k_logical_to_physical) {
    t.setDim(c.dim).setStride(c.stride);
    CHECK(t.getLogicalToPhysicalPermuteOrder() == c.expect);
  }
  for (const auto &c : k_physical_to_logical) {
    t.setDim(c.dim).setStride(c.stride);
    CHECK(t.getPhysicalToLogicalPermuteOrder() == c.expect);
  }
  for (const auto &c : k_valid_representation) {
    t.setDim(c.dim).setStride(c.stride);
    CHECK(t.hasValidPhysicalRepresentation() == c.expect);
  }
}

TEST("layout: stride orders and generators") {
  // reference tensor_attributes.h:156-193 examples
  CHECK((getContiguousStrideOrder(4) == std::vector<size_t>{3, 2, 1, 0}));
  CHECK((getChannelsLastStrideOrder(4) == std::vector<size_t>{3, 0, 2, 1}));
  CHECK((getChannelsLastStrideOrder(5) == std::vector<size_t>{4, 0, 3, 2, 1}));
  CHECK((generateStrideOrderPreservingFormat({10, 30, 20}, 3) ==
         std::vector<size_t>{0, 2, 1}));
  CHECK((generateStrideOrderPreservingFormat({10, 30, 20}, 5) ==
         std::vector<size_t>{0, 2, 1, 3, 4}));
  // dim (10,3,12,12), order {3,0,2,1} -> stride (432,1,36,3)
  CHECK((generateStrideFromDim({10, 3, 12, 12}, {3, 0, 2, 1}) ==
         Dims{432, 1, 36, 3}));
  // benchmark config 3 layouts
  CHECK((generateStrideFromDim({32, 64, 56, 56}, getChannelsLastStrideOrder(4)) ==
         Dims{200704, 1, 3584, 64}));
  CHECK((generateStrideFromDim({128, 64, 3, 3}, getChannelsLastStrideOrder(4)) ==
         Dims{576, 1, 192, 64}));
  CHECK((getChannelsLastToContiguousPermuteOrder(4) == Dims{0, 3, 1, 2}));
  CHECK((getContiguousToChannelsLastPermuteOrder(4) == Dims{0, 2, 3, 1}));
  CHECK((inversePermutation({0, 2, 3, 1}) == Dims{0, 3, 1, 2}));
  auto nhwc = generateStrideFromLayout({2, 3, 4, 5}, "NHWC");
  REQUIRE(isOk(nhwc));
  CHECK((*nhwc == Dims{60, 1, 15, 3}));
  auto bad = generateStrideFromLayout({2, 3, 4, 5}, "NWHC");
  CHECK_ERROR(ErrorObject(bad), ErrorCode::InvalidArgument,
              "Invalid layout string: NWHC");
  auto rank = generateStrideFromLayout({2, 3, 4}, "NCHW");
  CHECK_ERROR(ErrorObject(rank), ErrorCode::InvalidArgument,
              "Invalid input dimensions and layout: they must have the same "
              "rank");
}

TEST("layout: broadcast shape") {
  auto s = computeBroadcastShape({{64, 16, 1, 1}, {1, 32, 1}});
  REQUIRE(isOk(s));
  CHECK((*s == Dims{64, 16, 32, 1}));
  auto e = computeBroadcastShape({{3, 4}, {5, 4}});
  CHECK_ERROR(ErrorObject(e), ErrorCode::InvalidAttribute,
              "Cannot broadcast two non unit dimensions");
  auto empty = computeBroadcastShape({{}, {}});
  CHECK_ERROR(ErrorObject(empty), ErrorCode::InvalidAttribute,
              "All input shapes are empty");
}

TEST("TensorAttr: validate codes and messages") {
  TensorAttr t;
  t.setName("x");
  CHECK_ERROR(t.validate(), ErrorCode::AttributeNotSet, "Tensor 'x' dims not set");
  t.setDim({2, 3});
  CHECK_ERROR(t.validate(), ErrorCode::AttributeNotSet,
              "Tensor 'x' strides not set");
  t.setStride({3});
  CHECK_ERROR(t.validate(), ErrorCode::InvalidAttribute,
              "Tensor 'x' uses dim and stride of different dimensionality");
  t.setStride({5, 1});
  CHECK_ERROR(t.validate(), ErrorCode::InvalidAttribute,
              "Tensor 'x' has invalid physical representation. It must be a "
              "valid permutation of the logical dimensions");
  t.setStride({3, 1});
  CHECK_ERROR(t.validate(), ErrorCode::AttributeNotSet,
              "Tensor 'x' data type not set");
  t.setDataType(DataType::Float);
  CHECK(isOk(t.validate()));
  t.setIsScalar(true);
  CHECK_ERROR(t.validate(), ErrorCode::InvalidAttribute,
              "Tensor 'x' is marked as a scalar but does not have a scalar "
              "value set");
  TensorAttr s(2.5f);
  s.setName("s");
  CHECK(isOk(s.validate()));
  CHECK(s.isScalar() && s.getDataType() == DataType::Float &&
        s.getDim() == Dims{1} && scalarAsDouble(s) == 2.5);
  s.setIsVirtual(true);
  CHECK_ERROR(s.validate(), ErrorCode::InvalidAttribute,
              "Tensor 's' cannot be both virtual (intermediate) and a scalar "
              "constant");
  TensorAttr d;
  d.setName("d").setDim({4, 8}).setStride({8, 1}).setDataType(DataType::Float);
  d.setDynamicDim(5);
  CHECK_ERROR(d.validate(), ErrorCode::InvalidAttribute,
              "Tensor 'd' has dynamic dim index 5 out of range for rank 2");
}

TEST("TensorAttr: dtype fill, contiguity, volume") {
  Context ctx;
  ctx.setIODataType(DataType::Half).setIntermediateDataType(DataType::Float);
  TensorAttr io, virt;
  virt.setIsVirtual(true);
  io.fillFromContext(ctx);
  virt.fillFromContext(ctx);
  CHECK(io.getDataType() == DataType::Half);
  CHECK(virt.getDataType() == DataType::Float);
  TensorAttr t;
  t.setDim({2, 3, 4, 5}).setStride({60, 20, 5, 1});
  CHECK(t.isContiguous() && !t.isChannelsLast() && t.getVolume() == 120);
  t.setStride({60, 1, 15, 3});
  CHECK(!t.isContiguous() && t.isChannelsLast());
  t.setDim({8, 2, 64, 128}).setStride({0, 0, 128, 1});
  CHECK(t.hasBroadcastDims());
  CHECK((t.getUnexpandedDim() == Dims{1, 1, 64, 128}));
}

// ---- helpers ----------------------------------------------------------------
static TensorAttr mk(const std::string &name, Dims dim, Dims stride,
                     DataType dt = DataType::Float) {
  return TensorAttr().setName(name).setDim(dim).setStride(stride).setDataType(dt);
}
static Dims contig(const Dims &d) {
  return generateStrideFromDim(d, getContiguousStrideOrder(d.size()));
}
static Dims chlast(const Dims &d) {
  return generateStrideFromDim(d, getChannelsLastStrideOrder(d.size()));
}
static Graph newGraph(const std::string &name, DataType dt = DataType::Float) {
  Graph g;
  g.setName(name).setIODataType(dt).setIntermediateDataType(DataType::Float)
      .setComputeDataType(DataType::Float);
  return g;
}

// ---- node validation ----------------------------------------------------------
TEST("conv node: inference and errors") {
  {
    Graph g = newGraph("conv_infer", DataType::BFloat16);
    auto x = g.tensor(mk("x", {32, 64, 56, 56}, chlast({32, 64, 56, 56}),
                         DataType::BFloat16));
    auto w = g.tensor(mk("w", {128, 64, 3, 3}, chlast({128, 64, 3, 3}),
                         DataType::BFloat16));
    ConvFPropAttr a;
    a.setPadding({1, 1}).setStride({1, 1}).setDilation({1, 1});
    auto y = g.convFProp(x, w, a);
    y->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK((y->getDim() == Dims{32, 128, 56, 56}));
    CHECK((y->getStride() == Dims{401408, 1, 7168, 128})); // follows X: NHWC
    CHECK(y->getName() == "conv_fprop_0_Y");
    CHECK(y->getDataType() == DataType::BFloat16);
  }
  {
    Graph g = newGraph("conv_shape");
    auto x = g.tensor(mk("x", {2, 6, 9, 11}, contig({2, 6, 9, 11})));
    auto w = g.tensor(mk("w", {4, 3, 3, 2}, contig({4, 3, 3, 2})));
    ConvFPropAttr a;
    a.setPadding({0, 1}).setStride({2, 1}).setDilation({1, 2});
    auto y = g.convFProp(x, w, a);
    y->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK((y->getDim() == Dims{2, 4, 4, 11})); // 1+(9-2-1)/2, 1+(11+2-2-1)/1
    CHECK(y->isContiguous());
  }
  auto build = [](auto &&tweak) {
    Graph g = newGraph("conv_err");
    auto x = g.tensor(mk("x", {2, 8, 5, 5}, contig({2, 8, 5, 5})));
    auto w = g.tensor(mk("w", {4, 8, 1, 1}, contig({4, 8, 1, 1})));
    ConvFPropAttr a;
    a.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    tweak(g, x, w, a);
    auto y = g.convFProp(x, w, a);
    y->setOutput(true);
    return g.validate();
  };
  CHECK_ERROR(build([](auto &, auto &, auto &, auto &a) { a.setPadding({}); }),
              ErrorCode::AttributeNotSet, "Conv padding not set");
  CHECK_ERROR(build([](auto &, auto &, auto &, auto &a) { a.setStride({1}); }),
              ErrorCode::InvalidAttribute,
              "Conv stride size does not match number of spatial dimensions");
  CHECK_ERROR(build([](auto &, auto &x, auto &, auto &) {
                x->setStride({1, 2, 16, 80});
              }),
              ErrorCode::NotImplemented,
              "Tensor 'x' is neither contiguous nor channels-last as defined "
              "by its stride");
  CHECK_ERROR(build([](auto &, auto &, auto &w, auto &) {
                w->setDim({4, 3, 1, 1}).setStride({3, 1, 1, 1});
              }),
              ErrorCode::InvalidAttribute,
              "Conv input channels must be divisible by the filter channels");
  CHECK_ERROR(build([](auto &, auto &, auto &w, auto &) {
                w->setDim({3, 4, 1, 1}).setStride({4, 1, 1, 1});
              }),
              ErrorCode::InvalidAttribute,
              "Conv output channels must be divisible by the group count");
}

TEST("conv gradient nodes: inference and errors") {
  // tests/test_conv_node.cpp:503-1333 of the reference
  const int64_t n = 16, c = 256, h = 64, w = 32, k = 128;
  {
    // wgrad: DW keeps the caller's dims and takes DY's layout (NHWC here)
    Graph g = newGraph("wgrad_infer", DataType::Half);
    auto dy = g.tensor(mk("dy", {n, k, h, w}, chlast({n, k, h, w}), DataType::Half));
    auto x = g.tensor(mk("x", {n, c, h, w}, chlast({n, c, h, w}), DataType::Half));
    ConvWGradAttr a;
    a.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    auto dw = g.convWGrad(dy, x, a);
    dw->setDim({k, c, 1, 1}).setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK(dw->getName() == "conv_wgrad_0_DW");
    CHECK((dw->getStride() == chlast({k, c, 1, 1})));
    CHECK(dw->getDataType() == DataType::Half);
  }
  {
    // dgrad: DX keeps the caller's dims and takes DY's layout (contiguous)
    Graph g = newGraph("dgrad_infer", DataType::Half);
    auto dy = g.tensor(mk("dy", {n, k, h, w}, contig({n, k, h, w}), DataType::Half));
    auto wt = g.tensor(mk("w", {k, c, 1, 1}, contig({k, c, 1, 1}), DataType::Half));
    ConvDGradAttr a;
    a.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    auto dx = g.convDGrad(dy, wt, a);
    dx->setDim({n, c, h, w}).setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK(dx->getName() == "conv_dgrad_0_DX");
    CHECK(dx->isContiguous());
  }
  Context ctx;
  auto T = [](const char *name, Dims d, Dims st) {
    return std::make_shared<TensorAttr>(mk(name, d, st));
  };
  auto wnode = [&](auto &&tweak) {
    ConvWGradAttr a;
    a.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    a.setDY(T("DY", {n, k, h, w}, chlast({n, k, h, w})))
        .setX(T("X", {n, c, h, w}, chlast({n, c, h, w})))
        .setDW(T("DW", {k, c, 1, 1}, contig({k, c, 1, 1})));
    tweak(a);
    return ConvWGradNode(std::move(a), ctx);
  };
  auto dnode = [&](auto &&tweak) {
    ConvDGradAttr a;
    a.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    a.setDY(T("DY", {n, k, h, w}, chlast({n, k, h, w})))
        .setW(T("W", {k, c, 1, 1}, contig({k, c, 1, 1})))
        .setDX(T("DX", {n, c, h, w}, chlast({n, c, h, w})));
    tweak(a);
    return ConvDGradNode(std::move(a), ctx);
  };
  REQUIRE_OK(wnode([](auto &) {}).preValidateNode());
  REQUIRE_OK(dnode([](auto &) {}).preValidateNode());
  CHECK_ERROR(wnode([](auto &a) { a.setPadding(Dims{}); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvWGrad padding not set");
  CHECK_ERROR(wnode([](auto &a) { a.setStride(Dims{}); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvWGrad stride not set");
  CHECK_ERROR(wnode([](auto &a) { a.setDilation(Dims{}); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvWGrad dilation not set");
  CHECK_ERROR(wnode([](auto &a) { a.setDY(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvWGrad gradient tensor DY not set");
  CHECK_ERROR(wnode([](auto &a) { a.setX(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvWGrad input tensor X not set");
  CHECK_ERROR(wnode([](auto &a) { a.setDW(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvWGrad output tensor DW not set");
  CHECK_ERROR(dnode([](auto &a) { a.setPadding(Dims{}); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvDGrad padding not set");
  CHECK_ERROR(dnode([](auto &a) { a.setDY(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvDGrad gradient tensor DY not set");
  CHECK_ERROR(dnode([](auto &a) { a.setW(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvDGrad input tensor W not set");
  CHECK_ERROR(dnode([](auto &a) { a.setDX(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "ConvDGrad output tensor DX not set");
  // ranks
  CHECK_ERROR(wnode([&](auto &a) {
                a.setDY(std::make_shared<TensorAttr>(mk("DY", {n, k}, {k, 1})));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvWGrad input tensors DY/X must have a rank of at least 3");
  CHECK_ERROR(wnode([&](auto &a) {
                a.setX(std::make_shared<TensorAttr>(
                    mk("X", {n, c, 2, h, w}, contig({n, c, 2, h, w}))));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvWGrad tensors DY and X have different ranks");
  CHECK_ERROR(wnode([](auto &a) { a.setStride({1}); }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvWGrad stride size does not match number of spatial dimensions");
  CHECK_ERROR(dnode([](auto &a) { a.setDilation({1, 1, 1}); }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvDGrad dilation size does not match number of spatial "
              "dimensions");
  CHECK_ERROR(dnode([&](auto &a) {
                a.setW(std::make_shared<TensorAttr>(mk("W", {k, c}, {c, 1})));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvDGrad input tensors DY/W must have a rank of at least 3");
  // layouts
  CHECK_ERROR(wnode([&](auto &a) {
                a.setX(std::make_shared<TensorAttr>(
                    mk("X", {n, c, h, w}, {c * h * w, w, 1, h})));
              }).preValidateNode(),
              ErrorCode::NotImplemented,
              "Tensor 'X' is neither contiguous nor channels-last as defined "
              "by its stride");
  // group counts
  CHECK_ERROR(wnode([&](auto &a) {
                a.setDW(std::make_shared<TensorAttr>(
                    mk("DW", {k, 7, 1, 1}, contig({k, 7, 1, 1}))));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvWGrad input (X) channels must be divisible by the filter "
              "(W) channels");
  CHECK_ERROR(dnode([&](auto &a) {
                a.setW(std::make_shared<TensorAttr>(
                    mk("W", {k, 7, 1, 1}, contig({k, 7, 1, 1}))));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvDGrad input (DX) channels must be divisible by the filter "
              "(W) channels");
  CHECK_ERROR(dnode([&](auto &a) {
                // 256 / 1 = 256 groups > 128 output channels
                a.setW(std::make_shared<TensorAttr>(
                    mk("W", {k, 1, 1, 1}, contig({k, 1, 1, 1}))));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "ConvDGrad group count must be greater than 0 and less than or "
              "equal to the numbers of input and outputs channels");
  // post-validation: rank and shape agreement
  {
    auto node = wnode([&](auto &a) {
      a.setDW(std::make_shared<TensorAttr>(mk("DW", {k, c}, {c, 1})));
    });
    REQUIRE_OK(node.preValidateNode());
    REQUIRE_OK(node.inferPropertiesNode());
    CHECK_ERROR(node.postValidateNode(), ErrorCode::InvalidAttribute,
                "ConvWGrad weight gradient tensor DW must have a rank of at "
                "least 3");
  }
  {
    auto node = wnode([&](auto &a) { // {c, k, r, s} instead of {k, c, r, s}
      a.setDW(std::make_shared<TensorAttr>(
          mk("DW", {c, k, 1, 1}, contig({c, k, 1, 1}))));
    });
    REQUIRE_OK(node.preValidateNode());
    REQUIRE_OK(node.inferPropertiesNode());
    CHECK_ERROR(node.postValidateNode(), ErrorCode::InvalidAttribute,
                "ConvWGrad output DW dimensions do not match the expected "
                "shapes inferred based on input dimensions");
  }
  {
    auto node = dnode([&](auto &a) {
      a.setW(std::make_shared<TensorAttr>(
          mk("W", {c, k, 1, 1}, contig({c, k, 1, 1}))));
    });
    REQUIRE_OK(node.preValidateNode());
    REQUIRE_OK(node.inferPropertiesNode());
    CHECK_ERROR(node.postValidateNode(), ErrorCode::InvalidAttribute,
                "ConvDGrad DY dimensions do not match the expected shapes "
                "inferred based on DX and W");
  }
  {
    auto node = dnode([&](auto &a) {
      a.setPadding({0, 0, 0}).setStride({1, 1, 1}).setDilation({1, 1, 1});
      a.setDY(std::make_shared<TensorAttr>(
          mk("DY", {n, k, 2, h, w}, contig({n, k, 2, h, w}))));
    });
    REQUIRE_OK(node.preValidateNode());
    CHECK_ERROR(node.postValidateNode(), ErrorCode::InvalidAttribute,
                "ConvDGrad tensors DY and DX have different ranks");
  }
}

TEST("matmul node: inference and errors") {
  {
    Graph g = newGraph("mm");
    auto a = g.tensor(mk("a", {16, 16, 32, 64}, contig({16, 16, 32, 64})));
    auto b = g.tensor(mk("b", {1, 1, 64, 128}, contig({1, 1, 64, 128})));
    MatmulAttr m;
    auto c = g.matmul(a, b, m);
    c->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK((c->getDim() == Dims{16, 16, 32, 128}));
    CHECK(c->isContiguous());
    CHECK(c->getName() == "matmul_0_C");
  }
  auto build = [](Dims ad, Dims as, Dims bd, Dims bs,
                  DataType bdt = DataType::Float) {
    Graph g = newGraph("mm_err");
    auto a = g.tensor(mk("a", ad, as));
    auto b = g.tensor(mk("b", bd, bs, bdt));
    MatmulAttr m;
    auto c = g.matmul(a, b, m);
    c->setOutput(true);
    return g.validate();
  };
  CHECK_ERROR(build({4}, {1}, {4, 4}, {4, 1}), ErrorCode::InvalidAttribute,
              "Matmul input tensor A must have a rank of at least 2");
  CHECK_ERROR(build({2, 4, 4}, {16, 4, 1}, {4, 4}, {4, 1}),
              ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B must have the same rank: A has "
              "rank=3, B has rank=2");
  CHECK_ERROR(build({4, 8}, {8, 1}, {7, 4}, {4, 1}),
              ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B have incompatible inner "
              "dimensions (K): A has K=8, B has K=7");
  CHECK_ERROR(build({3, 4, 8}, {32, 8, 1}, {2, 8, 4}, {32, 4, 1}),
              ErrorCode::InvalidAttribute,
              "Matmul input tensors A and B have incompatible batch dimensions "
              "for broadcasting at index 0: A has dim=3, B has dim=2");
  CHECK_ERROR(build({2, 4, 8}, {8, 16, 1}, {2, 8, 4}, {32, 4, 1}),
              ErrorCode::InvalidAttribute,
              "Matmul tensor A has batch dimensions that are not outermost or "
              "are transposed");
  CHECK_ERROR(build({4, 8}, {8, 1}, {8, 4}, {4, 1}, DataType::Half),
              ErrorCode::InvalidAttribute,
              "Mixed precision matmul is only supported when input tensors A "
              "and B are of rank 3 (single batch dim): A and B have rank=2");
}

TEST("pointwise node: inference and errors") {
  {
    Graph g = newGraph("pw");
    auto a = g.tensor(mk("a", {3, 1, 8}, contig({3, 1, 8})));
    auto b = g.tensor(mk("b", {5, 8}, contig({5, 8})));
    PointwiseAttr p;
    p.setMode(PointwiseAttr::Mode::CMP_LT);
    auto o = g.pointwise(a, b, p);
    o->setOutput(true).setStride(contig({3, 5, 8}));
    REQUIRE_OK(g.validate());
    CHECK((o->getDim() == Dims{3, 5, 8}));
    CHECK(o->getDataType() == DataType::Boolean); // forced
    CHECK(o->getName() == "pointwise_0_OUT_0");
  }
  {
    Graph g = newGraph("pw_stride");
    auto a = g.tensor(mk("a", {2, 3, 4, 5}, chlast({2, 3, 4, 5})));
    PointwiseAttr p;
    p.setMode(PointwiseAttr::Mode::RELU_FWD);
    auto o = g.pointwise(a, p);
    o->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK((o->getStride() == chlast({2, 3, 4, 5}))); // inherits IN_0
  }
  {
    Graph g = newGraph("pw_err");
    auto a = g.tensor(mk("a", {4}, {1}));
    PointwiseAttr p;
    auto o = g.pointwise(a, p);
    o->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::AttributeNotSet,
                "Pointwise mode not set");
  }
  {
    Graph g = newGraph("pw_err2");
    auto a = g.tensor(mk("a", {4}, {1}));
    PointwiseAttr p;
    p.setMode(PointwiseAttr::Mode::ADD);
    auto o = g.pointwise(a, p);
    o->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::AttributeNotSet,
                "ADD mode requires IN_1 input");
  }
  {
    Graph g = newGraph("pw_err3");
    auto a = g.tensor(mk("a", {4}, {1}));
    auto b = g.tensor(mk("b", {4}, {1}));
    PointwiseAttr p;
    p.setMode(PointwiseAttr::Mode::RELU_FWD);
    auto o = g.pointwise(a, b, p);
    o->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::InvalidAttribute,
                "RELU_FWD mode should not have IN_1 input set");
  }
}

TEST("reduction node: inference and errors") {
  auto build = [](Dims ydim, ReductionAttr::Mode mode, DataType dt) {
    Graph g = newGraph("red", dt);
    auto x = g.tensor(mk("x", {2, 16, 8, 8}, contig({2, 16, 8, 8}), dt));
    ReductionAttr r;
    r.setMode(mode);
    auto y = g.reduction(x, r);
    y->setOutput(true);
    if (!ydim.empty())
      y->setDim(ydim);
    return g.validate();
  };
  CHECK(isOk(build({2, 16, 1, 1}, ReductionAttr::Mode::SUM, DataType::Float)));
  CHECK_ERROR(build({2, 16, 1, 1}, ReductionAttr::Mode::NOT_SET, DataType::Float),
              ErrorCode::AttributeNotSet, "Reduction mode not set");
  CHECK_ERROR(build({2, 16, 1}, ReductionAttr::Mode::SUM, DataType::Float),
              ErrorCode::InvalidAttribute,
              "Reduction input and output must have the same rank");
  CHECK_ERROR(build({2, 16, 1, 1}, ReductionAttr::Mode::AVG, DataType::Int32),
              ErrorCode::InvalidAttribute,
              "Reduction AVG is not supported for integral or boolean tensors");
  CHECK_ERROR(build({2, 16, 4, 1}, ReductionAttr::Mode::SUM, DataType::Float),
              ErrorCode::InvalidAttribute,
              "Reduction output dimension 2 must be 1 or match input dimension");
  CHECK_ERROR(build({}, ReductionAttr::Mode::SUM, DataType::Float),
              ErrorCode::InvalidAttribute,
              "Reduction requires at least one dimension to reduce (Y[i] == 1 "
              "where X[i] > 1)");
}

TEST("sdpa node: inference and errors") {
  auto build = [](Dims kd, bool gqa, bool causal, bool mask, float dropout,
                  Dims maskDim = {1, 1, 64, 64}) {
    Graph g = newGraph("sdpa", DataType::Half);
    auto q = g.tensor(mk("q", {1, 8, 64, 64}, contig({1, 8, 64, 64}), DataType::Half));
    auto k = g.tensor(mk("k", kd, contig(kd), DataType::Half));
    auto v = g.tensor(mk("v", kd, contig(kd), DataType::Half));
    std::shared_ptr<TensorAttr> m;
    if (mask)
      m = g.tensor(mk("m", maskDim, contig(maskDim), DataType::Half));
    SdpaAttr a;
    a.setEnableGqa(gqa).setIsCausal(causal).setDropout(dropout);
    auto o = g.sdpa(q, k, v, m, a);
    o->setOutput(true);
    auto st = g.validate();
    if (isOk(st)) {
      if (o->getDim() != Dims{1, 8, 64, 64} || !o->isContiguous() ||
          o->getName() != "sdpa_0_O")
        return error(ErrorCode::InternalError, "bad inferred output");
    }
    return st;
  };
  CHECK(isOk(build({1, 8, 64, 64}, false, true, false, 0.f)));
  CHECK(isOk(build({1, 2, 64, 64}, true, false, true, 0.f)));
  CHECK_ERROR(build({1, 2, 64, 64}, false, false, false, 0.f),
              ErrorCode::InvalidAttribute,
              "SDPA without GQA requires Q heads (8) to equal K heads (2)");
  CHECK_ERROR(build({1, 3, 64, 64}, true, false, false, 0.f),
              ErrorCode::InvalidAttribute,
              "SDPA with GQA requires Q heads (8) to be a multiple of K heads "
              "(3)");
  CHECK_ERROR(build({1, 8, 64, 64}, false, true, true, 0.f),
              ErrorCode::InvalidAttribute,
              "SDPA attention mask and is_causal are mutually exclusive");
  CHECK_ERROR(build({1, 8, 64, 64}, false, false, true, 0.f, {1, 1, 32, 64}),
              ErrorCode::InvalidAttribute,
              "SDPA attention mask seq_q dim (32) must be 1 or match Q "
              "sequence length (64)");
  CHECK_ERROR(build({1, 8, 64, 64}, false, false, false, 1.0f),
              ErrorCode::InvalidAttribute,
              "SDPA dropout probability must be in [0, 1)");
  CHECK_ERROR(build({1, 8, 64, 32}, false, false, false, 0.f),
              ErrorCode::InvalidAttribute,
              "SDPA input tensors Q and K must have matching head_dim");
}

TEST("norm nodes: inference and errors") {
  {
    Graph g = newGraph("rms");
    auto x = g.tensor(mk("x", {2, 3, 32, 32}, chlast({2, 3, 32, 32})));
    auto s = g.tensor(TensorAttr().setName("s").setDataType(DataType::Float));
    RmsnormAttr a;
    a.setForwardPhase(NormFwdPhase::INFERENCE)
        .setEpsilon(g.tensor(TensorAttr(1e-5f)));
    auto [y, r] = g.rmsnorm(x, s, a);
    y->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK(r == nullptr);
    CHECK((s->getDim() == Dims{1, 3, 32, 32}));
    CHECK((s->getStride() == chlast({1, 3, 32, 32}))); // follows X's format
    CHECK((y->getStride() == x->getStride()));
    CHECK(y->getName() == "rmsnorm_0_Y");
  }
  {
    Graph g = newGraph("rms_train");
    auto x = g.tensor(mk("x", {2, 8}, {8, 1}));
    RmsnormAttr a;
    a.setForwardPhase(NormFwdPhase::TRAINING)
        .setEpsilon(g.tensor(TensorAttr(1e-5f)));
    auto [y, r] = g.rmsnorm(x, nullptr, a);
    y->setOutput(true);
    r->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::NotImplemented,
                "RmsNorm training mode is not yet supported: torch-mlir does "
                "not lower the training variant");
  }
  {
    Graph g = newGraph("rms_err");
    auto x = g.tensor(mk("x", {2, 8}, {8, 1}));
    RmsnormAttr a;
    a.setForwardPhase(NormFwdPhase::INFERENCE);
    auto [y, r] = g.rmsnorm(x, nullptr, a);
    y->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::AttributeNotSet,
                "RmsNorm epsilon not set");
  }
  {
    Graph g = newGraph("ln_train");
    auto x = g.tensor(mk("x", {4, 3, 8, 8}, contig({4, 3, 8, 8})));
    auto s = g.tensor(mk("s", {1, 3, 8, 8}, contig({1, 3, 8, 8})));
    auto b = g.tensor(mk("b", {1, 3, 8, 8}, contig({1, 3, 8, 8})));
    LayernormAttr a;
    a.setForwardPhase(NormFwdPhase::TRAINING)
        .setEpsilon(g.tensor(TensorAttr(1e-5f)));
    auto [y, m, v] = g.layernorm(x, s, b, a);
    y->setOutput(true);
    m->setOutput(true);
    v->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK((m->getDim() == Dims{4, 1, 1, 1}));
    CHECK((v->getStride() == Dims{1, 1, 1, 1}));
    CHECK(m->getName() == "layernorm_0_MEAN" &&
          v->getName() == "layernorm_0_INV_VARIANCE");
  }
  {
    Graph g = newGraph("ln_err");
    auto x = g.tensor(mk("x", {4, 3, 8, 8}, contig({4, 3, 8, 8})));
    auto s = g.tensor(mk("s", {1, 3, 8, 4}, contig({1, 3, 8, 4})));
    LayernormAttr a;
    a.setForwardPhase(NormFwdPhase::INFERENCE)
        .setEpsilon(g.tensor(TensorAttr(1e-5f)));
    auto [y, m, v] = g.layernorm(x, s, nullptr, a);
    y->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::InvalidAttribute,
                "LayerNorm input tensor SCALE must have shape as tensor X with "
                "single batch");
  }
}

// ---- graph state machine ----------------------------------------------------
struct ConvGraph {
  std::unique_ptr<Graph> graph;
  std::shared_ptr<TensorAttr> x, w, y;
};
// The reference's executable test graph: all-ones f16 1x1 conv, C = 128
// (tests/test_graph.cpp:198-223).
static ConvGraph makeConvGraph(const std::string &name) {
  ConvGraph c;
  c.graph = std::make_unique<Graph>();
  c.graph->setName(name).setIODataType(DataType::Half)
      .setComputeDataType(DataType::Float);
  c.x = c.graph->tensor(mk("image", {16, 128, 64, 64},
                           contig({16, 128, 64, 64}), DataType::Half));
  c.w = c.graph->tensor(mk("filter", {256, 128, 1, 1},
                           contig({256, 128, 1, 1}), DataType::Half));
  ConvFPropAttr a;
  a.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1}).setName("conv_fprop");
  c.y = c.graph->convFProp(c.x, c.w, a);
  c.y->setOutput(true);
  return c;
}

TEST("batchnorm node: inference and errors") {
  // tests/test_batchnorm_node.cpp of the reference
  const Dims xd = {2, 4, 8, 8};
  {
    Graph g = newGraph("bn_train");
    auto x = g.tensor(mk("x", xd, chlast(xd)));
    BatchnormAttr a;
    a.setForwardPhase(NormFwdPhase::TRAINING)
        .setEpsilon(g.tensor(TensorAttr(1e-5f)))
        .setMomentum(g.tensor(TensorAttr(0.1f)));
    auto scale = g.tensor(TensorAttr().setName("scale").setDataType(DataType::Float));
    auto [y, m, v] = g.batchnorm(x, scale, nullptr, nullptr, nullptr, a);
    y->setOutput(true);
    m->setOutput(true);
    v->setOutput(true);
    REQUIRE_OK(g.validate());
    CHECK(y->getName() == "batchnorm_0_Y");
    CHECK(m->getName() == "batchnorm_0_SAVED_MEAN");
    CHECK(v->getName() == "batchnorm_0_SAVED_INV_VARIANCE");
    CHECK((y->getDim() == xd));
    CHECK((y->getStride() == chlast(xd))); // follows X
    CHECK((scale->getDim() == Dims{4}));
    CHECK((scale->getStride() == Dims{1}));
    CHECK((m->getDim() == Dims{4}));
    CHECK((v->getStride() == Dims{1}));
  }
  {
    Graph g = newGraph("bn_infer");
    auto x = g.tensor(mk("x", xd, contig(xd)));
    auto mean = g.tensor(mk("mean", {4}, {1}));
    auto var = g.tensor(mk("var", {4}, {1}));
    BatchnormAttr a;
    a.setForwardPhase(NormFwdPhase::INFERENCE)
        .setEpsilon(g.tensor(TensorAttr(1e-5f)))
        .setMomentum(g.tensor(TensorAttr(0.1f)));
    auto [y, m, v] = g.batchnorm(x, nullptr, nullptr, mean, var, a);
    y->setOutput(true);
    CHECK(m == nullptr);
    CHECK(v == nullptr);
    REQUIRE_OK(g.validate());
    CHECK(y->isContiguous());
  }
  Context ctx;
  auto T = [](const char *name, Dims d, Dims st) {
    return std::make_shared<TensorAttr>(mk(name, d, st));
  };
  auto S = [](float v) { return std::make_shared<TensorAttr>(TensorAttr(v)); };
  auto node = [&](bool training, auto &&tweak) {
    BatchnormAttr a;
    a.setForwardPhase(training ? NormFwdPhase::TRAINING : NormFwdPhase::INFERENCE)
        .setEpsilon(S(1e-5f)).setMomentum(S(0.1f));
    a.setX(T("X", xd, contig(xd))).setY(T("Y", xd, contig(xd)));
    if (training)
      a.setSAVED_MEAN(T("SM", {4}, {1})).setSAVED_INV_VARIANCE(T("SV", {4}, {1}));
    else
      a.setMEAN(T("MEAN", {4}, {1})).setVAR(T("VAR", {4}, {1}));
    tweak(a);
    return BatchNormNode(std::move(a), ctx);
  };
  REQUIRE_OK(node(false, [](auto &) {}).preValidateNode());
  REQUIRE_OK(node(true, [](auto &) {}).preValidateNode());
  CHECK_ERROR(node(false, [](auto &a) {
                a.setForwardPhase(NormFwdPhase::NOT_SET);
              }).preValidateNode(),
              ErrorCode::AttributeNotSet, "BatchNorm forward phase not set");
  CHECK_ERROR(node(false, [](auto &a) { a.setX(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "BatchNorm input tensor X not set");
  CHECK_ERROR(node(false, [](auto &a) { a.setY(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "BatchNorm output tensor Y not set");
  CHECK_ERROR(node(false, [](auto &a) { a.setEpsilon(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "BatchNorm epsilon not set");
  CHECK_ERROR(node(false, [](auto &a) { a.setMomentum(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet, "BatchNorm momentum not set");
  CHECK_ERROR(node(false, [&](auto &a) {
                a.setEpsilon(T("eps", {1}, {1}));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "BatchNorm epsilon must be a scalar constant");
  CHECK_ERROR(node(false, [&](auto &a) {
                a.setMomentum(T("mom", {1}, {1}));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "BatchNorm momentum must be a scalar constant");
  CHECK_ERROR(node(false, [&](auto &a) { a.setX(T("X", {8}, {1})); }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "BatchNorm input tensor X must have a rank of at least 2");
  CHECK_ERROR(node(false, [&](auto &a) {
                a.setX(T("X", xd, {256, 8, 1, 64}));
              }).preValidateNode(),
              ErrorCode::NotImplemented,
              "Tensor 'X' is neither contiguous nor channels-last as defined "
              "by its stride");
  CHECK_ERROR(node(false, [](auto &a) { a.setMEAN(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet,
              "BatchNorm inference requires running MEAN");
  CHECK_ERROR(node(false, [](auto &a) { a.setVAR(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet,
              "BatchNorm inference requires running VAR");
  CHECK_ERROR(node(false, [&](auto &a) {
                a.setSAVED_MEAN(T("SM", {4}, {1}));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "BatchNorm SAVED_MEAN should not be set in inference mode");
  CHECK_ERROR(node(false, [&](auto &a) {
                a.setSAVED_INV_VARIANCE(T("SV", {4}, {1}));
              }).preValidateNode(),
              ErrorCode::InvalidAttribute,
              "BatchNorm SAVED_INV_VARIANCE should not be set in inference mode");
  CHECK_ERROR(node(true, [](auto &a) { a.setSAVED_MEAN(nullptr); }).preValidateNode(),
              ErrorCode::AttributeNotSet,
              "BatchNorm training requires SAVED_MEAN output");
  CHECK_ERROR(node(true, [](auto &a) {
                a.setSAVED_INV_VARIANCE(nullptr);
              }).preValidateNode(),
              ErrorCode::AttributeNotSet,
              "BatchNorm training requires SAVED_INV_VARIANCE output");
  // post-validation
  auto post = [&](bool training, auto &&tweak) {
    auto n = node(training, tweak);
    ErrorObject e = n.preValidateNode();
    if (isOk(e))
      e = n.inferPropertiesNode();
    return isOk(e) ? n.postValidateNode() : e;
  };
  REQUIRE_OK(post(false, [](auto &) {}));
  CHECK_ERROR(post(false, [&](auto &a) {
                a.setY(T("Y", {2, 4, 8, 7}, contig({2, 4, 8, 7})));
              }),
              ErrorCode::InvalidAttribute,
              "BatchNorm output Y tensor must have the same shape as input X "
              "tensor");
  CHECK_ERROR(post(false, [&](auto &a) { a.setY(T("Y", xd, {256, 8, 1, 64})); }),
              ErrorCode::NotImplemented,
              "Tensor 'Y' is neither contiguous nor channels-last as defined "
              "by its stride");
  CHECK_ERROR(post(false, [&](auto &a) { a.setSCALE(T("S", {5}, {1})); }),
              ErrorCode::InvalidAttribute,
              "BatchNorm tensor SCALE must be 1D with size equal to channel "
              "dimension C");
  CHECK_ERROR(post(false, [&](auto &a) { a.setBIAS(T("B", {1, 4}, {4, 1})); }),
              ErrorCode::InvalidAttribute,
              "BatchNorm tensor BIAS must be 1D with size equal to channel "
              "dimension C");
  CHECK_ERROR(post(false, [&](auto &a) { a.setVAR(T("VAR", {4}, {2})); }),
              ErrorCode::InvalidAttribute,
              "BatchNorm tensor VAR must have unit stride");
  CHECK_ERROR(post(true, [&](auto &a) { a.setSAVED_MEAN(T("SM", {8}, {1})); }),
              ErrorCode::InvalidAttribute,
              "BatchNorm tensor SAVED_MEAN must be 1D with size equal to "
              "channel dimension C");
}

TEST("graph: name, symbol uniqueness, broadcast outputs") {
  {
    Graph g;
    CHECK_ERROR(g.validate(), ErrorCode::AttributeNotSet, "Graph name not set");
  }
  {
    Graph g = newGraph("dup");
    auto a = g.tensor(mk("t", {4}, {1}));
    auto b = g.tensor(mk("t", {4}, {1}));
    PointwiseAttr p;
    p.setMode(PointwiseAttr::Mode::ADD);
    auto o = g.pointwise(a, b, p);
    o->setOutput(true);
    CHECK_ERROR(g.validate(), ErrorCode::InvalidAttribute,
                "Symbol name 't' already in use");
  }
  {
    Graph g = newGraph("dupnode");
    auto a = g.tensor(mk("a", {4}, {1}));
    PointwiseAttr p1, p2;
    p1.setMode(PointwiseAttr::Mode::RELU_FWD).setName("same");
    p2.setMode(PointwiseAttr::Mode::RELU_FWD).setName("same");
    auto m = g.pointwise(a, p1);
    auto o = g.pointwise(m, p2);
    o->setOutput(true);
    auto st = g.validate();
    CHECK(st.getCode() == ErrorCode::InvalidAttribute);
  }
  {
    Graph g = newGraph("bcast_out");
    auto a = g.tensor(mk("a", {4, 8}, {8, 1}));
    PointwiseAttr p;
    p.setMode(PointwiseAttr::Mode::RELU_FWD);
    auto o = g.pointwise(a, p);
    o->setOutput(true).setDim({4, 8}).setStride({0, 1});
    CHECK_ERROR(g.validate(), ErrorCode::InvalidAttribute,
                "Tensor 'pointwise_0_OUT_0' has broadcast strides (stride=0) "
                "on an operation output, which is not yet supported");
  }
}

TEST("graph: compile/execute preconditions") {
  auto c = makeConvGraph("preconditions");
  auto art = c.graph->compileToArtifact(Backend::AMDGPU);
  CHECK_ERROR(ErrorObject(art), ErrorCode::NotValidated,
              "Graph must be validated before being compiled");
  REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
  CHECK_ERROR(c.graph->loadFromArtifact(cpu, std::vector<uint8_t>{1, 2, 3}),
              ErrorCode::NotValidated,
              "Graph must be validated before loading a compiled artifact");
  REQUIRE_OK(c.graph->validate());
  REQUIRE_ASSIGN(auto ws0, c.graph->getWorkspaceSize());
  CHECK(!ws0.has_value()); // nothing loaded yet
  std::unordered_map<std::shared_ptr<TensorAttr>, std::shared_ptr<Buffer>> pack;
  auto st = c.graph->execute(cpu, pack, nullptr);
  CHECK(st.getCode() == ErrorCode::NotCompiled);

  REQUIRE_OK(c.graph->compile(cpu, /*remove=*/true));
  CHECK(c.graph->getKernelCount() == std::optional<size_t>(1));
  CHECK_ERROR(c.graph->execute(cpu, pack, nullptr), ErrorCode::InvalidArgument,
              "Graph::execute requires getWorkspaceSize() to be called before "
              "workspace allocation and execution");
  REQUIRE_ASSIGN(auto ws, c.graph->getWorkspaceSize());
  REQUIRE(ws.has_value());
  CHECK(*ws == 0);
  CHECK_ERROR(c.graph->execute(cpu, pack, nullptr), ErrorCode::VariantPackError,
              "Output tensor missing from variantPack");

  auto bufOf = [&](const std::shared_ptr<TensorAttr> &t) {
    size_t n = static_cast<size_t>(t->getVolume());
    auto b = Buffer::allocate(cpu, {n}, std::vector<half>(n, half(1.0f)));
    return std::make_shared<Buffer>(std::move(*b));
  };
  pack[c.y] = bufOf(c.y);
  CHECK_ERROR(c.graph->execute(cpu, pack, nullptr), ErrorCode::VariantPackError,
              "Input tensor missing from variantPack");
  pack[c.x] = bufOf(c.x);
  pack[c.w] = bufOf(c.w);
  // Everything is in order; only the missing execution engine stops it.
  auto run = c.graph->execute(cpu, pack, nullptr);
  CHECK(run.getCode() == ErrorCode::NotImplemented);
  // A buffer that is too small is caught before any launch.
  auto small = Buffer::allocate(cpu, {8}, std::vector<half>(8, half(0.f)));
  pack[c.y] = std::make_shared<Buffer>(std::move(*small));
  CHECK(c.graph->execute(cpu, pack, nullptr).getCode() ==
        ErrorCode::VariantPackError);
}

TEST("graph: virtual and scalar tensors must stay out of the variant pack") {
  Graph g = newGraph("pack_rules");
  auto a = g.tensor(mk("a", {2, 5}, {5, 1}));
  auto two = g.tensor(TensorAttr(2.0f).setName("two"));
  PointwiseAttr p1, p2;
  p1.setMode(PointwiseAttr::Mode::MUL);
  p2.setMode(PointwiseAttr::Mode::RELU_FWD);
  auto mid = g.pointwise(a, two, p1); // stays virtual
  auto out = g.pointwise(mid, p2);
  out->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
  REQUIRE_OK(g.compile(cpu, /*remove=*/true));
  REQUIRE_ASSIGN(auto ws, g.getWorkspaceSize());
  REQUIRE(ws.has_value());
  CHECK(*ws >= 2 * 5 * 4); // the virtual tensor between the two kernels
  CHECK(g.getKernelCount() == std::optional<size_t>(2));
  auto buf = [&] {
    auto b = Buffer::allocate(cpu, {10}, std::vector<float>(10, 1.f));
    return std::make_shared<Buffer>(std::move(*b));
  };
  auto wsBuf = std::make_shared<Buffer>(std::move(*Buffer::allocateRaw(cpu, *ws)));
  std::unordered_map<std::shared_ptr<TensorAttr>, std::shared_ptr<Buffer>> pack =
      {{a, buf()}, {out, buf()}, {mid, buf()}};
  CHECK_ERROR(g.execute(cpu, pack, wsBuf), ErrorCode::VariantPackError,
              "Virtual output tensor found in variantPack");
  pack.erase(mid);
  pack[two] = buf();
  CHECK_ERROR(g.execute(cpu, pack, wsBuf), ErrorCode::VariantPackError,
              "Scalar constant tensor found in variantPack");
  pack.erase(two);
  CHECK_ERROR(g.execute(cpu, pack, nullptr), ErrorCode::InvalidArgument,
              "Workspace buffer required but not provided (size=" +
                  std::to_string(*ws) + " bytes)");
  auto tiny = std::make_shared<Buffer>(std::move(*Buffer::allocateRaw(cpu, 8)));
  CHECK_ERROR(g.execute(cpu, pack, tiny), ErrorCode::InvalidArgument,
              "Workspace buffer too small: provided 8 bytes, required " +
                  std::to_string(*ws) + " bytes");
}

TEST("graph: artifact contract") {
  REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
  auto consumer = makeConvGraph("aot_consumer");
  REQUIRE_OK(consumer.graph->validate());
  std::vector<uint8_t> bytes;
  {
    auto producer = makeConvGraph("aot_producer");
    REQUIRE_OK(producer.graph->validate());
    REQUIRE_ASSIGN(bytes, producer.graph->compileToArtifact(Backend::CPU, /*remove=*/true));
  }
  CHECK(!bytes.empty());
  // another instance's artifact loads into an identically built graph
  REQUIRE_OK(consumer.graph->loadFromArtifact(cpu, bytes));
  REQUIRE_ASSIGN(auto ws, consumer.graph->getWorkspaceSize());
  CHECK(ws.has_value());
  // compileToArtifact for another backend leaves the loaded state alone
  REQUIRE_ASSIGN(auto other, consumer.graph->compileToArtifact(Backend::AMDGPU, /*remove=*/true));
  CHECK(!other.empty());
  REQUIRE_ASSIGN(auto ws2, consumer.graph->getWorkspaceSize());
  CHECK(ws2.has_value());
  // wrong backend for this handle
  CHECK(consumer.graph->loadFromArtifact(cpu, other).getCode() ==
        ErrorCode::RuntimeFailure);
  REQUIRE_ASSIGN(auto cleared0, consumer.graph->getWorkspaceSize());
  CHECK(!cleared0.has_value());
  // garbage bytes fail and clear the loaded state
  REQUIRE_OK(consumer.graph->loadFromArtifact(cpu, bytes));
  auto st = consumer.graph->loadFromArtifact(
      cpu, std::vector<uint8_t>{0xde, 0xad, 0xbe, 0xef});
  CHECK(isError(st));
  REQUIRE_ASSIGN(auto cleared, consumer.graph->getWorkspaceSize());
  CHECK(!cleared.has_value());
  // a flipped byte is caught by the checksum
  auto corrupt = bytes;
  corrupt[corrupt.size() / 2] ^= 0x40;
  CHECK(isError(consumer.graph->loadFromArtifact(cpu, corrupt)));
  // an edited artifact whose checksum was recomputed (same header, same
  // signature field, one byte of a step changed) is not executed either
  {
    auto edited = bytes;
    edited[16 + 8 * 8 + 40] ^= 0x01; // inside the first step
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i + 8 < edited.size(); ++i)
      h = (h ^ edited[i]) * 1099511628211ull;
    std::memcpy(edited.data() + edited.size() - 8, &h, 8);
    CHECK_ERROR(consumer.graph->loadFromArtifact(cpu, edited),
                ErrorCode::RuntimeFailure,
                "Artifact does not match the plan of this graph (stale or "
                "edited artifact)");
    // counts that would wrap the length computation
    auto huge = bytes;
    const uint64_t big = ~0ull / 8;
    std::memcpy(huge.data() + 16 + 5 * 8, &big, 8); // nSteps
    h = 1469598103934665603ull;
    for (size_t i = 0; i + 8 < huge.size(); ++i)
      h = (h ^ huge[i]) * 1099511628211ull;
    std::memcpy(huge.data() + huge.size() - 8, &h, 8);
    CHECK_ERROR(consumer.graph->loadFromArtifact(cpu, huge),
                ErrorCode::RuntimeFailure,
                "Artifact length does not match its header");
  }
  // an artifact of a different graph is rejected
  Graph g = newGraph("different");
  auto a = g.tensor(mk("a", {4, 4}, {4, 1}));
  PointwiseAttr p;
  p.setMode(PointwiseAttr::Mode::RELU_FWD);
  auto o = g.pointwise(a, p);
  o->setOutput(true);
  REQUIRE_OK(g.validate());
  CHECK_ERROR(g.loadFromArtifact(cpu, bytes), ErrorCode::RuntimeFailure,
              "Artifact does not match this graph (signature mismatch)");
}

TEST("cache: files, RAII removal, hit and miss") {
  namespace fs = std::filesystem;
  // files live under ${FUSILLI_CACHE_DIR}/.cache/fusilli/<graph>/<file>
  const fs::path dir = CacheFile::getCacheDir();
  CHECK(dir.filename() == "fusilli");
  CHECK(CacheFile::getPath("g", "f") == dir / "g" / "f");
  // a name cannot leave the cache directory
  CHECK(CacheFile::getPath("../x/y", "f") == dir / ".._x_y" / "f");
  {
    REQUIRE_ASSIGN(CacheFile kept, CacheFile::create("cache_case", "kept", false));
    {
      REQUIRE_ASSIGN(CacheFile temp, CacheFile::create("cache_case", "temp", true));
      REQUIRE_OK(temp.write(std::string("abc")));
      REQUIRE_ASSIGN(std::string back, temp.read());
      CHECK(back == "abc");
      REQUIRE_ASSIGN(CacheFile again, CacheFile::open("cache_case", "temp"));
      CHECK(again.path == temp.path);
      // moving hands the removal over
      CacheFile moved = std::move(temp);
      CHECK(fs::exists(moved.path));
    }
    CHECK(!fs::exists(CacheFile::getPath("cache_case", "temp")));
    CHECK(isError(CacheFile::open("cache_case", "temp")));
    CHECK(fs::exists(kept.path)); // remove = false survives its object
    fs::remove(kept.path);
    fs::remove(kept.path.parent_path());
  }

  // the reference's cache test (tests/test_graph.cpp:242-299)
  auto cg = makeConvGraph("cache_graph");
  Graph &g = *cg.graph;
  CHECK_ERROR(g.emitAsm(), ErrorCode::NotValidated,
              "Graph must be validated before being compiled");
  REQUIRE_OK(g.validate());
  REQUIRE_ASSIGN(std::string text, g.emitAsm());
  CHECK(text.find("fusilli.graph @cache_graph") == 0);
  std::optional<bool> re;
  REQUIRE_ASSIGN(fs::path artifact, g.getCompiledArtifact(Backend::CPU, text, true, &re));
  CHECK(re.has_value() && *re); // empty cache: generated
  CHECK(fs::exists(artifact));
  re.reset();
  REQUIRE_OK(g.getCompiledArtifact(Backend::CPU, text, true, &re));
  CHECK(re.has_value() && !*re); // hit
  re.reset();
  REQUIRE_OK(g.getCompiledArtifact(Backend::AMDGPU, text, true, &re));
  CHECK(re.has_value() && *re); // another backend: another planner key
  re.reset();
  REQUIRE_OK(g.getCompiledArtifact(Backend::AMDGPU, text, true, &re));
  CHECK(re.has_value() && !*re);
  re.reset();
  REQUIRE_OK(g.getCompiledArtifact(Backend::CPU, text + " ", true, &re));
  CHECK(re.has_value() && *re); // another description
  re.reset();
  REQUIRE_OK(g.getCompiledArtifact(Backend::CPU, text + " ", true, &re));
  CHECK(re.has_value() && !*re);
  REQUIRE_ASSIGN(std::string cmd, g.readCompilationCacheFile(CachedAssetsType::Command));
  CHECK(cmd.find("--backend=CPU") != std::string::npos);
  REQUIRE_ASSIGN(std::string in, g.readCompilationCacheFile(CachedAssetsType::Input));
  CHECK(in == text + " ");
  // the statistics asset (reference graph/graph.h:449-468): one dispatch for
  // conv + bias + relu, as Graph::getKernelCount reports after compile()
  REQUIRE_ASSIGN(std::string stats, g.readCompilationCacheFile(CachedAssetsType::Statistics));
  CHECK(stats.find("\"dispatch-count\": 1") != std::string::npos);
  CHECK(stats.find("\"workspace-bytes\": 0") != std::string::npos);
  CHECK_ERROR(g.readCompilationCacheFile(static_cast<CachedAssetsType>(99)),
              ErrorCode::InvalidAttribute, "Unknown CachedAssetsType");
  // a deleted file is a miss, not an error of the second kind
  fs::remove(artifact);
  CHECK(isError(g.getCompiledArtifact(Backend::CPU, text + " ", true, &re)));
  const fs::path old_dir = artifact.parent_path();
  g.setName("cache_graph_renamed");
  re.reset();
  REQUIRE_ASSIGN(fs::path artifact2, g.getCompiledArtifact(Backend::CPU, text + " ", true, &re));
  CHECK(re.has_value() && *re); // new name, new paths
  CHECK(artifact2.parent_path() != old_dir);
  CHECK(!fs::exists(old_dir)); // the old files went with their objects

  // compile() goes through the cache; remove = true cleans up with the Graph
  fs::path compiled_dir;
  {
    REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
    auto tmp = makeConvGraph("cache_compile");
    REQUIRE_OK(tmp.graph->validate());
    REQUIRE_OK(tmp.graph->compile(cpu, /*remove=*/true));
    compiled_dir = CacheFile::getPath("cache_compile", kCacheOutputFileName).parent_path();
    CHECK(fs::exists(compiled_dir / kCacheOutputFileName));
    CHECK(fs::exists(compiled_dir / kCacheInputFileName));
    CHECK(fs::exists(compiled_dir / kCacheCommandFileName));
    CHECK(fs::exists(compiled_dir / kCacheStatisticsFileName));
    // the artifact in the cache is what compileToArtifact returns
    REQUIRE_ASSIGN(auto bytes, tmp.graph->compileToArtifact(Backend::CPU, true));
    REQUIRE_ASSIGN(CacheFile f, CacheFile::open("cache_compile", kCacheOutputFileName));
    REQUIRE_ASSIGN(auto disk, f.readBytes());
    CHECK(bytes == disk);
  }
  CHECK(!fs::exists(compiled_dir));
  // remove = false keeps the files
  {
    REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
    auto tmp = makeConvGraph("cache_keep");
    REQUIRE_OK(tmp.graph->validate());
    REQUIRE_OK(tmp.graph->compile(cpu));
  }
  const fs::path keep_dir = CacheFile::getPath("cache_keep", "x").parent_path();
  CHECK(fs::exists(keep_dir / kCacheOutputFileName));
  fs::remove_all(keep_dir);
}

TEST("planner: fusion decisions") {
  REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
  // conv -> add(bias) -> relu fuses into one kernel, no workspace
  // (reference lit stats: tests/lit/test_conv_asm_emitter_nhwc_krsc_with_relu.cpp:103-104)
  {
    Graph g = newGraph("fuse_conv", DataType::BFloat16);
    auto x = g.tensor(mk("x", {32, 64, 56, 56}, chlast({32, 64, 56, 56}), DataType::BFloat16));
    auto w = g.tensor(mk("w", {128, 64, 3, 3}, chlast({128, 64, 3, 3}), DataType::BFloat16));
    auto b = g.tensor(mk("b", {1, 128, 1, 1}, {128, 1, 128, 128}, DataType::BFloat16));
    ConvFPropAttr ca;
    ca.setPadding({1, 1}).setStride({1, 1}).setDilation({1, 1});
    auto y = g.convFProp(x, w, ca);
    PointwiseAttr add, relu;
    add.setMode(PointwiseAttr::Mode::ADD);
    relu.setMode(PointwiseAttr::Mode::RELU_FWD);
    auto t = g.pointwise(y, b, add);
    auto o = g.pointwise(t, relu);
    o->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(cpu, /*remove=*/true));
    CHECK(g.getKernelCount() == std::optional<size_t>(1));
    REQUIRE_ASSIGN(auto ws, g.getWorkspaceSize());
    CHECK(*ws == 0);
  }
  // rmsnorm -> mul(scalar) fuses (benchmark config 2)
  {
    Graph g = newGraph("fuse_rms", DataType::BFloat16);
    auto x = g.tensor(mk("x", {8192, 4096}, {4096, 1}, DataType::BFloat16));
    auto s = g.tensor(mk("s", {1, 4096}, {4096, 1}, DataType::BFloat16));
    RmsnormAttr ra;
    ra.setForwardPhase(NormFwdPhase::INFERENCE).setEpsilon(g.tensor(TensorAttr(1e-6f)));
    auto [y, r] = g.rmsnorm(x, s, ra);
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    auto o = g.pointwise(y, g.tensor(TensorAttr(0.5f)), mul);
    o->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(cpu, /*remove=*/true));
    CHECK(g.getKernelCount() == std::optional<size_t>(1));
  }
  // a virtual tensor with two consumers is not fused away
  {
    Graph g = newGraph("no_fuse");
    auto a = g.tensor(mk("a", {256, 128}, {128, 1}));
    auto b = g.tensor(mk("b", {128, 256}, {256, 1}));
    MatmulAttr m;
    auto c = g.matmul(a, b, m);
    PointwiseAttr p1, p2;
    p1.setMode(PointwiseAttr::Mode::RELU_FWD);
    p2.setMode(PointwiseAttr::Mode::ADD);
    auto r = g.pointwise(c, p1);
    auto o = g.pointwise(r, c, p2); // c is read twice
    o->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(cpu, /*remove=*/true));
    CHECK(g.getKernelCount() == std::optional<size_t>(3));
  }
}

// ---- handle / buffer ----------------------------------------------------------
TEST("handle: CPU rules and concurrent creation") {
  auto h = Handle::create(Backend::CPU, /*deviceId=*/0);
  CHECK_ERROR(ErrorObject(h), ErrorCode::InvalidArgument,
              "Stream can only be set on AMDGPU backend");
  auto h2 = Handle::create(Backend::CPU, 0, 0x1234);
  CHECK_ERROR(ErrorObject(h2), ErrorCode::InvalidArgument,
              "Stream can only be set on AMDGPU backend");
  // tests/test_handle.cpp:47-85: many threads create handles at once
  std::vector<std::thread> threads;
  std::vector<int> ok_(32, 0);
  for (int i = 0; i < 32; ++i)
    threads.emplace_back([&, i] {
      auto hh = Handle::create(Backend::CPU);
      ok_[i] = isOk(hh) && hh->getBackend() == Backend::CPU;
    });
  for (auto &t : threads)
    t.join();
  for (int v : ok_)
    CHECK(v == 1);
}

TEST("buffer: allocate / read / move / errors") {
  REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
  auto zero = Buffer::allocate(cpu, {0}, std::vector<float>{});
  CHECK_ERROR(ErrorObject(zero), ErrorCode::RuntimeFailure,
              "Buffer::allocate failed: cannot allocate a buffer with zero "
              "size");
  auto mism = Buffer::allocate(cpu, {2, 3}, std::vector<float>(5, 0.f));
  CHECK_ERROR(ErrorObject(mism), ErrorCode::RuntimeFailure,
              "Buffer::allocate failed: bufferData size (5) does not match "
              "product of bufferShape dimensions (6)");
  auto raw0 = Buffer::allocateRaw(cpu, 0);
  CHECK_ERROR(ErrorObject(raw0), ErrorCode::RuntimeFailure,
              "Buffer::allocateRaw failed: cannot allocate zero-size buffer");
  auto imp = Buffer::import(nullptr, 16);
  CHECK(ErrorObject(imp).getCode() == ErrorCode::RuntimeFailure);

  std::vector<float> data = {1, 2, 3, 4, 5, 6};
  REQUIRE_ASSIGN(Buffer b, Buffer::allocate(cpu, {2, 3}, data));
  CHECK(b != nullptr);
  std::vector<float> back;
  REQUIRE_OK(b.read(cpu, back));
  CHECK(back == data);
  CHECK_ERROR(b.read(cpu, back), ErrorCode::RuntimeFailure,
              "Buffer::read failed as outData is NOT empty");
  Buffer moved = std::move(b);
  CHECK(b == nullptr);
  CHECK(moved != nullptr);
  std::vector<float> again;
  REQUIRE_OK(moved.read(cpu, again));
  CHECK(again == data);
}

TEST("errors: ErrorOr and macros") {
  auto f = [](bool fail) -> ErrorOr<int> {
    FUSILLI_RETURN_ERROR_IF(fail, ErrorCode::InvalidArgument, "nope");
    return ok(7);
  };
  auto g = [&](bool fail) -> ErrorObject {
    FUSILLI_ASSIGN_OR_RETURN(int v, f(fail));
    FUSILLI_RETURN_ERROR_IF(v != 7, ErrorCode::InternalError, "bad value");
    return ok();
  };
  CHECK(isOk(g(false)));
  CHECK_ERROR(g(true), ErrorCode::InvalidArgument, "nope");
  ErrorOr<std::string> s = ok(std::string("hi"));
  CHECK(*s == "hi" && s->size() == 2);
  std::ostringstream os;
  os << error(ErrorCode::VariantPackError, "msg");
  CHECK(os.str() == "VARIANT_PACK_ERROR: msg");
  CHECK(dataTypeFromAsm("f8E4M3FN") == DataType::FP8E4M3);
  CHECK(std::string(dataTypeAsm(DataType::BFloat16)) == "bf16");
}

int main(int argc, char **argv) { return mini::run(argc, argv); }
