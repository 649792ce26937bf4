// End-to-end tests of the graph API on the GPU: the reference samples' known
// answers (samples/**, tests/test_graph.cpp:551-647) run through
// Graph::validate -> compile -> execute on Backend::AMDGPU, each executed
// twice, plus the benchmark configs at reduced size against plain host loops,
// and HIP interop (caller-owned stream and device pointers,
// tests/hip_tests/test_buffer.cpp:132-206).
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <fusilli.h>

#include <cmath>
#include <random>

#include "mini_test.h"

using namespace fusilli;
using Dims = std::vector<int64_t>;
using Pack = std::unordered_map<std::shared_ptr<TensorAttr>, std::shared_ptr<Buffer>>;

static Dims contig(const Dims &d) {
  return generateStrideFromDim(d, getContiguousStrideOrder(d.size()));
}
static Dims chlast(const Dims &d) {
  return generateStrideFromDim(d, getChannelsLastStrideOrder(d.size()));
}
static TensorAttr mk(const std::string &name, Dims dim, Dims stride, DataType dt) {
  return TensorAttr().setName(name).setDim(dim).setStride(stride).setDataType(dt);
}
static Handle &gpu() {
  static Handle h = [] {
    auto e = Handle::create(Backend::AMDGPU);
    if (isError(e)) {
      std::printf("no AMDGPU handle: %s\n", ErrorObject(e).getMessage().c_str());
      std::exit(2);
    }
    return std::move(*e);
  }();
  return h;
}
// Buffer shaped like the tensor's physical dims (tests/utils.h:144-243).
template <typename T>
static std::shared_ptr<Buffer> bufOf(const std::shared_ptr<TensorAttr> &t,
                                     const std::vector<T> &data) {
  std::vector<size_t> shape;
  for (int64_t d : t->getPhysicalDim())
    shape.push_back(static_cast<size_t>(d));
  auto b = Buffer::allocate(gpu(), shape, data);
  if (isError(b)) {
    std::printf("allocate failed: %s\n", ErrorObject(b).getMessage().c_str());
    std::exit(3);
  }
  return std::make_shared<Buffer>(std::move(*b));
}
template <typename T>
static std::shared_ptr<Buffer> fill(const std::shared_ptr<TensorAttr> &t, T v) {
  size_t n = 1;
  for (int64_t d : t->getPhysicalDim())
    n *= static_cast<size_t>(d);
  return bufOf(t, std::vector<T>(n, v));
}
static std::shared_ptr<Buffer> workspaceFor(Graph &g) {
  auto ws = g.getWorkspaceSize();
  if (isError(ws) || !ws->has_value() || **ws == 0)
    return nullptr;
  auto b = Buffer::allocateRaw(gpu(), **ws);
  return std::make_shared<Buffer>(std::move(*b));
}
template <typename T>
static std::vector<T> readBack(const std::shared_ptr<Buffer> &b) {
  std::vector<T> out;
  auto st = b->read(gpu(), out);
  if (isError(st))
    std::printf("read failed: %s\n", st.getMessage().c_str());
  return out;
}
static Graph newGraph(const std::string &name, DataType io,
                      DataType inter = DataType::Float) {
  Graph g;
  g.setName(name).setIODataType(io).setIntermediateDataType(inter)
      .setComputeDataType(DataType::Float);
  return g;
}
template <typename T> static bool allEqual(const std::vector<T> &v, float x) {
  for (const T &e : v)
    if (static_cast<float>(e) != x)
      return false;
  return !v.empty();
}

static std::vector<float> randomVec(size_t n, uint32_t seed, float lo, float hi) {
  std::mt19937 rng(seed);
  std::vector<float> v(n);
  for (auto &x : v)
    x = lo + (hi - lo) * (rng() >> 8) * (1.0f / 16777216.0f);
  return v;
}

// ---- convolution samples -----------------------------------------------------
static void convOnes(bool nhwc, bool bias, bool relu, int64_t r, int64_t pad,
                     float expectCorner, float expectCentre) {
  const int64_t n = 4, c = 128, h = 8, w = 8, k = 32;
  Graph g = newGraph(std::string("conv_") + (nhwc ? "nhwc" : "nchw") +
                         (bias ? "_b" : "") + (relu ? "_r" : "") + std::to_string(r),
                     DataType::Half);
  auto lay = [&](const Dims &d) { return nhwc ? chlast(d) : contig(d); };
  auto X = g.tensor(mk("x", {n, c, h, w}, lay({n, c, h, w}), DataType::Half));
  auto W = g.tensor(mk("w", {k, c, r, r}, lay({k, c, r, r}), DataType::Half));
  ConvFPropAttr ca;
  ca.setPadding({pad, pad}).setStride({1, 1}).setDilation({1, 1});
  auto Y = g.convFProp(X, W, ca);
  std::shared_ptr<TensorAttr> B;
  if (bias) {
    B = g.tensor(mk("b", {1, k, 1, 1}, {k, 1, k, k}, DataType::Half));
    PointwiseAttr add;
    add.setMode(PointwiseAttr::Mode::ADD);
    Y = g.pointwise(Y, B, add);
  }
  if (relu) {
    PointwiseAttr rl;
    rl.setMode(PointwiseAttr::Mode::RELU_FWD);
    Y = g.pointwise(Y, rl);
  }
  Y->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), /*remove=*/true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1)); // fused
  Pack pack = {{X, fill(X, half(1.0f))}, {W, fill(W, half(1.0f))},
               {Y, fill(Y, half(0.0f))}};
  if (bias)
    pack[B] = fill(B, half(1.0f));
  auto ws = workspaceFor(g);
  for (int rep = 0; rep < 2; ++rep) { // samples execute twice
    REQUIRE_OK(g.execute(gpu(), pack, ws));
    auto out = readBack<half>(pack[Y]);
    REQUIRE(out.size() == static_cast<size_t>(n * k * h * w));
    // logical (0,0,0,0) is storage element 0 in both layouts
    CHECK(static_cast<float>(out[0]) == expectCorner);
    // logical (0,0,3,3)
    const size_t centre = nhwc ? static_cast<size_t>((3 * w + 3) * k)
                               : static_cast<size_t>(3 * w + 3);
    CHECK(static_cast<float>(out[centre]) == expectCentre);
    if (r == 1)
      CHECK(allEqual(out, expectCorner));
  }
}

TEST("samples: conv fprop all-ones known answers") {
  convOnes(false, false, false, 1, 0, 128.f, 128.f); // test_graph.cpp:198-223
  convOnes(true, false, false, 1, 0, 128.f, 128.f);  // conv_fprop_nhwc_krsc.cpp:95
  convOnes(true, true, false, 1, 0, 129.f, 129.f);   // conv_fprop_with_bias.cpp:107
  convOnes(true, true, true, 1, 0, 129.f, 129.f);    // ..._with_relu_and_bias.cpp:112
  convOnes(true, false, false, 3, 1, 512.f, 1152.f); // ..._with_pad.cpp:94
  convOnes(false, true, true, 3, 1, 513.f, 1153.f);
}

// ---- convolution gradient samples ----------------------------------------------
// samples/convolution/conv_dgrad_nhwc_krsc{,_grouped}.cpp and
// conv_wgrad_nhwc_krsc{,_grouped,_grouped_strided}.cpp: all-ones f16, 1x1
// filters, NHWC activations and gradients, KRSC filters; each run twice.
static void convGradOnes(bool dgrad, int64_t c, int64_t k, int64_t fc,
                         int64_t st, bool biasGrad, float expect) {
  const int64_t n = 4, h = 8, w = 8, ho = h / st, wo = w / st;
  Graph g = newGraph(std::string(dgrad ? "dgrad_" : "wgrad_") + std::to_string(c) +
                         "_" + std::to_string(fc) + "_" + std::to_string(st) +
                         (biasGrad ? "_db" : ""),
                     DataType::Half);
  auto DY = g.tensor(mk("dy", {n, k, ho, wo}, chlast({n, k, ho, wo}), DataType::Half));
  std::shared_ptr<TensorAttr> IN, OUT, DB;
  if (dgrad) {
    IN = g.tensor(mk("w", {k, fc, 1, 1}, contig({k, fc, 1, 1}), DataType::Half));
    ConvDGradAttr a;
    a.setPadding({0, 0}).setStride({st, st}).setDilation({1, 1});
    OUT = g.convDGrad(DY, IN, a);
    OUT->setDim({n, c, h, w}).setOutput(true);
  } else {
    IN = g.tensor(mk("x", {n, c, h, w}, chlast({n, c, h, w}), DataType::Half));
    ConvWGradAttr a;
    a.setPadding({0, 0}).setStride({st, st}).setDilation({1, 1});
    OUT = g.convWGrad(DY, IN, a);
    OUT->setDim({k, fc, 1, 1}).setOutput(true);
  }
  if (biasGrad) { // bias gradient: DY summed over batch and space
    ReductionAttr ra;
    ra.setMode(ReductionAttr::Mode::SUM).setName("bias_reduction");
    DB = g.reduction(DY, ra);
    DB->setDim({1, k, 1, 1}).setStride({1, 1, 1, 1}).setOutput(true);
  }
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), /*remove=*/true));
  Pack pack = {{DY, fill(DY, half(1.0f))}, {IN, fill(IN, half(1.0f))},
               {OUT, fill(OUT, half(0.0f))}};
  if (biasGrad)
    pack[DB] = fill(DB, half(0.0f));
  auto ws = workspaceFor(g);
  for (int rep = 0; rep < 2; ++rep) {
    REQUIRE_OK(g.execute(gpu(), pack, ws));
    auto out = readBack<half>(pack[OUT]);
    REQUIRE(out.size() ==
            static_cast<size_t>(dgrad ? n * c * h * w : k * fc));
    CHECK(allEqual(out, expect));
    if (biasGrad)
      CHECK(allEqual(readBack<half>(pack[DB]), static_cast<float>(n * ho * wo)));
  }
}

TEST("samples: conv dgrad / wgrad all-ones known answers") {
  convGradOnes(true, 8, 16, 8, 1, false, 16.f);  // conv_dgrad_nhwc_krsc.cpp:98: K
  convGradOnes(true, 8, 16, 8, 1, true, 16.f);   // ...:207-217 with the bias gradient
  convGradOnes(true, 16, 32, 4, 1, false, 8.f);  // ..._grouped.cpp:99: K / groups
  convGradOnes(false, 8, 16, 8, 1, false, 256.f); // conv_wgrad_nhwc_krsc.cpp:99: N*H*W
  convGradOnes(false, 8, 16, 8, 1, true, 256.f);  // ...:208-217
  convGradOnes(false, 16, 32, 4, 1, false, 256.f); // ..._grouped.cpp:99
  convGradOnes(false, 16, 32, 4, 2, false, 64.f);  // ..._grouped_strided.cpp:103
}

TEST("conv gradients: f32 3x3 stride 2 pad 1 against host loops") {
  const int64_t n = 2, c = 6, h = 9, w = 10, k = 4, r = 3, st = 2, pad = 1;
  const int64_t ho = 1 + (h + 2 * pad - r) / st, wo = 1 + (w + 2 * pad - r) / st;
  auto xf = randomVec(n * c * h * w, 21, -1.f, 1.f);
  auto wf = randomVec(k * c * r * r, 22, -1.f, 1.f);
  auto gf = randomVec(n * k * ho * wo, 23, -1.f, 1.f);
  // contiguous NCHW / KCRS throughout
  std::vector<double> dxRef(xf.size(), 0.0), dwRef(wf.size(), 0.0);
  for (int64_t in = 0; in < n; ++in)
    for (int64_t kk = 0; kk < k; ++kk)
      for (int64_t p = 0; p < ho; ++p)
        for (int64_t q = 0; q < wo; ++q) {
          const double gy = gf[((in * k + kk) * ho + p) * wo + q];
          for (int64_t cc = 0; cc < c; ++cc)
            for (int64_t fr = 0; fr < r; ++fr)
              for (int64_t fs = 0; fs < r; ++fs) {
                const int64_t ih = p * st - pad + fr, iw = q * st - pad + fs;
                if (ih < 0 || ih >= h || iw < 0 || iw >= w)
                  continue;
                const size_t xi = ((in * c + cc) * h + ih) * w + iw;
                const size_t wi = ((kk * c + cc) * r + fr) * r + fs;
                dxRef[xi] += gy * wf[wi];
                dwRef[wi] += gy * xf[xi];
              }
        }
  Graph g = newGraph("conv_grads_f32", DataType::Float);
  auto DY = g.tensor(mk("dy", {n, k, ho, wo}, contig({n, k, ho, wo}), DataType::Float));
  auto X = g.tensor(mk("x", {n, c, h, w}, contig({n, c, h, w}), DataType::Float));
  auto W = g.tensor(mk("w", {k, c, r, r}, contig({k, c, r, r}), DataType::Float));
  ConvDGradAttr da;
  da.setPadding({pad, pad}).setStride({st, st}).setDilation({1, 1});
  auto DX = g.convDGrad(DY, W, da);
  DX->setDim({n, c, h, w}).setOutput(true);
  ConvWGradAttr wa;
  wa.setPadding({pad, pad}).setStride({st, st}).setDilation({1, 1});
  auto DW = g.convWGrad(DY, X, wa);
  DW->setDim({k, c, r, r}).setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(2));
  Pack pack = {{DY, bufOf(DY, gf)}, {X, bufOf(X, xf)}, {W, bufOf(W, wf)},
               {DX, fill(DX, 0.f)}, {DW, fill(DW, 0.f)}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto dx = readBack<float>(pack[DX]);
  auto dw = readBack<float>(pack[DW]);
  REQUIRE(dx.size() == dxRef.size());
  REQUIRE(dw.size() == dwRef.size());
  double worst = 0;
  for (size_t i = 0; i < dx.size(); ++i)
    worst = std::max(worst, std::fabs(dx[i] - dxRef[i]) - 1e-4 * (std::fabs(dxRef[i]) + 1.0));
  for (size_t i = 0; i < dw.size(); ++i)
    worst = std::max(worst, std::fabs(dw[i] - dwRef[i]) - 1e-4 * (std::fabs(dwRef[i]) + 1.0));
  CHECK(worst <= 0.0);
}

// ---- batch norm samples ----------------------------------------------------------
// samples/batchnorm/*.cpp with the generators of batchnorm_utils.h:22-107.
static void batchnormSample(bool training, bool nhwc, bool affine) {
  const int64_t n = 2, c = 4, h = 8, w = 8;
  const float eps = 1e-5f, scale = 2.0f, bias = 0.5f;
  Graph g = newGraph(std::string("bn_") + (training ? "train" : "infer") +
                         (nhwc ? "_nhwc" : "_nchw") + (affine ? "_sb" : ""),
                     DataType::Float);
  const Dims xd = {n, c, h, w};
  auto X = g.tensor(mk("x", xd, nhwc ? chlast(xd) : contig(xd), DataType::Float));
  std::shared_ptr<TensorAttr> SC, BI, MEAN, VAR;
  if (affine) {
    SC = g.tensor(mk("scale", {c}, {1}, DataType::Float));
    BI = g.tensor(mk("bias", {c}, {1}, DataType::Float));
  }
  if (!training) {
    MEAN = g.tensor(mk("mean", {c}, {1}, DataType::Float));
    VAR = g.tensor(mk("var", {c}, {1}, DataType::Float));
  }
  BatchnormAttr a;
  a.setForwardPhase(training ? NormFwdPhase::TRAINING : NormFwdPhase::INFERENCE)
      .setEpsilon(g.tensor(TensorAttr(eps).setName("epsilon")))
      .setMomentum(g.tensor(TensorAttr(0.1f).setName("momentum")))
      .setName("batchnorm");
  auto [Y, SM, SV] = g.batchnorm(X, SC, BI, MEAN, VAR, a);
  Y->setName("y").setDataType(DataType::Float).setOutput(true);
  if (training) {
    SM->setName("saved_mean").setDataType(DataType::Float).setOutput(true);
    SV->setName("saved_inv_var").setDataType(DataType::Float).setOutput(true);
  }
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), /*remove=*/true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1));
  // logical NCHW values, written through X's strides
  const float invStd = 1.0f / std::sqrt(1.0f + eps);
  std::vector<float> xin(n * c * h * w), want(xin.size());
  for (int64_t ni = 0; ni < n; ++ni)
    for (int64_t ci = 0; ci < c; ++ci)
      for (int64_t hi = 0; hi < h; ++hi)
        for (int64_t wi = 0; wi < w; ++wi) {
          const float xv = training
                               ? (ni * h * w + hi * w + wi < n * h * w / 2 ? -1.f : 1.f)
                               : static_cast<float>(ci + 1);
          const size_t idx = nhwc ? ((ni * h + hi) * w + wi) * c + ci
                                  : ((ni * c + ci) * h + hi) * w + wi;
          xin[idx] = xv;
          want[idx] = (affine ? scale : 1.f) * xv * invStd + (affine ? bias : 0.f);
        }
  Pack pack = {{X, bufOf(X, xin)}, {Y, fill(Y, 0.f)}};
  if (affine) {
    pack[SC] = fill(SC, scale);
    pack[BI] = fill(BI, bias);
  }
  if (training) {
    pack[SM] = fill(SM, 7.f);
    pack[SV] = fill(SV, 7.f);
  } else {
    pack[MEAN] = fill(MEAN, 0.f);
    pack[VAR] = fill(VAR, 1.f);
  }
  auto ws = workspaceFor(g);
  for (int rep = 0; rep < 2; ++rep) {
    REQUIRE_OK(g.execute(gpu(), pack, ws));
    auto out = readBack<float>(pack[Y]);
    REQUIRE(out.size() == want.size());
    float worst = 0;
    for (size_t i = 0; i < out.size(); ++i)
      worst = std::max(worst, std::fabs(out[i] - want[i]));
    CHECK(worst < 1e-4f); // the samples' tolerance
    if (training) {
      auto sm = readBack<float>(pack[SM]);
      auto sv = readBack<float>(pack[SV]);
      REQUIRE(sm.size() == static_cast<size_t>(c));
      REQUIRE(sv.size() == static_cast<size_t>(c));
      for (int64_t ci = 0; ci < c; ++ci) {
        CHECK(std::fabs(sm[ci]) < 1e-4f);
        CHECK(std::fabs(sv[ci] - invStd) < 1e-4f);
      }
    }
  }
}

TEST("samples: batchnorm inference and training known answers") {
  batchnormSample(false, false, false); // batchnorm_infer_nchw.cpp
  batchnormSample(false, false, true);  // batchnorm_infer_nchw_scale_bias.cpp
  batchnormSample(false, true, true);   // batchnorm_infer_nhwc_scale_bias.cpp
  batchnormSample(true, false, false);  // batchnorm_train_nchw.cpp
  batchnormSample(true, false, true);   // batchnorm_train_nchw_scale_bias.cpp
  batchnormSample(true, true, true);
}

// ---- dynamic dims --------------------------------------------------------------
// samples/dynamic_shapes/conv_fprop_dynamic_batch.cpp,
// reduction_min_max_dynamic_batch.cpp, sdpa_basic_dynamic_sequence.cpp: one
// compiled graph, buffers of several extents in the dynamic dim.
template <typename T>
static std::shared_ptr<Buffer> shaped(const Dims &shape, T v) {
  std::vector<size_t> sh(shape.begin(), shape.end());
  size_t n = 1;
  for (size_t d : sh)
    n *= d;
  auto b = Buffer::allocate(gpu(), sh, std::vector<T>(n, v));
  if (isError(b)) {
    std::printf("allocate failed: %s\n", ErrorObject(b).getMessage().c_str());
    std::exit(3);
  }
  return std::make_shared<Buffer>(std::move(*b));
}

TEST("dynamic dims: conv batch, reduction batch and sdpa sequence from one compiled graph each") {
  {
    const int64_t n = 4, c = 4, h = 4, w = 4, k = 4;
    Graph g = newGraph("dynamic_conv_fprop", DataType::Half);
    auto X = g.tensor(mk("image", {n, c, h, w}, contig({n, c, h, w}), DataType::Half)
                          .setDynamicDims({0}));
    auto W = g.tensor(mk("filter", {k, c, 1, 1}, contig({k, c, 1, 1}), DataType::Half));
    ConvFPropAttr ca;
    ca.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    auto Y = g.convFProp(X, W, ca);
    Y->setDynamicDims({0}).setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    auto ws = g.getWorkspaceSize();
    REQUIRE(!isError(ws) && ws->has_value());
    CHECK(**ws == 0);
    auto wBuf = fill(W, half(1.f));
    for (int64_t rn : {int64_t{1}, int64_t{2}, n, int64_t{2}}) {
      Pack pack = {{X, shaped<half>({rn, c, h, w}, half(1.f))}, {W, wBuf},
                   {Y, shaped<half>({rn, k, h, w}, half(0.f))}};
      REQUIRE_OK(g.execute(gpu(), pack, nullptr));
      auto out = readBack<half>(pack[Y]);
      REQUIRE(out.size() == static_cast<size_t>(rn * k * h * w));
      CHECK(allEqual(out, 4.f)); // conv_fprop_dynamic_batch.cpp:110
    }
    // a non-dynamic dim must keep its extent
    Pack bad = {{X, shaped<half>({2, c, h, w + 1}, half(1.f))}, {W, wBuf},
                {Y, shaped<half>({2, k, h, w}, half(0.f))}};
    CHECK_ERROR(g.execute(gpu(), bad, nullptr), ErrorCode::VariantPackError,
                "Buffer for tensor 'image' has extent 5 in dim 3, which is not "
                "a dynamic dim (expected 4)");
  }
  {
    // NHWC activations: the buffer's shape is in physical order
    const int64_t n = 4, c = 8, h = 3, w = 5, k = 16;
    Graph g = newGraph("dynamic_conv_nhwc", DataType::Half);
    auto X = g.tensor(mk("image", {n, c, h, w}, chlast({n, c, h, w}), DataType::Half)
                          .setDynamicDims({0}));
    auto W = g.tensor(mk("filter", {k, c, 1, 1}, chlast({k, c, 1, 1}), DataType::Half));
    ConvFPropAttr ca;
    ca.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    auto Y = g.convFProp(X, W, ca);
    Y->setDynamicDims({0}).setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    REQUIRE(!isError(g.getWorkspaceSize()));
    auto wBuf = fill(W, half(1.f));
    for (int64_t rn : {int64_t{3}, n}) {
      Pack pack = {{X, shaped<half>({rn, h, w, c}, half(1.f))}, {W, wBuf},
                   {Y, shaped<half>({rn, h, w, k}, half(0.f))}};
      REQUIRE_OK(g.execute(gpu(), pack, nullptr));
      auto out = readBack<half>(pack[Y]);
      REQUIRE(out.size() == static_cast<size_t>(rn * k * h * w));
      CHECK(allEqual(out, 8.f));
    }
  }
  {
    const int64_t n = 4, c = 6, l = 10;
    Graph g = newGraph("dynamic_reduction", DataType::Float);
    auto X = g.tensor(mk("x", {n, c, l}, contig({n, c, l}), DataType::Float)
                          .setDynamicDims({0}));
    ReductionAttr ra;
    ra.setMode(ReductionAttr::Mode::MAX);
    auto Y = g.reduction(X, ra);
    Y->setDim({n, c, 1}).setStride({c, 1, 1}).setDynamicDims({0}).setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    REQUIRE(!isError(g.getWorkspaceSize()));
    for (int64_t rn : {int64_t{1}, int64_t{3}, n}) {
      std::vector<float> xin(rn * c * l);
      for (size_t i = 0; i < xin.size(); ++i)
        xin[i] = static_cast<float>((i * 7) % 23) - 11.f;
      std::vector<size_t> sh = {static_cast<size_t>(rn), static_cast<size_t>(c),
                                static_cast<size_t>(l)};
      auto xb = Buffer::allocate(gpu(), sh, xin);
      REQUIRE(!isError(xb));
      Pack pack = {{X, std::make_shared<Buffer>(std::move(*xb))},
                   {Y, shaped<float>({rn, c, 1}, 0.f)}};
      REQUIRE_OK(g.execute(gpu(), pack, nullptr));
      auto out = readBack<float>(pack[Y]);
      REQUIRE(out.size() == static_cast<size_t>(rn * c));
      bool same = true;
      for (int64_t r = 0; r < rn * c; ++r) {
        float mx = xin[r * l];
        for (int64_t i = 1; i < l; ++i)
          mx = std::max(mx, xin[r * l + i]);
        same = same && out[r] == mx;
      }
      CHECK(same);
    }
  }
  {
    const int64_t b = 1, hh = 8, sq = 64, d = 64;
    Graph g = newGraph("dynamic_sdpa", DataType::Half);
    const Dims dims = {b, hh, sq, d};
    auto Q = g.tensor(mk("q", dims, contig(dims), DataType::Half).setDynamicDims({2}));
    auto K = g.tensor(mk("k", dims, contig(dims), DataType::Half).setDynamicDims({2}));
    auto V = g.tensor(mk("v", dims, contig(dims), DataType::Half).setDynamicDims({2}));
    SdpaAttr sa;
    auto O = g.sdpa(Q, K, V, nullptr, sa);
    O->setDynamicDims({2}).setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    REQUIRE(!isError(g.getWorkspaceSize()));
    for (int64_t rs : {int64_t{16}, int64_t{32}, sq}) {
      const Dims rd = {b, hh, rs, d};
      Pack pack = {{Q, shaped<half>(rd, half(0.01f))}, {K, shaped<half>(rd, half(0.01f))},
                   {V, shaped<half>(rd, half(0.01f))}, {O, shaped<half>(rd, half(0.f))}};
      REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
      auto out = readBack<half>(pack[O]);
      REQUIRE(out.size() == static_cast<size_t>(b * hh * rs * d));
      float worst = 0;
      for (half v : out) // constant V => O = V (sdpa_basic_dynamic_sequence.cpp)
        worst = std::max(worst, std::fabs(static_cast<float>(v) - 0.01f));
      CHECK(worst < 1e-3f);
    }
  }
}

// ---- matmul samples ----------------------------------------------------------
TEST("samples: matmul all-ones, transposed B, bias, batched broadcast") {
  for (int variant = 0; variant < 3; ++variant) {
    const int64_t m = 64, k = 128, n = 256;
    Graph g = newGraph("mm_" + std::to_string(variant), DataType::Half);
    auto A = g.tensor(mk("a", {m, k}, {k, 1}, DataType::Half));
    auto B = g.tensor(mk("b", {k, n}, variant == 1 ? Dims{1, k} : Dims{n, 1},
                         DataType::Half));
    MatmulAttr ma;
    auto C = g.matmul(A, B, ma);
    std::shared_ptr<TensorAttr> bias;
    if (variant == 2) {
      bias = g.tensor(mk("bias", {1, n}, {n, 1}, DataType::Half));
      PointwiseAttr add;
      add.setMode(PointwiseAttr::Mode::ADD);
      C = g.pointwise(C, bias, add);
    }
    C->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    Pack pack = {{A, fill(A, half(1.f))}, {B, fill(B, half(1.f))},
                 {C, fill(C, half(0.f))}};
    if (bias)
      pack[bias] = fill(bias, half(2.f));
    auto ws = workspaceFor(g);
    for (int rep = 0; rep < 2; ++rep) {
      REQUIRE_OK(g.execute(gpu(), pack, ws));
      CHECK(allEqual(readBack<half>(pack[C]), variant == 2 ? 130.f : 128.f));
    }
  }
  { // samples/matmul/matmul_batched.cpp: [16,16,M,K] x [1,1,K,N], f32
    const int64_t m = 16, k = 32, n = 64;
    Graph g = newGraph("mm_bcast", DataType::Float);
    auto A = g.tensor(mk("a", {16, 16, m, k}, contig({16, 16, m, k}), DataType::Float));
    auto B = g.tensor(mk("b", {1, 1, k, n}, contig({1, 1, k, n}), DataType::Float));
    MatmulAttr ma;
    auto C = g.matmul(A, B, ma);
    C->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    Pack pack = {{A, fill(A, 1.f)}, {B, fill(B, 1.f)}, {C, fill(C, 0.f)}};
    auto ws = workspaceFor(g);
    REQUIRE_OK(g.execute(gpu(), pack, ws));
    CHECK(allEqual(readBack<float>(pack[C]), 32.f));
  }
}

// ---- sdpa samples ------------------------------------------------------------
TEST("samples: sdpa constant fill equals V") {
  struct V { bool causal, mask, gqa; int64_t sq, skv; };
  for (const V &v : {V{false, false, false, 64, 64}, V{true, false, false, 64, 64},
                     V{false, true, false, 64, 64}, V{false, false, true, 64, 64},
                     V{false, false, false, 32, 128}}) {
    const int64_t b = 1, hq = 8, hkv = v.gqa ? 2 : 8, d = 64;
    Graph g = newGraph("sdpa_" + std::to_string(v.causal) + std::to_string(v.mask) +
                           std::to_string(v.gqa) + std::to_string(v.skv),
                       DataType::Half);
    auto Q = g.tensor(mk("q", {b, hq, v.sq, d}, contig({b, hq, v.sq, d}), DataType::Half));
    auto K = g.tensor(mk("k", {b, hkv, v.skv, d}, contig({b, hkv, v.skv, d}), DataType::Half));
    auto Vt = g.tensor(mk("v", {b, hkv, v.skv, d}, contig({b, hkv, v.skv, d}), DataType::Half));
    std::shared_ptr<TensorAttr> M;
    if (v.mask)
      M = g.tensor(mk("m", {b, 1, v.sq, v.skv}, contig({b, 1, v.sq, v.skv}), DataType::Half));
    SdpaAttr sa;
    sa.setIsCausal(v.causal).setEnableGqa(v.gqa);
    auto O = g.sdpa(Q, K, Vt, M, sa);
    O->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    Pack pack = {{Q, fill(Q, half(0.01f))}, {K, fill(K, half(0.01f))},
                 {Vt, fill(Vt, half(0.01f))}, {O, fill(O, half(0.f))}};
    if (M)
      pack[M] = fill(M, half(-1.0f));
    auto ws = workspaceFor(g);
    for (int rep = 0; rep < 2; ++rep) {
      REQUIRE_OK(g.execute(gpu(), pack, ws));
      auto out = readBack<half>(pack[O]);
      bool okAll = !out.empty();
      for (half e : out)
        okAll = okAll && std::fabs(static_cast<float>(e) - 0.01f) < 1e-2f;
      CHECK(okAll); // samples/sdpa_utils.cpp:241-246
    }
  }
}

// ---- norm samples ------------------------------------------------------------
TEST("samples: rmsnorm and layernorm two-value patterns") {
  const int64_t n = 2, c = 3, h = 32, w = 32;
  const size_t inner = static_cast<size_t>(c * h * w);
  for (bool nhwc : {false, true}) {
    const float eps = 1e-5f, sc = 2.0f;
    Graph g = newGraph(std::string("rms_") + (nhwc ? "nhwc" : "nchw"), DataType::Float);
    auto lay = [&](const Dims &d) { return nhwc ? chlast(d) : contig(d); };
    auto X = g.tensor(mk("x", {n, c, h, w}, lay({n, c, h, w}), DataType::Float));
    auto S = g.tensor(mk("s", {1, c, h, w}, lay({1, c, h, w}), DataType::Float));
    RmsnormAttr ra;
    ra.setForwardPhase(NormFwdPhase::INFERENCE).setEpsilon(g.tensor(TensorAttr(eps)));
    auto [Y, R] = g.rmsnorm(X, S, ra);
    Y->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    std::vector<float> xin(n * inner), expect(n * inner);
    for (int64_t b = 0; b < n; ++b) { // samples/rmsnorm/rmsnorm_utils.h:26-66
      const float x0 = 2.f * b + 1.f, x1 = x0 + 2.f;
      const float rms = std::sqrt((x0 * x0 + x1 * x1) / 2.f + eps);
      for (size_t i = 0; i < inner; ++i) {
        const bool first = i < inner / 2;
        xin[b * inner + i] = first ? x0 : x1;
        expect[b * inner + i] = sc * (first ? x0 : x1) / rms;
      }
    }
    Pack pack = {{X, bufOf(X, xin)}, {S, fill(S, sc)}, {Y, fill(Y, 0.f)}};
    auto ws = workspaceFor(g);
    REQUIRE_OK(g.execute(gpu(), pack, ws));
    auto out = readBack<float>(pack[Y]);
    bool okAll = out.size() == expect.size();
    for (size_t i = 0; okAll && i < out.size(); ++i)
      okAll = std::fabs(out[i] - expect[i]) < 1e-4f;
    CHECK(okAll);
  }
  { // samples/layernorm/layernorm_utils.h:25-82 (training outputs)
    const float eps = 1e-5f, sc = 2.f, bi = 1.f;
    Graph g = newGraph("ln_train", DataType::Float);
    auto X = g.tensor(mk("x", {n, c, h, w}, contig({n, c, h, w}), DataType::Float));
    auto S = g.tensor(mk("s", {1, c, h, w}, contig({1, c, h, w}), DataType::Float));
    auto B = g.tensor(mk("b", {1, c, h, w}, contig({1, c, h, w}), DataType::Float));
    LayernormAttr la;
    la.setForwardPhase(NormFwdPhase::TRAINING).setEpsilon(g.tensor(TensorAttr(eps)));
    auto [Y, M, V] = g.layernorm(X, S, B, la);
    Y->setOutput(true);
    M->setOutput(true);
    V->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    std::vector<float> xin(n * inner);
    for (int64_t b = 0; b < n; ++b)
      for (size_t i = 0; i < inner; ++i)
        xin[b * inner + i] = i < inner / 2 ? 2.f * b : 2.f * b + 2.f;
    Pack pack = {{X, bufOf(X, xin)}, {S, fill(S, sc)}, {B, fill(B, bi)},
                 {Y, fill(Y, 0.f)}, {M, fill(M, 0.f)}, {V, fill(V, 0.f)}};
    auto ws = workspaceFor(g);
    REQUIRE_OK(g.execute(gpu(), pack, ws));
    auto y = readBack<float>(pack[Y]);
    auto m = readBack<float>(pack[M]);
    auto v = readBack<float>(pack[V]);
    const float r = 1.f / std::sqrt(1.f + eps);
    bool okAll = true;
    for (int64_t b = 0; b < n; ++b)
      for (size_t i = 0; i < inner; ++i)
        okAll = okAll && std::fabs(y[b * inner + i] -
                                   ((i < inner / 2 ? -sc : sc) * r + bi)) < 1e-4f;
    CHECK(okAll);
    CHECK(std::fabs(m[0] - 1.f) < 1e-4f && std::fabs(m[1] - 3.f) < 1e-4f);
    CHECK(std::fabs(v[0] - r) < 1e-4f && std::fabs(v[1] - r) < 1e-4f);
  }
}

// ---- reduction sample --------------------------------------------------------
TEST("samples: reduction table, element (0,0)") {
  using M = ReductionAttr::Mode;
  // samples/reduction/reduction_ops.cpp: [2,16,8,8] -> [2,16,1,1]; inputs
  // i % 100 - 50; element (0,0) reduces inputs 0..63 = -50..13.
  struct Row { M mode; float expect; };
  double sum = 0, sumsq = 0, sumabs = 0;
  for (int i = 0; i < 64; ++i) {
    const double x = i - 50;
    sum += x, sumsq += x * x, sumabs += std::fabs(x);
  }
  for (const Row &row : {Row{M::ADD, (float)sum}, Row{M::SUM, (float)sum},
                         Row{M::MIN, -50.f}, Row{M::MAX, 13.f}, Row{M::AMAX, 50.f},
                         Row{M::AVG, (float)(sum / 64)}, Row{M::NORM1, (float)sumabs},
                         Row{M::NORM2, (float)std::sqrt(sumsq)}}) {
    Graph g = newGraph(std::string("red_") + ReductionAttr::modeName(row.mode),
                       DataType::Float);
    auto X = g.tensor(mk("x", {2, 16, 8, 8}, contig({2, 16, 8, 8}), DataType::Float));
    ReductionAttr ra;
    ra.setMode(row.mode);
    auto Y = g.reduction(X, ra);
    Y->setOutput(true).setDim({2, 16, 1, 1});
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    std::vector<float> xin(2 * 16 * 64);
    for (size_t i = 0; i < xin.size(); ++i)
      xin[i] = static_cast<float>(static_cast<int>(i % 100) - 50);
    Pack pack = {{X, bufOf(X, xin)}, {Y, fill(Y, 0.f)}};
    REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
    auto out = readBack<float>(pack[Y]);
    CHECK(std::fabs(out[0] - row.expect) < 0.01f);
  }
  { // int32 product with a 2 and a 3 => 6
    Graph g = newGraph("red_mul_i32", DataType::Int32);
    auto X = g.tensor(mk("x", {2, 16, 8, 8}, contig({2, 16, 8, 8}), DataType::Int32));
    ReductionAttr ra;
    ra.setMode(M::MUL);
    auto Y = g.reduction(X, ra);
    Y->setOutput(true).setDim({2, 16, 1, 1});
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    std::vector<int32_t> xin(2 * 16 * 64, 1);
    xin[0] = 2, xin[1] = 3;
    Pack pack = {{X, bufOf(X, xin)}, {Y, fill(Y, int32_t(0))}};
    REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
    CHECK(readBack<int32_t>(pack[Y])[0] == 6);
  }
}

// ---- pointwise samples -------------------------------------------------------
TEST("samples: pointwise transposed add, scalar mul, AOT int32 add") {
  { // samples/pointwise/pointwise_add_transposed.cpp:22-112
    Graph g = newGraph("pw_t", DataType::Float);
    auto A = g.tensor(mk("a", {3, 2}, {2, 1}, DataType::Float));
    auto B = g.tensor(mk("b", {3, 2}, {1, 3}, DataType::Float));
    PointwiseAttr add;
    add.setMode(PointwiseAttr::Mode::ADD);
    auto O = g.pointwise(A, B, add);
    O->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    std::vector<float> data = {1, 2, 3, 4, 5, 6};
    Pack pack = {{A, bufOf(A, data)}, {B, bufOf(B, data)}, {O, fill(O, 0.f)}};
    REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
    CHECK((readBack<float>(pack[O]) == std::vector<float>{2, 6, 5, 9, 8, 12}));
  }
  { // samples/pointwise/pointwise_scalar_mul.cpp:22-78
    Graph g = newGraph("pw_s", DataType::Float);
    auto A = g.tensor(mk("a", {2, 16, 8}, contig({2, 16, 8}), DataType::Float));
    auto two = g.tensor(TensorAttr(2.0f));
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    auto O = g.pointwise(A, two, mul);
    O->setOutput(true);
    REQUIRE_OK(g.validate());
    REQUIRE_OK(g.compile(gpu(), true));
    Pack pack = {{A, fill(A, 3.f)}, {O, fill(O, 0.f)}};
    REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
    CHECK(allEqual(readBack<float>(pack[O]), 6.f));
  }
  { // samples/aot/single_backend.cpp:52-110
    auto build = [](const std::string &name, std::shared_ptr<TensorAttr> &a,
                    std::shared_ptr<TensorAttr> &b, std::shared_ptr<TensorAttr> &o) {
      auto g = std::make_unique<Graph>();
      g->setName(name).setIODataType(DataType::Int32).setComputeDataType(DataType::Int32);
      a = g->tensor(mk("a", {4, 8}, {8, 1}, DataType::Int32));
      b = g->tensor(mk("b", {4, 8}, {8, 1}, DataType::Int32));
      PointwiseAttr add;
      add.setMode(PointwiseAttr::Mode::ADD);
      o = g->pointwise(a, b, add);
      o->setOutput(true);
      return g;
    };
    std::shared_ptr<TensorAttr> a1, b1, o1, a2, b2, o2;
    auto producer = build("aot", a1, b1, o1);
    REQUIRE_OK(producer->validate());
    REQUIRE_ASSIGN(auto bytes, producer->compileToArtifact(Backend::AMDGPU, true));
    auto consumer = build("aot", a2, b2, o2);
    REQUIRE_OK(consumer->validate());
    REQUIRE_OK(consumer->loadFromArtifact(gpu(), bytes));
    Pack pack = {{a2, fill(a2, int32_t(2))}, {b2, fill(b2, int32_t(3))},
                 {o2, fill(o2, int32_t(0))}};
    REQUIRE_OK(consumer->execute(gpu(), pack, workspaceFor(*consumer)));
    CHECK(allEqual(readBack<int32_t>(pack[o2]), 5.f));
  }
}

TEST("AOT: a graph with a data gradient (planner scratch) and a batch norm survives the artifact round trip") {
  const int64_t n = 2, c = 64, h = 6, w = 6, k = 64;
  std::shared_ptr<TensorAttr> dy[2], wt[2], dx[2], y[2];
  auto build = [&](int i) {
    auto g = std::make_unique<Graph>();
    g->setName("aot_grad").setIODataType(DataType::BFloat16)
        .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
    dy[i] = g->tensor(mk("dy", {n, k, h, w}, chlast({n, k, h, w}), DataType::BFloat16));
    wt[i] = g->tensor(mk("w", {k, c, 1, 1}, chlast({k, c, 1, 1}), DataType::BFloat16));
    ConvDGradAttr da;
    da.setPadding({0, 0}).setStride({1, 1}).setDilation({1, 1});
    dx[i] = g->convDGrad(dy[i], wt[i], da);
    dx[i]->setDim({n, c, h, w}).setOutput(true);
    BatchnormAttr ba;
    ba.setForwardPhase(NormFwdPhase::INFERENCE)
        .setEpsilon(g->tensor(TensorAttr(0.0f)))
        .setMomentum(g->tensor(TensorAttr(0.1f)));
    auto mean = g->tensor(mk("mean", {k}, {1}, DataType::Float));
    auto var = g->tensor(mk("var", {k}, {1}, DataType::Float));
    auto out = g->batchnorm(dy[i], nullptr, nullptr, mean, var, ba);
    y[i] = out[0];
    y[i]->setOutput(true);
    return std::make_tuple(std::move(g), mean, var);
  };
  auto [producer, m0, v0] = build(0);
  REQUIRE_OK(producer->validate());
  REQUIRE_ASSIGN(auto bytes, producer->compileToArtifact(Backend::AMDGPU, true));
  auto [consumer, m1, v1] = build(1);
  REQUIRE_OK(consumer->validate());
  REQUIRE_OK(consumer->loadFromArtifact(gpu(), bytes));
  CHECK(consumer->getKernelCount() == std::optional<size_t>(2));
  auto ws = consumer->getWorkspaceSize();
  REQUIRE(!isError(ws) && ws->has_value());
  CHECK(**ws >= static_cast<size_t>(k * c * 2)); // the mirrored filter
  Pack pack = {{dy[1], fill(dy[1], bf16(1.f))}, {wt[1], fill(wt[1], bf16(0.5f))},
               {dx[1], fill(dx[1], bf16(0.f))}, {y[1], fill(y[1], bf16(0.f))},
               {m1, fill(m1, 0.5f)}, {v1, fill(v1, 4.f)}};
  REQUIRE_OK(consumer->execute(gpu(), pack, workspaceFor(*consumer)));
  CHECK(allEqual(readBack<bf16>(pack[dx[1]]), 32.f)); // K * 1 * 0.5
  CHECK(allEqual(readBack<bf16>(pack[y[1]]), 0.25f)); // (1 - 0.5) / sqrt(4)
  // a corrupted artifact is rejected
  bytes[bytes.size() / 2] ^= 0x5a;
  CHECK(isError(consumer->loadFromArtifact(gpu(), bytes)));
}

// ---- benchmark configs through the graph API ---------------------------------

TEST("config 1: f32 matmul 1x256x512x256 vs host loop, rel 1e-4") {
  const int64_t m = 256, k = 512, n = 256;
  Graph g = newGraph("cfg1", DataType::Float);
  auto A = g.tensor(mk("a", {1, m, k}, contig({1, m, k}), DataType::Float));
  auto B = g.tensor(mk("b", {1, k, n}, contig({1, k, n}), DataType::Float));
  MatmulAttr ma;
  auto C = g.matmul(A, B, ma);
  C->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  auto a = randomVec(m * k, 1, -1.f, 1.f), b = randomVec(k * n, 2, -1.f, 1.f);
  Pack pack = {{A, bufOf(A, a)}, {B, bufOf(B, b)}, {C, fill(C, 0.f)}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<float>(pack[C]);
  double rms = 0, worst = 0;
  std::vector<double> ref(m * n, 0.0);
  for (int64_t i = 0; i < m; ++i)
    for (int64_t kk = 0; kk < k; ++kk)
      for (int64_t j = 0; j < n; ++j)
        ref[i * n + j] += (double)a[i * k + kk] * b[kk * n + j];
  for (double r : ref)
    rms += r * r;
  rms = std::sqrt(rms / ref.size());
  for (size_t i = 0; i < ref.size(); ++i)
    worst = std::max(worst, std::fabs(out[i] - ref[i]) -
                                1e-4 * (std::fabs(ref[i]) + rms));
  CHECK(worst <= 0.0);
}

TEST("config 3 (reduced): bf16 NHWC conv 3x3 + bias + relu vs host loop") {
  const int64_t n = 2, c = 64, h = 14, w = 14, k = 128;
  Graph g = newGraph("cfg3", DataType::BFloat16, DataType::Float);
  auto X = g.tensor(mk("x", {n, c, h, w}, chlast({n, c, h, w}), DataType::BFloat16));
  auto W = g.tensor(mk("w", {k, c, 3, 3}, chlast({k, c, 3, 3}), DataType::BFloat16));
  auto B = g.tensor(mk("b", {1, k, 1, 1}, {k, 1, k, k}, DataType::BFloat16));
  ConvFPropAttr ca;
  ca.setPadding({1, 1}).setStride({1, 1}).setDilation({1, 1});
  auto Y = g.convFProp(X, W, ca);
  PointwiseAttr add, relu;
  add.setMode(PointwiseAttr::Mode::ADD);
  relu.setMode(PointwiseAttr::Mode::RELU_FWD);
  auto O = g.pointwise(g.pointwise(Y, B, add), relu);
  O->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1));
  auto xf = randomVec(n * h * w * c, 3, -1.f, 1.f);
  auto wf = randomVec(k * 9 * c, 4, -0.1f, 0.1f);
  auto bf = randomVec(k, 5, -1.f, 1.f);
  std::vector<bf16> xb(xf.size()), wb(wf.size()), bb(bf.size());
  for (size_t i = 0; i < xf.size(); ++i) xb[i] = (bf16)xf[i], xf[i] = (float)xb[i];
  for (size_t i = 0; i < wf.size(); ++i) wb[i] = (bf16)wf[i], wf[i] = (float)wb[i];
  for (size_t i = 0; i < bf.size(); ++i) bb[i] = (bf16)bf[i], bf[i] = (float)bb[i];
  Pack pack = {{X, bufOf(X, xb)}, {W, bufOf(W, wb)}, {B, bufOf(B, bb)},
               {O, fill(O, bf16(0.f))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<bf16>(pack[O]);
  // physical layouts: x [n][h][w][c], w [k][r][s][c], out [n][p][q][k]
  double worst = 0, rms = 0;
  std::vector<double> ref(n * h * w * k);
  for (int64_t in = 0; in < n; ++in)
    for (int64_t p = 0; p < h; ++p)
      for (int64_t q = 0; q < w; ++q)
        for (int64_t kk = 0; kk < k; ++kk) {
          double acc = 0;
          for (int64_t r = 0; r < 3; ++r)
            for (int64_t s = 0; s < 3; ++s) {
              const int64_t ih = p - 1 + r, iw = q - 1 + s;
              if (ih < 0 || ih >= h || iw < 0 || iw >= w)
                continue;
              for (int64_t cc = 0; cc < c; ++cc)
                acc += (double)xf[((in * h + ih) * w + iw) * c + cc] *
                       wf[((kk * 3 + r) * 3 + s) * c + cc];
            }
          acc += bf[kk];
          ref[((in * h + p) * w + q) * k + kk] = acc > 0 ? acc : 0;
        }
  for (double r : ref)
    rms += r * r;
  rms = std::sqrt(rms / ref.size());
  for (size_t i = 0; i < ref.size(); ++i)
    worst = std::max(worst, std::fabs((float)out[i] - ref[i]) -
                                2e-2 * (std::fabs(ref[i]) + rms));
  CHECK(worst <= 0.0);
}

TEST("config 3 data gradient (reduced): bf16 NHWC on the MFMA kernel, scratch from the plan's workspace") {
  const int64_t n = 2, c = 64, h = 14, w = 14, k = 128;
  Graph g = newGraph("cfg3_dgrad", DataType::BFloat16, DataType::Float);
  auto DY = g.tensor(mk("dy", {n, k, h, w}, chlast({n, k, h, w}), DataType::BFloat16));
  auto W = g.tensor(mk("w", {k, c, 3, 3}, chlast({k, c, 3, 3}), DataType::BFloat16));
  ConvDGradAttr da;
  da.setPadding({1, 1}).setStride({1, 1}).setDilation({1, 1});
  auto DX = g.convDGrad(DY, W, da);
  DX->setDim({n, c, h, w}).setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  auto wsSize = g.getWorkspaceSize();
  REQUIRE(!isError(wsSize) && wsSize->has_value());
  CHECK(**wsSize >= static_cast<size_t>(k * c * 9 * 2)); // the mirrored filter
  auto gf = randomVec(n * h * w * k, 31, -1.f, 1.f);
  auto wf = randomVec(k * 9 * c, 32, -0.1f, 0.1f);
  std::vector<bf16> gb(gf.size()), wb(wf.size());
  for (size_t i = 0; i < gf.size(); ++i) gb[i] = (bf16)gf[i], gf[i] = (float)gb[i];
  for (size_t i = 0; i < wf.size(); ++i) wb[i] = (bf16)wf[i], wf[i] = (float)wb[i];
  Pack pack = {{DY, bufOf(DY, gb)}, {W, bufOf(W, wb)}, {DX, fill(DX, bf16(0.f))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<bf16>(pack[DX]);
  // physical layouts: dy [n][p][q][k], w [k][r][s][c], dx [n][h][w][c]
  std::vector<double> ref(n * h * w * c, 0.0);
  for (int64_t in = 0; in < n; ++in)
    for (int64_t p = 0; p < h; ++p)
      for (int64_t q = 0; q < w; ++q)
        for (int64_t r = 0; r < 3; ++r)
          for (int64_t s = 0; s < 3; ++s) {
            const int64_t ih = p - 1 + r, iw = q - 1 + s;
            if (ih < 0 || ih >= h || iw < 0 || iw >= w)
              continue;
            for (int64_t kk = 0; kk < k; ++kk) {
              const double gy = gf[((in * h + p) * w + q) * k + kk];
              for (int64_t cc = 0; cc < c; ++cc)
                ref[((in * h + ih) * w + iw) * c + cc] +=
                    gy * wf[((kk * 3 + r) * 3 + s) * c + cc];
            }
          }
  REQUIRE(out.size() == ref.size());
  double worst = 0, rms = 0;
  for (double r : ref)
    rms += r * r;
  rms = std::sqrt(rms / ref.size());
  for (size_t i = 0; i < ref.size(); ++i)
    worst = std::max(worst, std::fabs((float)out[i] - ref[i]) -
                                2e-2 * (std::fabs(ref[i]) + rms));
  CHECK(worst <= 0.0);
}

TEST("config 3 weight gradient (reduced): bf16 NHWC on batched MFMA GEMMs, scratch from the plan's workspace") {
  const int64_t n = 2, c = 64, h = 14, w = 14, k = 128;
  Graph g = newGraph("cfg3_wgrad", DataType::BFloat16, DataType::Float);
  auto DY = g.tensor(mk("dy", {n, k, h, w}, chlast({n, k, h, w}), DataType::BFloat16));
  auto X = g.tensor(mk("x", {n, c, h, w}, chlast({n, c, h, w}), DataType::BFloat16));
  ConvWGradAttr wa;
  wa.setPadding({1, 1}).setStride({1, 1}).setDilation({1, 1});
  auto DW = g.convWGrad(DY, X, wa);
  DW->setDim({k, c, 3, 3}).setDataType(DataType::Float).setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  auto wsSize = g.getWorkspaceSize();
  REQUIRE(!isError(wsSize) && wsSize->has_value());
  CHECK(**wsSize > 0); // padded operand copies and partial sums
  auto gf = randomVec(n * h * w * k, 41, -1.f, 1.f);
  auto xf = randomVec(n * h * w * c, 42, -1.f, 1.f);
  std::vector<bf16> gb(gf.size()), xb(xf.size());
  for (size_t i = 0; i < gf.size(); ++i) gb[i] = (bf16)gf[i], gf[i] = (float)gb[i];
  for (size_t i = 0; i < xf.size(); ++i) xb[i] = (bf16)xf[i], xf[i] = (float)xb[i];
  Pack pack = {{DY, bufOf(DY, gb)}, {X, bufOf(X, xb)}, {DW, fill(DW, 0.f)}};
  auto ws = workspaceFor(g);
  for (int rep = 0; rep < 2; ++rep)
    REQUIRE_OK(g.execute(gpu(), pack, ws));
  auto out = readBack<float>(pack[DW]);
  // physical layouts: dy [n][p][q][k], x [n][h][w][c], dw [k][r][s][c]
  std::vector<double> ref(k * 9 * c, 0.0);
  for (int64_t in = 0; in < n; ++in)
    for (int64_t p = 0; p < h; ++p)
      for (int64_t q = 0; q < w; ++q)
        for (int64_t r = 0; r < 3; ++r)
          for (int64_t s = 0; s < 3; ++s) {
            const int64_t ih = p - 1 + r, iw = q - 1 + s;
            if (ih < 0 || ih >= h || iw < 0 || iw >= w)
              continue;
            for (int64_t kk = 0; kk < k; ++kk) {
              const double gy = gf[((in * h + p) * w + q) * k + kk];
              for (int64_t cc = 0; cc < c; ++cc)
                ref[((kk * 3 + r) * 3 + s) * c + cc] +=
                    gy * xf[((in * h + ih) * w + iw) * c + cc];
            }
          }
  REQUIRE(out.size() == ref.size());
  double worst = 0, rms = 0;
  for (double r : ref)
    rms += r * r;
  rms = std::sqrt(rms / ref.size());
  for (size_t i = 0; i < ref.size(); ++i)
    worst = std::max(worst, std::fabs(out[i] - ref[i]) - 1e-3 * (std::fabs(ref[i]) + rms));
  CHECK(worst <= 0.0);
}

TEST("config 5a (reduced): int8 matmul is bit exact") {
  const int64_t m = 256, k = 512, n = 384;
  Graph g = newGraph("cfg5a", DataType::Int8);
  auto A = g.tensor(mk("a", {m, k}, {k, 1}, DataType::Int8));
  auto B = g.tensor(mk("b", {k, n}, {n, 1}, DataType::Int8));
  MatmulAttr ma;
  auto C = g.matmul(A, B, ma);
  C->setOutput(true).setDataType(DataType::Int32);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  std::mt19937 rng(5);
  std::vector<int8_t> a(m * k), b(k * n);
  for (auto &x : a) x = (int8_t)((int)(rng() % 255) - 127);
  for (auto &x : b) x = (int8_t)((int)(rng() % 255) - 127);
  Pack pack = {{A, bufOf(A, a)}, {B, bufOf(B, b)}, {C, fill(C, int32_t(0))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<int32_t>(pack[C]);
  bool exact = true;
  for (int64_t i = 0; i < m && exact; ++i)
    for (int64_t j = 0; j < n && exact; ++j) {
      int32_t acc = 0;
      for (int64_t kk = 0; kk < k; ++kk)
        acc += (int32_t)a[i * k + kk] * (int32_t)b[kk * n + j];
      exact = out[i * n + j] == acc;
    }
  CHECK(exact);
}

// worst violation of |got - ref| <= rtol * (|ref| + rms(ref)); <= 0 passes
template <typename T>
static double worstViolation(const std::vector<T> &got,
                             const std::vector<double> &ref, double rtol) {
  double rms = 0, worst = -1;
  for (double r : ref)
    rms += r * r;
  rms = std::sqrt(rms / (ref.empty() ? 1 : ref.size()));
  if (got.size() != ref.size())
    return 1e30;
  for (size_t i = 0; i < ref.size(); ++i)
    worst = std::max(worst, std::fabs((double)(float)got[i] - ref[i]) -
                                rtol * (std::fabs(ref[i]) + rms));
  return worst;
}

TEST("config 2 (reduced): bf16 rmsnorm + scalar MUL is one kernel, vs host loop") {
  const int64_t rows = 96, cols = 4096;
  const float eps = 1e-6f, mul = 0.5f;
  Graph g = newGraph("cfg2", DataType::BFloat16, DataType::Float);
  auto X = g.tensor(mk("x", {rows, cols}, {cols, 1}, DataType::BFloat16));
  auto S = g.tensor(mk("s", {1, cols}, {cols, 1}, DataType::BFloat16));
  RmsnormAttr ra;
  ra.setForwardPhase(NormFwdPhase::INFERENCE).setEpsilon(g.tensor(TensorAttr(eps)));
  auto [Y, R] = g.rmsnorm(X, S, ra);
  (void)R;
  PointwiseAttr pm;
  pm.setMode(PointwiseAttr::Mode::MUL);
  auto O = g.pointwise(Y, g.tensor(TensorAttr(mul)), pm);
  O->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1));
  auto xf = randomVec(rows * cols, 21, -3.f, 3.f), sf = randomVec(cols, 22, 0.9f, 1.1f);
  std::vector<bf16> xb(xf.size()), sb(sf.size());
  for (size_t i = 0; i < xf.size(); ++i) xb[i] = (bf16)xf[i], xf[i] = (float)xb[i];
  for (size_t i = 0; i < sf.size(); ++i) sb[i] = (bf16)sf[i], sf[i] = (float)sb[i];
  Pack pack = {{X, bufOf(X, xb)}, {S, bufOf(S, sb)}, {O, fill(O, bf16(0.f))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<bf16>(pack[O]);
  std::vector<double> ref(rows * cols);
  for (int64_t r = 0; r < rows; ++r) {
    double ss = 0;
    for (int64_t c = 0; c < cols; ++c)
      ss += (double)xf[r * cols + c] * xf[r * cols + c];
    const double inv = 1.0 / std::sqrt(ss / cols + eps);
    for (int64_t c = 0; c < cols; ++c)
      ref[r * cols + c] = xf[r * cols + c] * inv * sf[c] * mul;
  }
  CHECK(worstViolation(out, ref, 2e-2) <= 0.0);
}

TEST("config 4 (reduced): bf16 causal sdpa B1 H2 S320 D128 vs host loop") {
  const int64_t b = 1, h = 2, s = 320, d = 128;
  Graph g = newGraph("cfg4", DataType::BFloat16, DataType::Float);
  const Dims dims = {b, h, s, d};
  auto Q = g.tensor(mk("q", dims, contig(dims), DataType::BFloat16));
  auto K = g.tensor(mk("k", dims, contig(dims), DataType::BFloat16));
  auto V = g.tensor(mk("v", dims, contig(dims), DataType::BFloat16));
  SdpaAttr sa;
  sa.setIsCausal(true);
  auto O = g.sdpa(Q, K, V, nullptr, sa);
  O->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1));
  const size_t n = b * h * s * d;
  auto qf = randomVec(n, 31, -1.f, 1.f), kf = randomVec(n, 32, -1.f, 1.f),
       vf = randomVec(n, 33, -1.f, 1.f);
  std::vector<bf16> qb(n), kb(n), vb(n);
  for (size_t i = 0; i < n; ++i) {
    qb[i] = (bf16)qf[i], qf[i] = (float)qb[i];
    kb[i] = (bf16)kf[i], kf[i] = (float)kb[i];
    vb[i] = (bf16)vf[i], vf[i] = (float)vb[i];
  }
  Pack pack = {{Q, bufOf(Q, qb)}, {K, bufOf(K, kb)}, {V, bufOf(V, vb)},
               {O, fill(O, bf16(0.f))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<bf16>(pack[O]);
  std::vector<double> ref(n, 0.0), p(s);
  const double scale = 1.0 / std::sqrt((double)d);
  for (int64_t hh = 0; hh < b * h; ++hh)
    for (int64_t i = 0; i < s; ++i) { // samples/sdpa_utils.cpp:49-102
      double mx = -1e300, sum = 0;
      for (int64_t j = 0; j <= i; ++j) {
        double acc = 0;
        for (int64_t c = 0; c < d; ++c)
          acc += (double)qf[(hh * s + i) * d + c] * kf[(hh * s + j) * d + c];
        p[j] = acc * scale;
        mx = std::max(mx, p[j]);
      }
      for (int64_t j = 0; j <= i; ++j)
        p[j] = std::exp(p[j] - mx), sum += p[j];
      for (int64_t j = 0; j <= i; ++j)
        for (int64_t c = 0; c < d; ++c)
          ref[(hh * s + i) * d + c] += p[j] / sum * vf[(hh * s + j) * d + c];
    }
  CHECK(worstViolation(out, ref, 2e-2) <= 0.0);
}

// e4m3fn byte of the nearest representable value (round to nearest even,
// saturating at 448), by search over the 127 non-negative finite codes
static uint8_t toE4m3(float x) {
  auto val = [](int code) {
    const int e = code >> 3, m = code & 7;
    return e == 0 ? std::ldexp(m / 8.0, -6) : std::ldexp(1.0 + m / 8.0, e - 7);
  };
  const double a = std::fabs((double)x);
  int best = 0;
  for (int code = 1; code <= 0x7e; ++code) {
    const double db = std::fabs(val(best) - a), dc = std::fabs(val(code) - a);
    if (dc < db || (dc == db && (code & 1) == 0))
      best = code;
  }
  return (uint8_t)(best | (x < 0 ? 0x80 : 0));
}
static double fromE4m3(uint8_t bits) {
  const int code = bits & 0x7f, e = code >> 3, m = code & 7;
  const double v = e == 0 ? std::ldexp(m / 8.0, -6) : std::ldexp(1.0 + m / 8.0, e - 7);
  return bits & 0x80 ? -v : v;
}

TEST("config 5b (reduced): fp8 e4m3 matmul x scale -> bf16 is one kernel, vs host loop") {
  const int64_t m = 256, k = 512, n = 384;
  Graph g = newGraph("cfg5b", DataType::FP8E4M3, DataType::Float);
  auto A = g.tensor(mk("a", {m, k}, {k, 1}, DataType::FP8E4M3));
  auto B = g.tensor(mk("b", {k, n}, {n, 1}, DataType::FP8E4M3));
  MatmulAttr ma;
  auto C = g.matmul(A, B, ma);
  C->setDataType(DataType::Float);
  const float sa = 1.5f / 448.f, sb = 0.75f / 448.f;
  PointwiseAttr pm;
  pm.setMode(PointwiseAttr::Mode::MUL);
  auto O = g.pointwise(C, g.tensor(TensorAttr(sa * sb)), pm);
  O->setOutput(true).setDataType(DataType::BFloat16);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1));
  auto af = randomVec(m * k, 41, -448.f, 448.f), bf = randomVec(k * n, 42, -448.f, 448.f);
  std::vector<fp8e4m3> a8(af.size()), b8(bf.size());
  for (size_t i = 0; i < af.size(); ++i) a8[i].bits = toE4m3(af[i]);
  for (size_t i = 0; i < bf.size(); ++i) b8[i].bits = toE4m3(bf[i]);
  Pack pack = {{A, bufOf(A, a8)}, {B, bufOf(B, b8)}, {O, fill(O, bf16(0.f))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<bf16>(pack[O]);
  std::vector<double> ref(m * n, 0.0);
  for (int64_t i = 0; i < m; ++i)
    for (int64_t kk = 0; kk < k; ++kk) {
      const double av = fromE4m3(a8[i * k + kk].bits);
      for (int64_t j = 0; j < n; ++j)
        ref[i * n + j] += av * fromE4m3(b8[kk * n + j].bits);
    }
  for (double &r : ref)
    r *= (double)(sa * sb);
  CHECK(worstViolation(out, ref, 2e-2) <= 0.0);
}

TEST("fused chain: bf16 matmul -> add bias -> gelu -> mul scalar is one kernel") {
  const int64_t m = 256, k = 256, n = 384;
  Graph g = newGraph("chain4", DataType::BFloat16, DataType::Float);
  auto A = g.tensor(mk("a", {m, k}, {k, 1}, DataType::BFloat16));
  auto B = g.tensor(mk("b", {k, n}, {n, 1}, DataType::BFloat16));
  auto Bias = g.tensor(mk("bias", {1, n}, {n, 1}, DataType::BFloat16));
  MatmulAttr ma;
  PointwiseAttr add, gelu, mul;
  add.setMode(PointwiseAttr::Mode::ADD);
  gelu.setMode(PointwiseAttr::Mode::GELU_FWD);
  mul.setMode(PointwiseAttr::Mode::MUL);
  auto C = g.matmul(A, B, ma);
  auto O = g.pointwise(g.pointwise(g.pointwise(C, Bias, add), gelu),
                       g.tensor(TensorAttr(0.25f)), mul);
  O->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(1));
  auto af = randomVec(m * k, 51, -1.f, 1.f), bf = randomVec(k * n, 52, -0.2f, 0.2f),
       cf = randomVec(n, 53, -1.f, 1.f);
  std::vector<bf16> ab(af.size()), bb(bf.size()), cb(cf.size());
  for (size_t i = 0; i < af.size(); ++i) ab[i] = (bf16)af[i], af[i] = (float)ab[i];
  for (size_t i = 0; i < bf.size(); ++i) bb[i] = (bf16)bf[i], bf[i] = (float)bb[i];
  for (size_t i = 0; i < cf.size(); ++i) cb[i] = (bf16)cf[i], cf[i] = (float)cb[i];
  Pack pack = {{A, bufOf(A, ab)}, {B, bufOf(B, bb)}, {Bias, bufOf(Bias, cb)},
               {O, fill(O, bf16(0.f))}};
  REQUIRE_OK(g.execute(gpu(), pack, workspaceFor(g)));
  auto out = readBack<bf16>(pack[O]);
  std::vector<double> ref(m * n, 0.0);
  for (int64_t i = 0; i < m; ++i)
    for (int64_t kk = 0; kk < k; ++kk)
      for (int64_t j = 0; j < n; ++j)
        ref[i * n + j] += (double)af[i * k + kk] * bf[kk * n + j];
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      const double x = ref[i * n + j] + cf[j];
      ref[i * n + j] = 0.25 * 0.5 * x * (1.0 + std::erf(x / std::sqrt(2.0)));
    }
  CHECK(worstViolation(out, ref, 2e-2) <= 0.0);
}

TEST("unfused chain uses the workspace for virtual tensors") {
  Graph g = newGraph("chain", DataType::Float);
  auto A = g.tensor(mk("a", {64, 32}, {32, 1}, DataType::Float));
  PointwiseAttr p1, p2, p3;
  p1.setMode(PointwiseAttr::Mode::EXP);
  p2.setMode(PointwiseAttr::Mode::LOG);
  p3.setMode(PointwiseAttr::Mode::ADD);
  auto e = g.pointwise(A, p1);
  auto l = g.pointwise(e, p2);
  auto O = g.pointwise(l, A, p3);
  O->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(gpu(), true));
  CHECK(g.getKernelCount() == std::optional<size_t>(3));
  auto ws = workspaceFor(g);
  REQUIRE(ws != nullptr);
  auto a = randomVec(64 * 32, 9, -2.f, 2.f);
  Pack pack = {{A, bufOf(A, a)}, {O, fill(O, 0.f)}};
  REQUIRE_OK(g.execute(gpu(), pack, ws));
  auto out = readBack<float>(pack[O]);
  bool okAll = true;
  for (size_t i = 0; i < a.size(); ++i)
    okAll = okAll && std::fabs(out[i] - 2.f * a[i]) < 1e-4f;
  CHECK(okAll);
}

// ---- HIP interop -------------------------------------------------------------
TEST("interop: caller-owned stream and imported device pointers") {
  hipStream_t stream;
  REQUIRE(hipStreamCreate(&stream) == hipSuccess);
  REQUIRE_ASSIGN(Handle h, Handle::create(Backend::AMDGPU, 0,
                                          reinterpret_cast<uintptr_t>(stream)));
  const size_t n = 1024;
  float *a = nullptr, *o = nullptr;
  REQUIRE(hipMalloc(reinterpret_cast<void **>(&a), n * 4) == hipSuccess);
  REQUIRE(hipMalloc(reinterpret_cast<void **>(&o), n * 4) == hipSuccess);
  std::vector<float> host(n, -3.f);
  REQUIRE(hipMemcpy(a, host.data(), n * 4, hipMemcpyHostToDevice) == hipSuccess);
  Graph g = newGraph("interop", DataType::Float);
  auto A = g.tensor(mk("a", {32, 32}, {32, 1}, DataType::Float));
  PointwiseAttr p;
  p.setMode(PointwiseAttr::Mode::ABS);
  auto O = g.pointwise(A, p);
  O->setOutput(true);
  REQUIRE_OK(g.validate());
  REQUIRE_OK(g.compile(h, true));
  REQUIRE_ASSIGN(auto wsz, g.getWorkspaceSize());
  CHECK(wsz.has_value());
  REQUIRE_ASSIGN(Buffer ab, Buffer::import(a, n * 4, DataType::Float));
  REQUIRE_ASSIGN(Buffer ob, Buffer::import(o, n * 4, DataType::Float));
  Pack pack = {{A, std::make_shared<Buffer>(std::move(ab))},
               {O, std::make_shared<Buffer>(std::move(ob))}};
  REQUIRE_OK(g.execute(h, pack, nullptr));
  // stream-ordered: the result is visible after the caller's own sync
  REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
  REQUIRE(hipMemcpy(host.data(), o, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
  CHECK(allEqual(host, 3.f));
  std::vector<float> viaRead;
  REQUIRE_OK(pack[O]->read(h, viaRead));
  CHECK(allEqual(viaRead, 3.f));
  // a CPU-compiled plan is refused by an AMDGPU handle, and vice versa
  REQUIRE_ASSIGN(Handle cpu, Handle::create(Backend::CPU));
  CHECK_ERROR(g.execute(cpu, pack, nullptr), ErrorCode::InvalidArgument,
              "Graph::execute got a handle for backend CPU, but the loaded "
              "artifact uses backend AMDGPU");
  (void)hipFree(a);
  (void)hipFree(o);
  (void)hipStreamDestroy(stream);
}

int main(int argc, char **argv) { return mini::run(argc, argv); }
