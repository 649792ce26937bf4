// Benchmark driver over the C++ graph API: the counterpart of the reference's
// benchmarks/driver.cpp (subcommands and MIOpen-style flags: :878-965 conv,
// :973-1016 layernorm, :1019-1066 matmul, :1068-1110 sdpa; --iter / --device:
// :1277-1287).  Each command builds one graph, compiles it once, runs --iter
// back-to-back executes on the handle's stream (reference :864-865) and
// prints one CSV row:
//   name,iter,dispatch_count,avg_us,work,unit_per_s
// `dispatch_count` is the number of kernels the plan launches per execute.
// Inputs are constant fills like the reference's.  Extras beyond the
// reference: `rmsnorm` subcommand (`--mul s` fuses a scalar multiply), `--relu`
// for conv, int8 / fp8 matmul types, `--out_scale s` (matmul output x scalar).
#include <fusilli.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

using namespace fusilli;
using Dims = std::vector<int64_t>;
using TensorPtr = std::shared_ptr<TensorAttr>;
using Pack = std::unordered_map<TensorPtr, std::shared_ptr<Buffer>>;

namespace {

[[noreturn]] void die(const std::string &msg) {
  std::fprintf(stderr, "driver: %s\n", msg.c_str());
  std::exit(1);
}
#define OK(expr)                                                               \
  do {                                                                         \
    auto st_ = (expr);                                                         \
    if (isError(st_))                                                          \
      die(std::string(#expr) + ": " + ErrorObject(st_).getMessage());          \
  } while (0)

// argv after the subcommand -> {flag: value}; flags without value map to "1"
struct Args {
  std::map<std::string, std::string> kv;
  bool has(const std::string &k) const { return kv.count(k) != 0; }
  int64_t i(const std::string &a, const std::string &b, int64_t def) const {
    if (has(a))
      return std::atoll(kv.at(a).c_str());
    if (!b.empty() && has(b))
      return std::atoll(kv.at(b).c_str());
    return def;
  }
  std::string s(const std::string &a, const std::string &b,
                const std::string &def) const {
    if (has(a))
      return kv.at(a);
    if (!b.empty() && has(b))
      return kv.at(b);
    return def;
  }
};
Args parse(int argc, char **argv, int from) {
  Args a;
  for (int i = from; i < argc; ++i) {
    std::string k = argv[i];
    if (k.rfind("-", 0) != 0)
      die("unexpected argument " + k);
    const bool value = i + 1 < argc && (argv[i + 1][0] != '-' ||
                                        std::isdigit((unsigned char)argv[i + 1][1]));
    a.kv[k] = value ? argv[++i] : "1";
  }
  return a;
}

DataType dtypeOf(const std::string &t) {
  if (t == "f32")
    return DataType::Float;
  if (t == "f16")
    return DataType::Half;
  if (t == "bf16")
    return DataType::BFloat16;
  if (t == "i8" || t == "si8")
    return DataType::Int8;
  if (t == "i32" || t == "si32")
    return DataType::Int32;
  if (t == "f8E4M3FN" || t == "fp8")
    return DataType::FP8E4M3;
  die("unknown type " + t);
}

Dims contig(const Dims &d) {
  Dims s(d.size(), 1);
  for (int i = (int)d.size() - 2; i >= 0; --i)
    s[i] = s[i + 1] * d[i + 1];
  return s;
}
Dims chlast(const Dims &d) { // logical N C spatial..., stored N spatial... C
  Dims s(d.size());
  s[1] = 1;
  int64_t run = d[1];
  for (int i = (int)d.size() - 1; i >= 2; --i) {
    s[i] = run;
    run *= d[i];
  }
  s[0] = run;
  return s;
}
TensorAttr mk(const std::string &name, const Dims &dim, const Dims &stride,
              DataType dt) {
  return TensorAttr().setName(name).setDim(dim).setStride(stride).setDataType(dt);
}

// constant-filled device buffer shaped like the tensor's physical dims
std::shared_ptr<Buffer> constant(const Handle &h, const TensorPtr &t, float v) {
  std::vector<size_t> shape;
  size_t n = 1;
  for (int64_t d : t->getPhysicalDim()) {
    shape.push_back((size_t)d);
    n *= (size_t)d;
  }
  auto wrap = [&](auto e) {
    if (isError(e))
      die("allocate " + t->getName() + ": " + ErrorObject(e).getMessage());
    return std::make_shared<Buffer>(std::move(*e));
  };
  switch (t->getDataType()) {
  case DataType::Float:
    return wrap(Buffer::allocate(h, shape, std::vector<float>(n, v)));
  case DataType::Half:
    return wrap(Buffer::allocate(h, shape, std::vector<half>(n, (half)v)));
  case DataType::BFloat16:
    return wrap(Buffer::allocate(h, shape, std::vector<bf16>(n, (bf16)v)));
  case DataType::Int8:
    return wrap(Buffer::allocate(h, shape, std::vector<int8_t>(n, (int8_t)v)));
  case DataType::Int32:
    return wrap(Buffer::allocate(h, shape, std::vector<int32_t>(n, (int32_t)v)));
  case DataType::FP8E4M3: // 0x38 = 1.0 in e4m3
    return wrap(Buffer::allocate(h, shape, std::vector<fp8e4m3>(n, fp8e4m3{0x38})));
  default:
    die("no fill for this dtype");
  }
}

struct Run {
  std::string name;
  double work = 0; // FLOP or bytes
  const char *unit = "TFLOP/s";
};

void timeGraph(const Handle &h, Graph &g, Pack &pack, const Run &r, int iter) {
  OK(g.validate());
  OK(g.compile(h, /*remove=*/true));
  auto ws = g.getWorkspaceSize();
  std::shared_ptr<Buffer> wsBuf;
  if (!isError(ws) && ws->has_value() && **ws > 0) {
    auto b = Buffer::allocateRaw(h, **ws);
    if (isError(b))
      die("workspace allocation failed");
    wsBuf = std::make_shared<Buffer>(std::move(*b));
  }
  fhip_ctx *ctx = h.getContext();
  for (int i = 0; i < 3; ++i)
    OK(g.execute(h, pack, wsBuf));
  fhip_event *e0 = nullptr, *e1 = nullptr;
  if (fhip_event_create(ctx, &e0) || fhip_event_create(ctx, &e1))
    die(fhip_last_error(ctx));
  fhip_event_record(ctx, e0);
  for (int i = 0; i < iter; ++i)
    OK(g.execute(h, pack, wsBuf));
  fhip_event_record(ctx, e1);
  fhip_stream_sync(ctx);
  float ms = 0;
  fhip_event_elapsed_ms(ctx, e0, e1, &ms);
  fhip_event_destroy(ctx, e0);
  fhip_event_destroy(ctx, e1);
  const double us = ms * 1e3 / iter;
  const size_t kernels = g.getKernelCount().value_or(0);
  std::printf("name,iter,dispatch_count,avg_us,work,%s\n", r.unit);
  std::printf("%s,%d,%zu,%.3f,%.0f,%.3f\n", r.name.c_str(), iter, kernels, us,
              r.work, r.work / us / 1e6);
}

void runConv(const Handle &h, const Args &a, int iter) {
  const int64_t n = a.i("-n", "--batchsize", 1), c = a.i("-c", "--in_channels", 1),
                H = a.i("-H", "--in_h", 1), W = a.i("-W", "--in_w", 1),
                k = a.i("-k", "--out_channels", 1), y = a.i("-y", "--fil_h", 1),
                x = a.i("-x", "--fil_w", 1), p = a.i("-p", "--pad_h", 0),
                q = a.i("-q", "--pad_w", 0), u = a.i("-u", "--conv_stride_h", 1),
                v = a.i("-v", "--conv_stride_w", 1), l = a.i("-l", "--dilation_h", 1),
                j = a.i("-j", "--dilation_w", 1), gcount = a.i("-g", "--group_count", 1);
  // MIOpen's direction flag, as in the reference driver (driver.cpp:1159-1167):
  // 1 forward, 2 data gradient, 4 weight gradient
  const int64_t mode = a.i("-F", "--mode", 1);
  if (mode != 1 && mode != 2 && mode != 4)
    die("conv: -F must be 1 (forward), 2 (data gradient) or 4 (weight gradient)");
  const DataType dt = a.has("--bf16") ? DataType::BFloat16
                      : a.has("--fp16") ? DataType::Half : DataType::Float;
  const bool nhwc = a.s("--in_layout", "", "NCHW") == "NHWC";
  auto lay = [&](const Dims &d) { return nhwc ? chlast(d) : contig(d); };
  if (mode != 1) {
    const Dims xd = {n, c, H, W}, wd = {k, c / gcount, y, x};
    const Dims yd = getConvInferredOutputShape(xd, wd, {l, j}, {p, q}, {u, v});
    Graph g;
    g.setName(mode == 2 ? "benchmark_conv_dgrad" : "benchmark_conv_wgrad")
        .setIODataType(dt).setIntermediateDataType(DataType::Float)
        .setComputeDataType(DataType::Float);
    auto DY = g.tensor(mk("dy", yd, lay(yd), dt));
    TensorPtr IN, OUT;
    if (mode == 2) {
      IN = g.tensor(mk("w", wd, lay(wd), dt));
      ConvDGradAttr da;
      da.setPadding({p, q}).setStride({u, v}).setDilation({l, j});
      OUT = g.convDGrad(DY, IN, da);
      OUT->setDim(xd);
    } else {
      IN = g.tensor(mk("x", xd, lay(xd), dt));
      ConvWGradAttr wa;
      wa.setPadding({p, q}).setStride({u, v}).setDilation({l, j});
      OUT = g.convWGrad(DY, IN, wa);
      OUT->setDim(wd);
    }
    OUT->setOutput(true).setDataType(dt);
    OK(g.validate());
    Pack pack = {{DY, constant(h, DY, 1.f)}, {IN, constant(h, IN, 1.f)},
                 {OUT, constant(h, OUT, 0.f)}};
    Run r{mode == 2 ? "conv_dgrad" : "conv_wgrad",
          2.0 * n * yd[2] * yd[3] * k * (c / gcount) * y * x};
    timeGraph(h, g, pack, r, iter);
    return;
  }
  Graph g;
  g.setName("benchmark_conv_fprop").setIODataType(dt)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  auto X = g.tensor(mk("x", {n, c, H, W}, lay({n, c, H, W}), dt));
  auto Wt = g.tensor(mk("w", {k, c / gcount, y, x}, lay({k, c / gcount, y, x}), dt));
  ConvFPropAttr ca;
  ca.setPadding({p, q}).setStride({u, v}).setDilation({l, j});
  auto Y = g.convFProp(X, Wt, ca);
  Pack pack;
  TensorPtr B;
  if (a.has("-b") || a.has("--bias")) {
    B = g.tensor(mk("bias", {1, k, 1, 1}, {k, 1, k, k}, dt));
    PointwiseAttr add;
    add.setMode(PointwiseAttr::Mode::ADD);
    Y = g.pointwise(Y, B, add);
  }
  if (a.has("--relu")) {
    PointwiseAttr rl;
    rl.setMode(PointwiseAttr::Mode::RELU_FWD);
    Y = g.pointwise(Y, rl);
  }
  if (a.has("--mul")) { // y * scalar fused behind the norm
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    Y = g.pointwise(
        Y, g.tensor(TensorAttr((float)std::atof(a.s("--mul", "", "1").c_str()))), mul);
  }
  Y->setOutput(true).setDataType(dt);
  OK(g.validate());
  pack[X] = constant(h, X, 1.f);
  pack[Wt] = constant(h, Wt, 1.f);
  if (B)
    pack[B] = constant(h, B, 1.f);
  pack[Y] = constant(h, Y, 0.f);
  const Dims yd = Y->getDim();
  Run r{"conv_fprop", 2.0 * n * yd[2] * yd[3] * k * (c / gcount) * y * x};
  timeGraph(h, g, pack, r, iter);
}

void runMatmul(const Handle &h, const Args &a, int iter) {
  const int64_t M = a.i("-M", "--m", 1), N = a.i("-N", "--n", 1),
                K = a.i("-K", "--k", 1), Bt = a.i("-B", "--b", 1);
  const DataType at = dtypeOf(a.s("--a_type", "", "f32")),
                 bt = dtypeOf(a.s("--b_type", "", "f32")),
                 ot = dtypeOf(a.s("--out_type", "", "f32"));
  Graph g;
  g.setName("benchmark_matmul").setIODataType(at)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  const Dims ad = {Bt, M, K}, bd = {Bt, K, N};
  const Dims as = a.has("--transA") ? Dims{M * K, 1, M} : contig(ad);
  const Dims bs = a.has("--transB") ? Dims{K * N, 1, K} : contig(bd);
  auto A = g.tensor(mk("a", ad, as, at));
  auto B = g.tensor(mk("b", bd, bs, bt));
  MatmulAttr ma;
  auto C = g.matmul(A, B, ma);
  TensorPtr bias;
  if (a.has("--bias")) {
    bias = g.tensor(mk("bias", {1, 1, N}, {N, N, 1},
                       dtypeOf(a.s("--bias_type", "", a.s("--out_type", "", "f32")))));
    PointwiseAttr add;
    add.setMode(PointwiseAttr::Mode::ADD);
    C = g.pointwise(C, bias, add);
  }
  if (a.has("--out_scale")) { // C * scalar, as the fp8 configuration dequantises
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    C->setDataType(DataType::Float);
    C = g.pointwise(
        C, g.tensor(TensorAttr((float)std::atof(a.s("--out_scale", "", "1").c_str()))),
        mul);
  }
  C->setOutput(true).setDataType(ot);
  OK(g.validate());
  Pack pack = {{A, constant(h, A, 1.f)}, {B, constant(h, B, 1.f)},
               {C, constant(h, C, 0.f)}};
  if (bias)
    pack[bias] = constant(h, bias, 1.f);
  Run r{"matmul", 2.0 * Bt * M * N * K};
  timeGraph(h, g, pack, r, iter);
}

void runSdpa(const Handle &h, const Args &a, int iter) {
  const int64_t B = a.i("-B", "--batch", 1), Hq = a.i("--heads_q", "", 1),
                Hkv = a.i("--heads_kv", "", Hq), Sq = a.i("--seq_q", "", 1),
                Skv = a.i("--seq_kv", "", Sq), D = a.i("-d", "--head_dim", 64);
  const DataType dt = dtypeOf(a.s("-t", "--type", "f16"));
  Graph g;
  g.setName("benchmark_sdpa").setIODataType(dt)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  auto Q = g.tensor(mk("q", {B, Hq, Sq, D}, contig({B, Hq, Sq, D}), dt));
  auto K = g.tensor(mk("k", {B, Hkv, Skv, D}, contig({B, Hkv, Skv, D}), dt));
  auto V = g.tensor(mk("v", {B, Hkv, Skv, D}, contig({B, Hkv, Skv, D}), dt));
  SdpaAttr sa;
  sa.setIsCausal(a.has("--causal")).setEnableGqa(a.has("--gqa") || Hq != Hkv);
  if (a.has("-s") || a.has("--scale"))
    sa.setScale((float)std::atof(a.s("-s", "--scale", "1").c_str()));
  auto O = g.sdpa(Q, K, V, nullptr, sa);
  O->setOutput(true).setDataType(dt);
  OK(g.validate());
  Pack pack = {{Q, constant(h, Q, 0.01f)}, {K, constant(h, K, 0.01f)},
               {V, constant(h, V, 0.01f)}, {O, constant(h, O, 0.f)}};
  Run r{"sdpa", 4.0 * B * Hq * Sq * Skv * D * (a.has("--causal") ? 0.5 : 1.0)};
  timeGraph(h, g, pack, r, iter);
}

void runNorm(const Handle &h, const Args &a, int iter, bool layer) {
  Dims dims;
  {
    std::string x = a.s("-X", "--input", "");
    if (x.empty())
      die("norm: -X <d0xd1x...> is required");
    size_t pos = 0;
    while (pos <= x.size()) {
      const size_t e = x.find('x', pos);
      dims.push_back(std::atoll(x.substr(pos, e - pos).c_str()));
      if (e == std::string::npos)
        break;
      pos = e + 1;
    }
  }
  const DataType dt = dtypeOf(a.s("-t", "--type", "f32"));
  Graph g;
  g.setName(layer ? "benchmark_layernorm" : "benchmark_rmsnorm").setIODataType(dt)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  auto X = g.tensor(mk("x", dims, contig(dims), dt));
  Dims sd = dims;
  sd[0] = 1;
  const bool affine = a.has("--elementwise_affine") || !layer;
  TensorPtr S, Bi;
  if (affine)
    S = g.tensor(mk("scale", sd, contig(sd), dt));
  auto eps = g.tensor(TensorAttr((float)std::atof(a.s("-e", "--eps", "1e-5").c_str())));
  Pack pack;
  TensorPtr Y;
  if (layer) {
    if (affine)
      Bi = g.tensor(mk("bias", sd, contig(sd), dt));
    LayernormAttr la;
    la.setEpsilon(eps).setForwardPhase(NormFwdPhase::INFERENCE);
    auto outs = g.layernorm(X, S, Bi, la);
    Y = outs[0];
  } else {
    RmsnormAttr ra;
    ra.setEpsilon(eps).setForwardPhase(NormFwdPhase::INFERENCE);
    auto outs = g.rmsnorm(X, S, ra);
    Y = outs[0];
  }
  if (a.has("--mul")) { // y * scalar fused behind the norm
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    Y = g.pointwise(
        Y, g.tensor(TensorAttr((float)std::atof(a.s("--mul", "", "1").c_str()))), mul);
  }
  Y->setOutput(true).setDataType(dt);
  OK(g.validate());
  pack[X] = constant(h, X, 1.f);
  if (S)
    pack[S] = constant(h, S, 2.f);
  if (Bi)
    pack[Bi] = constant(h, Bi, 0.5f);
  pack[Y] = constant(h, Y, 0.f);
  double n = 1;
  for (int64_t d : dims)
    n *= (double)d;
  const double es = dt == DataType::Float ? 4 : 2;
  Run r{layer ? "layernorm" : "rmsnorm", 2.0 * n * es, "TB/s"};
  timeGraph(h, g, pack, r, iter);
}

} // namespace

int main(int argc, char **argv) {
  int iter = 100, device = 0, i = 1;
  for (; i < argc; ++i) {
    const std::string k = argv[i];
    if ((k == "--iter" || k == "-i") && i + 1 < argc)
      iter = std::atoi(argv[++i]);
    else if ((k == "--device" || k == "-D") && i + 1 < argc)
      device = std::atoi(argv[++i]);
    else if (k == "--dump" || k == "-d")
      ; // nothing to dump: there is no intermediate IR
    else
      break;
  }
  if (i >= argc)
    die("usage: driver [--device N] [--iter N] <conv|matmul|sdpa|layernorm|rmsnorm> flags...");
  const std::string cmd = argv[i];
  const Args a = parse(argc, argv, i + 1);
  auto he = Handle::create(Backend::AMDGPU, device);
  if (isError(he))
    die("Handle::create: " + ErrorObject(he).getMessage());
  Handle h = std::move(*he);
  if (cmd == "conv")
    runConv(h, a, iter);
  else if (cmd == "matmul")
    runMatmul(h, a, iter);
  else if (cmd == "sdpa")
    runSdpa(h, a, iter);
  else if (cmd == "layernorm")
    runNorm(h, a, iter, true);
  else if (cmd == "rmsnorm")
    runNorm(h, a, iter, false);
  else
    die("unknown subcommand " + cmd);
  return 0;
}
