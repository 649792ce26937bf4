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
#include <optional>
#include <set>
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

// argv after the subcommand -> {flag: value}; flags without value map to "1".
// Every lookup marks its keys as known; finish() rejects whatever the
// subcommand never asked for, so a flag this driver does not implement can
// not silently change the problem that is timed.
struct Args {
  std::map<std::string, std::string> kv;
  mutable std::set<std::string> known;
  bool has(const std::string &k) const {
    known.insert(k);
    return kv.count(k) != 0;
  }
  bool flag(const std::string &a, const std::string &b = "") const {
    const bool x = has(a), y = !b.empty() && has(b);
    return x || y;
  }
  int64_t i(const std::string &a, const std::string &b, int64_t def) const {
    const bool x = has(a), y = !b.empty() && has(b);
    if (x)
      return std::atoll(kv.at(a).c_str());
    if (y)
      return std::atoll(kv.at(b).c_str());
    return def;
  }
  // a required integer option (the reference marks it ->required())
  int64_t req(const std::string &a, const std::string &b) const {
    if (!flag(a, b))
      die("missing required option " + (b.empty() ? a : b + "," + a));
    return i(a, b, 0);
  }
  std::string s(const std::string &a, const std::string &b,
                const std::string &def) const {
    const bool x = has(a), y = !b.empty() && has(b);
    if (x)
      return kv.at(a);
    if (y)
      return kv.at(b);
    return def;
  }
  void finish(const std::string &cmd) const {
    for (const auto &e : kv)
      if (!known.count(e.first))
        die(cmd + ": unknown option " + e.first);
  }
};
Args parse(int argc, char **argv, int from) {
  Args a;
  for (int i = from; i < argc; ++i) {
    std::string k = argv[i];
    if (k.rfind("-", 0) != 0)
      die("unexpected argument " + k);
    const bool value = i + 1 < argc && (argv[i + 1][0] != '-' ||
                                        std::isdigit((unsigned char)argv[i + 1][1]) ||
                                        argv[i + 1][1] == '.');
    if (a.kv.count(k))
      die("option " + k + " given twice");
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

// The device handle, created on first use: flags are checked first, so a
// rejected command line never touches a device.
struct LazyHandle {
  int device = 0;
  std::optional<Handle> handle;
  const Handle &get() {
    if (!handle) {
      auto he = Handle::create(Backend::AMDGPU, device);
      if (isError(he))
        die("Handle::create: " + ErrorObject(he).getMessage());
      handle.emplace(std::move(*he));
    }
    return *handle;
  }
};

struct Run {
  std::string name;
  double work = 0; // FLOP or bytes
  const char *unit = "TFLOP/s";
};

int g_warmup = 3; // untimed executes before the --iter loop (--warmup)

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
  for (int i = 0; i < g_warmup; ++i)
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

// Strides of `dims` under a layout name of the reference's list
// (benchmarks/driver.cpp:39-40).
Dims layoutStrides(const Dims &dims, const std::string &layout, const char *what) {
  auto st = generateStrideFromLayout(dims, layout);
  if (isError(st))
    die(std::string("conv: ") + what + ": " + ErrorObject(st).getMessage());
  return *st;
}

// Flags and graph construction follow the reference driver
// (benchmarks/driver.cpp:114-247 forward, :249-511 gradients, :874-965 flags,
// :1114-1170 checks): 2-D or 3-D, one layout per tensor, groups, bias.
void runConv(LazyHandle &lh, const Args &a, int iter) {
  const int64_t sdim = a.req("--spatial_dim", "");
  if (sdim != 2 && sdim != 3)
    die("conv: --spatial_dim must be 2 or 3");
  const int64_t n = a.req("-n", "--batchsize"), c = a.req("-c", "--in_channels"),
                D = a.i("--in_d", "", -1), H = a.req("-H", "--in_h"),
                W = a.req("-W", "--in_w"), k = a.req("-k", "--out_channels"),
                z = a.i("--fil_d", "", -1), y = a.req("-y", "--fil_h"),
                x = a.req("-x", "--fil_w"), o = a.i("--pad_d", "", -1),
                p = a.req("-p", "--pad_h"), q = a.req("-q", "--pad_w"),
                t = a.i("--conv_stride_d", "", -1), u = a.req("-u", "--conv_stride_h"),
                v = a.req("-v", "--conv_stride_w"), m = a.i("--dilation_d", "", -1),
                l = a.req("-l", "--dilation_h"), j = a.req("-j", "--dilation_w"),
                gcount = a.i("-g", "--group_count", 1);
  // MIOpen's direction flag, as in the reference driver (driver.cpp:1159-1167):
  // 1 forward, 2 data gradient, 4 weight gradient
  const int64_t mode = a.req("-F", "--mode");
  if (mode != 1 && mode != 2 && mode != 4)
    die("conv: -F must be 1 (forward), 2 (data gradient) or 4 (weight gradient)");
  if (a.flag("--fp16") && a.flag("--bf16"))
    die("conv: --fp16 excludes --bf16");
  const DataType dt = a.flag("--bf16") ? DataType::BFloat16
                      : a.flag("--fp16") ? DataType::Half : DataType::Float;
  const std::string inL = a.s("--in_layout", "", ""), filL = a.s("--fil_layout", "", ""),
                    outL = a.s("--out_layout", "", "");
  if (inL.empty() || filL.empty() || outL.empty())
    die("conv: --in_layout, --fil_layout and --out_layout are required");
  const size_t rank = (size_t)sdim + 2;
  if (inL.size() != rank || filL.size() != rank || outL.size() != rank)
    die("conv: Detected at least one invalid {input, filter, output} layout for " +
        std::to_string(sdim) + "D convolution.");
  if (sdim == 3 && (D == -1 || z == -1 || t == -1 || o == -1 || m == -1))
    die("conv: Detected at least one of {in_d, fil_d, conv_stride_d, pad_d, "
        "dilation_d} that was not set for 3D convolution.");
  if (gcount <= 0 || c % gcount != 0 || k % gcount != 0)
    die("conv: Detected invalid group count.");
  const bool bias = a.flag("-b", "--bias"), relu = a.flag("--relu"),
             mul = a.flag("--mul");
  const float mulBy = (float)std::atof(a.s("--mul", "", "1").c_str());
  a.finish("conv");
  const Handle &h = lh.get();

  const int64_t fc = c / gcount;
  const Dims xd = sdim == 2 ? Dims{n, c, H, W} : Dims{n, c, D, H, W};
  const Dims wd = sdim == 2 ? Dims{k, fc, y, x} : Dims{k, fc, z, y, x};
  const Dims cs = sdim == 2 ? Dims{u, v} : Dims{t, u, v};
  const Dims cp = sdim == 2 ? Dims{p, q} : Dims{o, p, q};
  const Dims cd = sdim == 2 ? Dims{l, j} : Dims{m, l, j};
  const Dims yd = getConvInferredOutputShape(xd, wd, cd, cp, cs);
  double taps = 1, opix = 1;
  for (size_t i = 2; i < rank; ++i)
    taps *= (double)wd[i], opix *= (double)yd[i];
  const double flop = 2.0 * n * opix * k * fc * taps;
  // one name per configuration, like the reference's (cache files are per
  // graph name)
  char nm[512];
  std::snprintf(nm, sizeof(nm),
                "n%lld_c%lld_d%lld_h%lld_w%lld_g%lld_k%lld_z%lld_y%lld_x%lld_t%lld_u%lld_"
                "v%lld_o%lld_p%lld_q%lld_m%lld_l%lld_j%lld_S%lld_I%s_O%s_F%s_bias%d",
                (long long)n, (long long)c, (long long)D, (long long)H, (long long)W,
                (long long)gcount, (long long)k, (long long)z, (long long)y,
                (long long)x, (long long)t, (long long)u, (long long)v, (long long)o,
                (long long)p, (long long)q, (long long)m, (long long)l, (long long)j,
                (long long)sdim, inL.c_str(), outL.c_str(), filL.c_str(), (int)bias);
  Dims biasDim(rank, 1), biasStride(rank, k);
  biasDim[1] = k;
  biasStride[1] = 1;

  if (mode != 1) {
    if (relu || mul)
      die("conv: --relu / --mul apply to the forward mode only");
    Graph g;
    g.setName(std::string(mode == 2 ? "benchmark_conv_dgrad_" : "benchmark_conv_wgrad_") + nm)
        .setIODataType(DataType::Float).setIntermediateDataType(DataType::Float)
        .setComputeDataType(DataType::Float);
    auto DY = g.tensor(mk("dy", yd, layoutStrides(yd, outL, "--out_layout"), dt));
    TensorPtr IN, OUT, DB;
    if (mode == 2) {
      IN = g.tensor(mk("filter", wd, layoutStrides(wd, filL, "--fil_layout"), dt));
      ConvDGradAttr da;
      da.setPadding(cp).setStride(cs).setDilation(cd);
      OUT = g.convDGrad(DY, IN, da);
      OUT->setDim(xd).setStride(layoutStrides(xd, inL, "--in_layout"));
    } else {
      IN = g.tensor(mk("input", xd, layoutStrides(xd, inL, "--in_layout"), dt));
      ConvWGradAttr wa;
      wa.setPadding(cp).setStride(cs).setDilation(cd);
      OUT = g.convWGrad(DY, IN, wa);
      OUT->setDim(wd).setStride(layoutStrides(wd, filL, "--fil_layout"));
    }
    OUT->setOutput(true).setDataType(dt);
    if (bias) { // the bias gradient: DY summed over batch and space (driver.cpp:319-330)
      ReductionAttr ra;
      ra.setMode(ReductionAttr::Mode::SUM);
      DB = g.reduction(DY, ra);
      DB->setDim(biasDim).setStride(biasStride).setOutput(true).setDataType(dt);
    }
    OK(g.validate());
    Pack pack = {{DY, constant(h, DY, 1.f)}, {IN, constant(h, IN, 1.f)},
                 {OUT, constant(h, OUT, 0.f)}};
    if (DB)
      pack[DB] = constant(h, DB, 0.f);
    Run r{mode == 2 ? "conv_dgrad" : "conv_wgrad", flop};
    timeGraph(h, g, pack, r, iter);
    return;
  }
  Graph g;
  g.setName(std::string("benchmark_conv_fprop_") + nm).setIODataType(DataType::Float)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  auto X = g.tensor(mk("input", xd, layoutStrides(xd, inL, "--in_layout"), dt));
  auto Wt = g.tensor(mk("filter", wd, layoutStrides(wd, filL, "--fil_layout"), dt));
  ConvFPropAttr ca;
  ca.setPadding(cp).setStride(cs).setDilation(cd);
  auto Y = g.convFProp(X, Wt, ca);
  Pack pack;
  TensorPtr B;
  if (bias) {
    B = g.tensor(mk("bias", biasDim, biasStride, dt));
    PointwiseAttr add;
    add.setMode(PointwiseAttr::Mode::ADD);
    Y = g.pointwise(Y, B, add);
  }
  if (relu) {
    PointwiseAttr rl;
    rl.setMode(PointwiseAttr::Mode::RELU_FWD);
    Y = g.pointwise(Y, rl);
  }
  if (mul) { // y * scalar fused behind the convolution
    PointwiseAttr pm;
    pm.setMode(PointwiseAttr::Mode::MUL);
    Y = g.pointwise(Y, g.tensor(TensorAttr(mulBy)), pm);
  }
  // the output tensor in the layout --out_layout names (the reference lets
  // the output follow the input's format; naming it gives the same strides
  // for its own commands and honours the flag where the two differ)
  Y->setOutput(true).setDataType(dt).setDim(yd).setStride(
      layoutStrides(yd, outL, "--out_layout"));
  OK(g.validate());
  pack[X] = constant(h, X, 1.f);
  pack[Wt] = constant(h, Wt, 1.f);
  if (B)
    pack[B] = constant(h, B, 1.f);
  pack[Y] = constant(h, Y, 0.f);
  Run r{"conv_fprop", flop};
  timeGraph(h, g, pack, r, iter);
}

void runMatmul(LazyHandle &lh, const Args &a, int iter) {
  const int64_t M = a.req("-M", "--m"), N = a.req("-N", "--n"),
                K = a.req("-K", "--k"), Bt = a.i("-B", "--b", 1);
  const std::string atn = a.s("--a_type", "", ""), btn = a.s("--b_type", "", ""),
                    otn = a.s("--out_type", "", "");
  if (atn.empty() || btn.empty() || otn.empty())
    die("matmul: --a_type, --b_type and --out_type are required");
  const DataType at = dtypeOf(atn), bt = dtypeOf(btn), ot = dtypeOf(otn);
  const bool transA = a.flag("--transA"), transB = a.flag("--transB"),
             withBias = a.flag("--bias"), outScale = a.flag("--out_scale");
  const std::string biasType = a.s("--bias_type", "", otn);
  const float outScaleBy = (float)std::atof(a.s("--out_scale", "", "1").c_str());
  a.finish("matmul");
  const Handle &h = lh.get();
  Graph g;
  g.setName("benchmark_matmul_b" + std::to_string(Bt) + "_m" + std::to_string(M) +
            "_n" + std::to_string(N) + "_k" + std::to_string(K) + "_" + atn + "_" +
            btn + "_" + otn + (transA ? "_tA" : "") + (transB ? "_tB" : "") +
            (withBias ? "_bias" + biasType : "") + (outScale ? "_scaled" : ""))
      .setIODataType(at)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  const Dims ad = {Bt, M, K}, bd = {Bt, K, N};
  const Dims as = transA ? Dims{M * K, 1, M} : contig(ad);
  const Dims bs = transB ? Dims{K * N, 1, K} : contig(bd);
  auto A = g.tensor(mk("a", ad, as, at));
  auto B = g.tensor(mk("b", bd, bs, bt));
  MatmulAttr ma;
  auto C = g.matmul(A, B, ma);
  TensorPtr bias;
  if (withBias) {
    bias = g.tensor(mk("bias", {1, 1, N}, {N, N, 1}, dtypeOf(biasType)));
    PointwiseAttr add;
    add.setMode(PointwiseAttr::Mode::ADD);
    C = g.pointwise(C, bias, add);
  }
  if (outScale) { // C * scalar, as the fp8 configuration dequantises
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    C->setDataType(DataType::Float);
    C = g.pointwise(C, g.tensor(TensorAttr(outScaleBy)), mul);
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

void runSdpa(LazyHandle &lh, const Args &a, int iter) {
  const int64_t B = a.req("-B", "--batch"), Hq = a.req("--heads_q", ""),
                Hkv = a.req("--heads_kv", ""), Sq = a.req("--seq_q", ""),
                Skv = a.req("--seq_kv", ""), D = a.req("-d", "--head_dim");
  const std::string tn = a.s("-t", "--type", "");
  if (tn.empty())
    die("sdpa: --type is required");
  const DataType dt = dtypeOf(tn);
  const bool causal = a.flag("--causal"), withMask = a.flag("--mask"),
             gqa = a.flag("--gqa"), hasScale = a.flag("-s", "--scale");
  const float scaleBy = (float)std::atof(a.s("-s", "--scale", "1").c_str());
  const float dropout = (float)std::atof(a.s("-p", "--dropout", "0").c_str());
  a.finish("sdpa");
  if (causal && withMask)
    die("sdpa: --causal excludes --mask");
  if (dropout < 0.f || dropout > 1.f)
    die("sdpa: --dropout must be within [0, 1]");
  const Handle &h = lh.get();
  Graph g;
  g.setName("benchmark_sdpa_b" + std::to_string(B) + "hq" + std::to_string(Hq) +
            "hkv" + std::to_string(Hkv) + "sq" + std::to_string(Sq) + "skv" +
            std::to_string(Skv) + "d" + std::to_string(D) + "_type" + tn +
            (causal ? "_causal" : "") + (withMask ? "_mask" : "") +
            (gqa ? "_gqa" : "") + (hasScale ? "_scale" : "") +
            (dropout > 0.f ? "_dropout" : ""))
      .setIODataType(dt)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  auto Q = g.tensor(mk("q", {B, Hq, Sq, D}, contig({B, Hq, Sq, D}), dt));
  auto K = g.tensor(mk("k", {B, Hkv, Skv, D}, contig({B, Hkv, Skv, D}), dt));
  auto V = g.tensor(mk("v", {B, Hkv, Skv, D}, contig({B, Hkv, Skv, D}), dt));
  // mask [batch, 1, seq_q, seq_kv], broadcast over the heads (reference
  // driver.cpp:668-679)
  TensorPtr Mk;
  if (withMask)
    Mk = g.tensor(mk("mask", {B, 1, Sq, Skv}, contig({B, 1, Sq, Skv}), dt));
  SdpaAttr sa;
  sa.setIsCausal(causal).setEnableGqa(gqa).setDropout(dropout);
  if (hasScale)
    sa.setScale(scaleBy);
  auto O = g.sdpa(Q, K, V, Mk, sa);
  O->setOutput(true).setDataType(dt);
  OK(g.validate());
  Pack pack = {{Q, constant(h, Q, 0.01f)}, {K, constant(h, K, 0.01f)},
               {V, constant(h, V, 0.01f)}, {O, constant(h, O, 0.f)}};
  if (Mk)
    pack[Mk] = constant(h, Mk, -1.f);
  Run r{"sdpa", 4.0 * B * Hq * Sq * Skv * D * (causal ? 0.5 : 1.0)};
  timeGraph(h, g, pack, r, iter);
}

void runNorm(LazyHandle &lh, const Args &a, int iter, bool layer) {
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
  const std::string tn = a.s("-t", "--type", "");
  if (tn.empty())
    die("norm: --type is required");
  const DataType dt = dtypeOf(tn);
  if (dims.size() < 2 || dims.size() > 5)
    die("norm: Input dimensions must have rank between 2 and 5");
  for (int64_t d : dims)
    if (d <= 0)
      die("norm: Invalid input dimensions: they must be positive");
  // -l / --layout: one of the reference's layout names of the input's rank
  // (required for layernorm, driver.cpp:997-1000; default contiguous here for
  // the rmsnorm extension)
  std::string layout = a.s("-l", "--layout", "");
  if (layer && layout.empty())
    die("layernorm: --layout is required");
  if (layout.empty())
    layout = dims.size() == 2 ? "NC" : dims.size() == 3 ? "NCH"
             : dims.size() == 4 ? "NCHW" : "NCDHW";
  if (layout.size() != dims.size())
    die("norm: Input dimensions and layout must have the same rank");
  if (layer) {
    const int64_t forw = a.req("-F", "--forw");
    if (forw != 1)
      die("layernorm: only --forw 1 (forward, training mode) is supported");
  }
  const bool affine = a.flag("--elementwise_affine") || !layer;
  const float epsv = (float)std::atof(a.s("-e", "--eps", "1e-5").c_str());
  const bool fuseMul = a.flag("--mul");
  const float mulBy = (float)std::atof(a.s("--mul", "", "1").c_str());
  a.finish(layer ? "layernorm" : "rmsnorm");
  auto xs = generateStrideFromLayout(dims, layout);
  if (isError(xs))
    die("norm: " + ErrorObject(xs).getMessage());
  const Handle &h = lh.get();
  Graph g;
  g.setName(std::string(layer ? "benchmark_layernorm_" : "benchmark_rmsnorm_") +
            a.s("-X", "--input", "") + "_" + tn + "_" + layout +
            (affine ? "_affine" : "") + (fuseMul ? "_mul" : ""))
      .setIODataType(dt)
      .setIntermediateDataType(DataType::Float).setComputeDataType(DataType::Float);
  auto X = g.tensor(mk("x", dims, *xs, dt));
  Dims sd = dims;
  sd[0] = 1;
  TensorPtr S, Bi;
  if (affine)
    S = g.tensor(mk("scale", sd, *generateStrideFromLayout(sd, layout), dt));
  auto eps = g.tensor(TensorAttr(epsv));
  Pack pack;
  TensorPtr Y, Mean, Rstd;
  if (layer) {
    if (affine)
      Bi = g.tensor(mk("bias", sd, *generateStrideFromLayout(sd, layout), dt));
    LayernormAttr la;
    la.setEpsilon(eps).setForwardPhase(NormFwdPhase::TRAINING);
    auto outs = g.layernorm(X, S, Bi, la);
    Y = outs[0];
    Mean = outs[1];
    Rstd = outs[2];
    Mean->setOutput(true).setDataType(dt);
    Rstd->setOutput(true).setDataType(dt);
  } else {
    RmsnormAttr ra;
    ra.setEpsilon(eps).setForwardPhase(NormFwdPhase::INFERENCE);
    auto outs = g.rmsnorm(X, S, ra);
    Y = outs[0];
  }
  if (fuseMul) { // y * scalar fused behind the norm
    PointwiseAttr mul;
    mul.setMode(PointwiseAttr::Mode::MUL);
    Y = g.pointwise(Y, g.tensor(TensorAttr(mulBy)), mul);
  }
  Y->setOutput(true).setDataType(dt);
  OK(g.validate());
  pack[X] = constant(h, X, 1.f);
  if (Mean) {
    pack[Mean] = constant(h, Mean, 0.f);
    pack[Rstd] = constant(h, Rstd, 0.f);
  }
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
    else if (k == "--warmup" && i + 1 < argc)
      g_warmup = std::atoi(argv[++i]);
    else if (k == "--dump" || k == "-d")
      ; // nothing to dump: there is no intermediate IR
    else
      break;
  }
  if (i >= argc)
    die("usage: driver [--device N] [--iter N] [--warmup N] <conv|matmul|sdpa|layernorm|rmsnorm> flags...");
  const std::string cmd = argv[i];
  const Args a = parse(argc, argv, i + 1);
  LazyHandle h;
  h.device = device;
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
