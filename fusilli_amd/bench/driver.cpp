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

#include <cmath>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
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

bool g_random = false; // --fill random: pseudo-random inputs instead of constants

// Values of a random fill: a 64-bit mix of the element index (splitmix64),
// uniform in [-1, 1) (integers: -127 .. 127).
struct RandomFill {
  uint64_t seed;
  double operator()(size_t i) const {
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (uint64_t)(i + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (double)(z >> 11) * (1.0 / 9007199254740992.0) * 2.0 - 1.0;
  }
};

// device buffer shaped like the tensor's physical dims, filled with the
// constant `v` (the reference driver's fills), or with pseudo-random values
// under --fill random (outputs, v == 0, stay zero)
std::shared_ptr<Buffer> constant(const Handle &h, const TensorPtr &t, float v) {
  std::vector<size_t> shape;
  size_t n = 1;
  for (int64_t d : t->getPhysicalDim()) {
    shape.push_back((size_t)d);
    n *= (size_t)d;
  }
  if (g_random && v != 0.f) {
    static uint64_t tensors = 0;
    const RandomFill rnd{0x5eed0000ull + 977 * ++tensors};
    auto wrapr = [&](auto e) {
      if (isError(e))
        die("allocate " + t->getName() + ": " + ErrorObject(e).getMessage());
      return std::make_shared<Buffer>(std::move(*e));
    };
    auto fill = [&](auto tag, double scale) {
      using T = decltype(tag);
      std::vector<T> data(n);
      for (size_t i = 0; i < n; ++i)
        data[i] = (T)(float)(rnd(i) * scale);
      return wrapr(Buffer::allocate(h, shape, data));
    };
    switch (t->getDataType()) {
    case DataType::Float:
      return fill(float{}, 1.0);
    case DataType::Half:
      return fill(half{}, 1.0);
    case DataType::BFloat16:
      return fill(bf16{}, 1.0);
    case DataType::Int8:
      return fill(int8_t{}, 127.0);
    case DataType::FP8E4M3: {
      std::vector<fp8e4m3> data(n);
      for (size_t i = 0; i < n; ++i) // any finite bit pattern: sign, exponent < 15, mantissa
        data[i] = fp8e4m3{(uint8_t)((uint64_t)((rnd(i) + 1.0) * 63.0) | (rnd(i + n) < 0 ? 0x80 : 0))};
      return wrapr(Buffer::allocate(h, shape, data));
    }
    default:
      break; // other types keep their constant
    }
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

// One output to check after the timed loop (--verify): the tensor, and the
// value every element must have as a function of its logical coordinates.
// With the constant fills of the inputs every answer here is a closed form
// (the reference's samples check the same ones: convolution = taps inside the
// image x channels of a group, matmul = K, attention over constant tensors = V,
// samples/sdpa_utils.cpp:49-102, tests/test_graph.cpp:198-223).
struct Expect {
  TensorPtr tensor;
  std::function<double(const Dims &)> value;
  double rtol = 0; // 0: by the tensor's type (1e-4 f32, 2e-2 16-bit / fp8, 0 integers)
  double atol = 0;
};

struct Run {
  std::string name;
  double work = 0; // FLOP or bytes
  const char *unit = "TFLOP/s";
  std::vector<Expect> expect;
};

int g_warmup = 3; // untimed executes before the --iter loop (--warmup)
bool g_host_time = false; // --host-time: also print the calling thread's time per execute (stderr)
bool g_verify = false; // --verify: compare the outputs with their closed forms

// The buffer's elements as doubles, in storage order.
std::vector<double> readAsDouble(const Handle &h, Buffer &b, DataType dt) {
  std::vector<double> out;
  auto pull = [&](auto tag) {
    using T = decltype(tag);
    std::vector<T> v;
    OK(b.read(h, v));
    out.reserve(v.size());
    for (const T &x : v)
      out.push_back((double)(float)x);
  };
  switch (dt) {
  case DataType::Float:
    pull(float{});
    break;
  case DataType::Half:
    pull(half{});
    break;
  case DataType::BFloat16:
    pull(bf16{});
    break;
  case DataType::Int32:
    pull(int32_t{});
    break;
  case DataType::Int8:
    pull(int8_t{});
    break;
  default:
    die("--verify: no reader for this output type");
  }
  return out;
}

// Compares every element of the expectation's tensor; prints the verdict line
// `verify,<tensor>,<elements>,<mismatches>,<max abs error>` and fails the run
// on a mismatch.
void verifyOutputs(const Handle &h, Pack &pack, const Run &r) {
  for (const Expect &e : r.expect) {
    const TensorPtr &t = e.tensor;
    const DataType dt = t->getDataType();
    const std::vector<double> got = readAsDouble(h, *pack.at(t), dt);
    const Dims &dim = t->getDim(), &st = t->getStride();
    double rtol = e.rtol;
    if (rtol == 0)
      rtol = dt == DataType::Float ? 1e-4 : (dt == DataType::Int32 || dt == DataType::Int8) ? 0 : 2e-2;
    Dims c(dim.size(), 0);
    size_t bad = 0, n = 0;
    double worst = 0;
    for (;;) {
      int64_t off = 0;
      for (size_t i = 0; i < dim.size(); ++i)
        off += c[i] * st[i];
      const double want = e.value(c), have = got.at((size_t)off);
      const double err = std::fabs(have - want);
      if (!(err <= rtol * std::fabs(want) + e.atol)) {
        if (bad < 5) {
          std::string at;
          for (int64_t x : c)
            at += (at.empty() ? "" : ",") + std::to_string(x);
          std::fprintf(stderr, "verify: %s[%s] = %.6g, expected %.6g\n", t->getName().c_str(),
                       at.c_str(), have, want);
        }
        ++bad;
      }
      worst = err > worst ? err : worst;
      ++n;
      int i = (int)dim.size() - 1;
      for (; i >= 0; --i) {
        if (++c[i] < dim[i])
          break;
        c[i] = 0;
      }
      if (i < 0)
        break;
    }
    std::printf("verify,%s,%zu,%zu,%.6g\n", t->getName().c_str(), n, bad, worst);
    if (bad)
      die("--verify: " + std::to_string(bad) + " of " + std::to_string(n) + " elements of " +
          t->getName() + " differ from the closed form");
  }
}

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
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < iter; ++i)
    OK(g.execute(h, pack, wsBuf));
  const auto t1 = std::chrono::steady_clock::now();
  fhip_event_record(ctx, e1);
  fhip_stream_sync(ctx);
  if (g_host_time) // (the enqueue loop alone: what one execute costs the calling thread; the
                   // launch queue takes a few hundred kernels before a launch waits for the GPU)
    std::fprintf(stderr, "host_us_per_execute,%s,%.3f\n", r.name.c_str(),
                 std::chrono::duration<double, std::micro>(t1 - t0).count() / iter);
  float ms = 0;
  fhip_event_elapsed_ms(ctx, e0, e1, &ms);
  fhip_event_destroy(ctx, e0);
  fhip_event_destroy(ctx, e1);
  const double us = ms * 1e3 / iter;
  const size_t kernels = g.getKernelCount().value_or(0);
  std::printf("name,iter,dispatch_count,avg_us,work,%s\n", r.unit);
  std::printf("%s,%d,%zu,%.3f,%.0f,%.3f\n", r.name.c_str(), iter, kernels, us,
              r.work, r.work / us / 1e6);
  if (g_verify)
    verifyOutputs(h, pack, r);
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
    // all-ones DY and W / X: every gradient element counts the (tap, output)
    // pairs that touch it, per spatial dim, times the channels summed over
    const size_t sp = (size_t)sdim;
    if (mode == 2) {
      // DX[n, c, i..] = (K / groups) x prod_dims #{(f, o): i + pad - f dil = o stride, 0 <= o < P}
      r.expect.push_back({OUT, [=](const Dims &at) {
        double v = (double)(k / gcount);
        for (size_t d = 0; d < sp; ++d) {
          int cnt = 0;
          for (int64_t f = 0; f < wd[2 + d]; ++f) {
            const int64_t num = at[2 + d] + cp[d] - f * cd[d];
            if (num >= 0 && num % cs[d] == 0 && num / cs[d] < yd[2 + d])
              ++cnt;
          }
          v *= cnt;
        }
        return v;
      }});
    } else {
      // DW[k, c, f..] = N x prod_dims #{o: 0 <= o stride - pad + f dil < H}
      r.expect.push_back({OUT, [=](const Dims &at) {
        double v = (double)n;
        for (size_t d = 0; d < sp; ++d) {
          int cnt = 0;
          for (int64_t o2 = 0; o2 < yd[2 + d]; ++o2) {
            const int64_t in = o2 * cs[d] - cp[d] + at[2 + d] * cd[d];
            if (in >= 0 && in < xd[2 + d])
              ++cnt;
          }
          v *= cnt;
        }
        return v;
      }});
    }
    if (DB) // the bias gradient sums DY over batch and space
      r.expect.push_back({DB, [=](const Dims &) { return (double)n * opix; }});
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
  {
    // all-ones X, W and bias: Y = (filter taps inside the image) x (channels of
    // a group) (+ 1) (x the scalar); ReLU leaves the positive values alone
    const size_t sp = (size_t)sdim;
    const double add = bias ? 1.0 : 0.0, scale = mul ? (double)mulBy : 1.0;
    r.expect.push_back({Y, [=](const Dims &at) {
      double v = (double)fc;
      for (size_t d = 0; d < sp; ++d) {
        int cnt = 0;
        for (int64_t f = 0; f < wd[2 + d]; ++f) {
          const int64_t in = at[2 + d] * cs[d] - cp[d] + f * cd[d];
          if (in >= 0 && in < xd[2 + d])
            ++cnt;
        }
        v *= cnt;
      }
      return (v + add) * scale;
    }});
  }
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
  {
    // all-ones operands (and bias): C = K (+ 1) (x the scalar)
    const double want = ((double)K + (withBias ? 1.0 : 0.0)) * (outScale ? (double)outScaleBy : 1.0);
    r.expect.push_back({C, [=](const Dims &) { return want; }});
  }
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
  // constant Q, K, V (and mask): every softmax is uniform over its live keys
  // and the output equals V's constant (reference samples/sdpa_utils.cpp:49-102,
  // tolerance 1e-2 there); dropout is not applied by the inference graph
  r.expect.push_back({O, [](const Dims &) { return 0.01; }, 1e-2, 1e-4});
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
  {
    // constant X = 1, scale = 2, bias = 0.5.  LayerNorm: x - mean = 0, so Y is
    // the bias (0 without the affine pair), mean = 1 and 1/sqrt(0 + eps);
    // RMSNorm: Y = scale / sqrt(1 + eps) (x the scalar)
    const double scale = fuseMul ? (double)mulBy : 1.0;
    if (layer) {
      const double yv = (affine ? 0.5 : 0.0) * scale;
      r.expect.push_back({Y, [=](const Dims &) { return yv; }, 0, 1e-3});
      r.expect.push_back({Mean, [](const Dims &) { return 1.0; }});
      const double rs = 1.0 / std::sqrt((double)epsv);
      r.expect.push_back({Rstd, [=](const Dims &) { return rs; }});
    } else {
      const double yv = (affine ? 2.0 : 1.0) / std::sqrt(1.0 + (double)epsv) * scale;
      r.expect.push_back({Y, [=](const Dims &) { return yv; }});
    }
  }
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
    else if (k == "--verify")
      g_verify = true;
    else if (k == "--host-time")
      g_host_time = true;
    else if (k == "--fill" && i + 1 < argc) {
      const std::string f = argv[++i];
      if (f != "random" && f != "constant")
        die("--fill takes `constant` (the default) or `random`");
      g_random = f == "random";
    }
    else if (k == "--dump" || k == "-d")
      ; // nothing to dump: there is no intermediate IR
    else
      break;
  }
  if (i >= argc)
    die("usage: driver [--device N] [--iter N] [--warmup N] [--verify] [--host-time] [--fill constant|random] <conv|matmul|sdpa|layernorm|rmsnorm> flags...");
  if (g_verify && g_random)
    die("--verify checks the closed forms of the constant fills: it excludes --fill random");
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
