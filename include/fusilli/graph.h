// Graph: the user-facing builder and executor.
//
// Same surface as the reference's graph/graph.h:75-401 (builders, validate,
// compile, compileToArtifact, loadFromArtifact, getWorkspaceSize, execute) and
// the same state machine and error behaviour (NotValidated / NotCompiled /
// VariantPackError / InvalidArgument cases of backend/runtime.h:383-529).
// compile() plans kernels (plan.h) instead of emitting MLIR for iree-compile;
// execute() launches them through the C ABI instead of invoking a VM.
#ifndef FUSILLI_GRAPH_H
#define FUSILLI_GRAPH_H

#include <array>
#include <map>
#include <optional>
#include <set>
#include <span>
#include <unordered_map>
#include <unordered_set>

#include "cache.h"
#include "plan.h"

namespace fusilli {

class Graph : public INode {
public:
  Graph() : INode(Context{}) {}
  Graph(const Graph &) = delete;
  Graph &operator=(const Graph &) = delete;
  Graph(Graph &&) noexcept = default;
  Graph &operator=(Graph &&) noexcept = default;
  ~Graph() = default;

  const std::string &getName() const override final {
    return context.getName();
  }
  Type getType() const override final { return Type::Composite; }

  Graph &setName(const std::string &name) {
    context.setName(name);
    return *this;
  }
  Graph &setIODataType(DataType t) {
    context.setIODataType(t);
    return *this;
  }
  Graph &setComputeDataType(DataType t) {
    context.setComputeDataType(t);
    return *this;
  }
  Graph &setIntermediateDataType(DataType t) {
    context.setIntermediateDataType(t);
    return *this;
  }

  // ---- validation -----------------------------------------------------------
  ErrorObject validate() {
    FUSILLI_LOG_LABEL_ENDL("INFO: Validating Graph");
    FUSILLI_RETURN_ERROR_IF(getName().empty(), ErrorCode::AttributeNotSet,
                            "Graph name not set");
    FUSILLI_CHECK_ERROR(validateSubtree());
    for (const auto &in : fullGraphInputs_)
      FUSILLI_CHECK_ERROR(in->validate());
    for (const auto &out : fullGraphOutputs_) {
      FUSILLI_CHECK_ERROR(out->validate());
      FUSILLI_RETURN_ERROR_IF(
          out->hasBroadcastDims(), ErrorCode::InvalidAttribute,
          "Tensor '" + out->getName() +
              "' has broadcast strides (stride=0) on an operation output, "
              "which is not yet supported");
    }
    isValidated_ = true;
    return ok();
  }

  // ---- compilation ------------------------------------------------------------
  // JIT: plan for the handle's backend, through the on-disk cache, and load
  // the plan.  `remove` = true deletes the cache files when this Graph goes
  // out of scope (reference graph.h:127-146).
  ErrorObject compile(const Handle &handle, bool remove = false) {
    FUSILLI_ASSIGN_OR_RETURN(auto bytes,
                             compileToArtifact(handle.getBackend(), remove));
    return loadFromArtifact(handle, bytes);
  }

  // AOT: the serialised plan, read back from the cache file that holds it.
  // Needs no handle; does not disturb a loaded plan.
  ErrorOr<std::vector<uint8_t>> compileToArtifact(Backend backend,
                                                  bool remove = false) {
    FUSILLI_ASSIGN_OR_RETURN(std::string text, emitAsm());
    FUSILLI_ASSIGN_OR_RETURN(std::filesystem::path artifact,
                             getCompiledArtifact(backend, text, remove));
    (void)artifact;
    return cache_->output.readBytes();
  }

  // A textual description of the validated graph (tensors, nodes, planned
  // steps): what the cache compares to decide whether its artifact is still
  // this graph's.  Takes the place of the reference's MLIR text
  // (graph.h:407-419); backend-independent.
  ErrorOr<std::string> emitAsm() {
    FUSILLI_RETURN_ERROR_IF(!isValidated_, ErrorCode::NotValidated,
                            "Graph must be validated before being compiled");
    plan::Planner planner(subNodes_, fullGraphInputsSorted_,
                          fullGraphOutputsSorted_, Backend::CPU);
    FUSILLI_ASSIGN_OR_RETURN(plan::Plan p, planner.run());
    std::ostringstream os;
    os << "fusilli.graph @" << getName() << " {\n";
    auto tensorLine = [&](const char *what, const TensorAttr &t) {
      os << "  " << what << " %" << t.getName() << " : dims[";
      for (size_t i = 0; i < t.getDim().size(); ++i)
        os << (i ? "," : "") << t.getDim()[i];
      os << "] strides[";
      for (size_t i = 0; i < t.getStride().size(); ++i)
        os << (i ? "," : "") << t.getStride()[i];
      os << "] dtype " << static_cast<int>(t.getDataType()) << "\n";
    };
    for (const auto &t : fullGraphInputsSorted_)
      tensorLine("input", *t);
    for (const auto &t : fullGraphOutputsSorted_)
      tensorLine("output", *t);
    for (const auto &n : subNodes_)
      os << "  node " << static_cast<int>(n->getType()) << " '" << n->getName()
         << "'\n";
    os << "  steps " << p.steps.size() << " workspace " << p.workspaceBytes
       << " plan 0x" << std::hex << p.signature << std::dec << "\n";
    for (const plan::Step &st : p.steps) {
      os << "    step kind " << st.kind << " slots";
      for (int sl : st.slot)
        os << ' ' << sl;
      os << "\n";
    }
    os << "}\n";
    return ok(os.str());
  }

  // The path of the artifact in the cache, (re)generating the cache files
  // unless they are still valid for this instance: same paths (graph name),
  // same description, same planner key (backend).  `reCompiled` reports
  // whether they were regenerated (reference graph.h:428-447, 557-644; the
  // cache is per Graph instance: a new instance always regenerates).
  ErrorOr<std::filesystem::path>
  getCompiledArtifact(Backend backend, const std::string &generatedAsm,
                      bool remove, std::optional<bool> *reCompiled = nullptr) {
    FUSILLI_ASSIGN_OR_RETURN(bool valid, validateCache(backend, generatedAsm));
    if (valid) {
      if (reCompiled)
        *reCompiled = false;
      return ok(cache_->output.path);
    }
    FUSILLI_RETURN_ERROR_IF(!isValidated_, ErrorCode::NotValidated,
                            "Graph must be validated before being compiled");
    plan::Planner planner(subNodes_, fullGraphInputsSorted_,
                          fullGraphOutputsSorted_, backend);
    FUSILLI_ASSIGN_OR_RETURN(plan::Plan p, planner.run());
    const std::vector<uint8_t> bytes = plan::serialize(p);
    cache_.reset(); // the old files (if owned) go first: same names
    FUSILLI_ASSIGN_OR_RETURN(
        CacheFile input, CacheFile::create(getName(), kCacheInputFileName, remove));
    FUSILLI_ASSIGN_OR_RETURN(
        CacheFile output,
        CacheFile::create(getName(), kCacheOutputFileName, remove));
    FUSILLI_ASSIGN_OR_RETURN(
        CacheFile command,
        CacheFile::create(getName(), kCacheCommandFileName, remove));
    FUSILLI_ASSIGN_OR_RETURN(
        CacheFile statistics,
        CacheFile::create(getName(), kCacheStatisticsFileName, remove));
    FUSILLI_CHECK_ERROR(input.write(generatedAsm));
    FUSILLI_CHECK_ERROR(output.write(bytes));
    FUSILLI_CHECK_ERROR(command.write(plannerKey(backend)));
    FUSILLI_CHECK_ERROR(statistics.write(planStatistics(p)));
    cache_.emplace(CachedAssets{std::move(input), std::move(output),
                                std::move(command), std::move(statistics)});
    if (reCompiled)
      *reCompiled = true;
    return ok(cache_->output.path);
  }

  // Contents of one of this instance's cache files.
  ErrorOr<std::string> readCompilationCacheFile(CachedAssetsType type) {
    FUSILLI_RETURN_ERROR_IF(!cache_.has_value(), ErrorCode::FileSystemFailure,
                            "Cache not populated yet");
    switch (type) {
    case CachedAssetsType::Input:
      return cache_->input.read();
    case CachedAssetsType::Output:
      return cache_->output.read();
    case CachedAssetsType::Command:
      return cache_->command.read();
    case CachedAssetsType::Statistics:
      return cache_->statistics.read();
    }
    return error(ErrorCode::InvalidAttribute, "Unknown CachedAssetsType");
  }

  // What the statistics file holds: the plan's dispatch count (one per fused
  // step; the figure the reference reads out of iree-compile's statistics
  // JSON, graph/graph.h:449-468 and benchmarks/driver.cpp) and its workspace.
  static std::string planStatistics(const plan::Plan &p) {
    std::ostringstream os;
    os << "{\n  \"dispatch-count\": " << p.steps.size()
       << ",\n  \"workspace-bytes\": " << p.workspaceBytes
       << ",\n  \"plan-signature\": \"0x" << std::hex << p.signature << std::dec
       << "\"\n}\n";
    return os.str();
  }

  // Loads a plan produced by this or an identically built graph.  Replaces
  // any previously loaded plan; on failure the graph is left not loaded.
  ErrorObject loadFromArtifact(const Handle &handle,
                               std::span<const uint8_t> bytes) {
    FUSILLI_RETURN_ERROR_IF(
        !isValidated_, ErrorCode::NotValidated,
        "Graph must be validated before loading a compiled artifact");
    clearRuntimeState();
    auto parsed = plan::deserialize(bytes);
    if (isError(parsed))
      return ErrorObject(parsed);
    FUSILLI_RETURN_ERROR_IF(
        parsed->backend != static_cast<uint32_t>(handle.getBackend()),
        ErrorCode::RuntimeFailure,
        std::string("Artifact was compiled for backend ") +
            backendName(static_cast<Backend>(parsed->backend)) +
            " but the handle is for backend " +
            backendName(handle.getBackend()));
    // The artifact must describe this graph: re-plan and compare signatures.
    plan::Planner planner(subNodes_, fullGraphInputsSorted_,
                          fullGraphOutputsSorted_, handle.getBackend());
    auto own = planner.run();
    if (isError(own))
      return ErrorObject(own);
    FUSILLI_RETURN_ERROR_IF(own->signature != parsed->signature,
                            ErrorCode::RuntimeFailure,
                            "Artifact does not match this graph (signature "
                            "mismatch)");
    // Only the plan this library derives from the graph is ever executed: the
    // artifact has to be that plan byte for byte (steps, slots, workspace
    // layout, argument table), so a stale or edited file with a valid
    // checksum is rejected rather than run.
    const std::vector<uint8_t> expect = plan::serialize(*own);
    FUSILLI_RETURN_ERROR_IF(
        expect.size() != bytes.size() ||
            std::memcmp(expect.data(), bytes.data(), bytes.size()) != 0,
        ErrorCode::RuntimeFailure,
        "Artifact does not match the plan of this graph (stale or edited "
        "artifact)");
    loadedPlan_ = std::move(*own);
    loadedBackend_ = handle.getBackend();
    return ok();
  }

  // What produced an artifact: changes with the backend and the plan format.
  static std::string plannerKey(Backend backend) {
    return std::string("fusilli_hip plan --backend=") + backendName(backend) +
           " --format=" + std::string(plan::kMagic, sizeof(plan::kMagic)) + "\n";
  }

  // The cache is valid when this instance generated it, the graph's name (the
  // paths) has not changed since, the files still exist, and the description
  // and the planner key they hold are the ones asked for.
  ErrorOr<bool> validateCache(Backend backend, const std::string &generatedAsm) {
    if (!cache_.has_value())
      return ok(false);
    if (cache_->input.path != CacheFile::getPath(getName(), kCacheInputFileName) ||
        cache_->output.path != CacheFile::getPath(getName(), kCacheOutputFileName) ||
        cache_->command.path != CacheFile::getPath(getName(), kCacheCommandFileName) ||
        cache_->statistics.path !=
            CacheFile::getPath(getName(), kCacheStatisticsFileName))
      return ok(false);
    FUSILLI_ASSIGN_OR_RETURN(CacheFile input,
                             CacheFile::open(getName(), kCacheInputFileName));
    FUSILLI_ASSIGN_OR_RETURN(CacheFile output,
                             CacheFile::open(getName(), kCacheOutputFileName));
    FUSILLI_ASSIGN_OR_RETURN(CacheFile command,
                             CacheFile::open(getName(), kCacheCommandFileName));
    FUSILLI_ASSIGN_OR_RETURN(CacheFile statistics,
                             CacheFile::open(getName(), kCacheStatisticsFileName));
    (void)output;
    (void)statistics;
    FUSILLI_ASSIGN_OR_RETURN(std::string inputContents, input.read());
    if (inputContents != generatedAsm)
      return ok(false);
    FUSILLI_ASSIGN_OR_RETURN(std::string commandContents, command.read());
    return ok(commandContents == plannerKey(backend));
  }

  // nullopt until a plan is loaded; must be called before execute().
  ErrorOr<std::optional<size_t>> getWorkspaceSize() {
    if (!loadedPlan_.has_value())
      return ok(std::optional<size_t>());
    const size_t need = static_cast<size_t>(loadedPlan_->workspaceBytes);
    if (!workspaceSize_.has_value() || need > *workspaceSize_)
      workspaceSize_ = need;
    return ok(workspaceSize_);
  }
  [[deprecated("Use Graph::getWorkspaceSize() instead.")]]
  ErrorOr<std::optional<size_t>> getWorkspaceSizeOrError() {
    return getWorkspaceSize();
  }

  // ---- execution ----------------------------------------------------------------
  // Results are written in place into the caller's output buffers; on AMDGPU
  // the call returns once the kernels are queued on the handle's stream.
  ErrorObject
  execute(const Handle &handle,
          const std::unordered_map<std::shared_ptr<TensorAttr>,
                                   std::shared_ptr<Buffer>> &variantPack,
          const std::shared_ptr<Buffer> &workspace) const {
    FUSILLI_LOG_LABEL_ENDL("INFO: Executing Graph");
    FUSILLI_RETURN_ERROR_IF(!loadedPlan_.has_value(), ErrorCode::NotCompiled,
                            "Graph::execute requires a successful compile() "
                            "first (no plan loaded)");
    FUSILLI_RETURN_ERROR_IF(!loadedBackend_.has_value(), ErrorCode::NotCompiled,
                            "Graph::execute requires a successful compile() "
                            "first (loaded backend not set)");
    FUSILLI_RETURN_ERROR_IF(
        handle.getBackend() != *loadedBackend_, ErrorCode::InvalidArgument,
        std::string("Graph::execute got a handle for backend ") +
            backendName(handle.getBackend()) +
            ", but the loaded artifact uses backend " +
            backendName(*loadedBackend_));
    FUSILLI_RETURN_ERROR_IF(
        !workspaceSize_.has_value(), ErrorCode::InvalidArgument,
        "Graph::execute requires getWorkspaceSize() to be called before "
        "workspace allocation and execution");

    // Tensors with dynamic dims take their extents from the buffers: a plan
    // specialised to those extents replaces the loaded one.
    FUSILLI_ASSIGN_OR_RETURN(const plan::Plan *planPtr,
                             planForBuffers(handle, variantPack));
    const plan::Plan &activePlan = *planPtr;
    std::vector<void *> args;
    args.reserve(activePlan.args.size());
    auto push = [&](const std::shared_ptr<TensorAttr> &t) -> ErrorObject {
      const std::shared_ptr<Buffer> &buf = variantPack.at(t);
      FUSILLI_RETURN_ERROR_IF(!buf || buf->data() == nullptr,
                              ErrorCode::VariantPackError,
                              "Tensor '" + t->getName() +
                                  "' has a null buffer in variantPack");
      const plan::ArgInfo &info = activePlan.args[args.size()];
      FUSILLI_RETURN_ERROR_IF(
          buf->sizeInBytes() < info.minBytes, ErrorCode::VariantPackError,
          "Buffer for tensor '" + t->getName() + "' holds " +
              std::to_string(buf->sizeInBytes()) + " bytes but the tensor "
              "needs " + std::to_string(info.minBytes));
      // A typed buffer must at least agree on the element width (raw byte
      // carriers for fp8 and workspaces are untyped or one byte wide).
      FUSILLI_RETURN_ERROR_IF(
          buf->isTyped() &&
              dataTypeSize(buf->getDataType()) !=
                  dataTypeSize(static_cast<DataType>(info.dtype)),
          ErrorCode::VariantPackError,
          "Buffer for tensor '" + t->getName() + "' has element type " +
              dataTypeAsm(buf->getDataType()) + " but the tensor is " +
              dataTypeAsm(static_cast<DataType>(info.dtype)));
      args.push_back(buf->data());
      return ok();
    };
    for (const auto &out : fullGraphOutputsSorted_) {
      if (out->isVirtual()) {
        FUSILLI_RETURN_ERROR_IF(variantPack.contains(out),
                                ErrorCode::VariantPackError,
                                "Virtual output tensor found in variantPack");
        continue;
      }
      FUSILLI_RETURN_ERROR_IF(!variantPack.contains(out),
                              ErrorCode::VariantPackError,
                              "Output tensor missing from variantPack");
      FUSILLI_CHECK_ERROR(push(out));
    }
    for (const auto &in : fullGraphInputsSorted_) {
      if (in->isScalar()) {
        FUSILLI_RETURN_ERROR_IF(variantPack.contains(in),
                                ErrorCode::VariantPackError,
                                "Scalar constant tensor found in variantPack");
        continue;
      }
      FUSILLI_RETURN_ERROR_IF(!variantPack.contains(in),
                              ErrorCode::VariantPackError,
                              "Input tensor missing from variantPack");
      FUSILLI_CHECK_ERROR(push(in));
    }

    void *workspacePtr = nullptr;
    if (*workspaceSize_ > 0) {
      FUSILLI_RETURN_ERROR_IF(
          workspace == nullptr, ErrorCode::InvalidArgument,
          "Workspace buffer required but not provided (size=" +
              std::to_string(*workspaceSize_) + " bytes)");
      FUSILLI_RETURN_ERROR_IF(
          workspace->sizeInBytes() < *workspaceSize_,
          ErrorCode::InvalidArgument,
          "Workspace buffer too small: provided " +
              std::to_string(workspace->sizeInBytes()) + " bytes, required " +
              std::to_string(*workspaceSize_) + " bytes");
      workspacePtr = workspace->data();
    } else if (workspace != nullptr) {
      FUSILLI_LOG_LABEL_ENDL("WARNING: Workspace buffer provided but not "
                             "needed (size=0), ignoring");
    }

    FUSILLI_RETURN_ERROR_IF(
        handle.getBackend() != Backend::AMDGPU, ErrorCode::NotImplemented,
        "Backend::CPU has no execution engine in this build: graphs run on "
        "Backend::AMDGPU (gfx950) only");
    for (const auto &kv : variantPack)
      FUSILLI_RETURN_ERROR_IF(kv.second && !kv.second->isDeviceMemory(),
                              ErrorCode::VariantPackError,
                              "Tensor '" + kv.first->getName() +
                                  "' is backed by host memory; AMDGPU "
                                  "execution needs device buffers");
    FUSILLI_RETURN_ERROR_IF(
        activePlan.workspaceBytes > *workspaceSize_, ErrorCode::InvalidArgument,
        "The buffers' extents need " +
            std::to_string(activePlan.workspaceBytes) +
            " bytes of workspace, more than getWorkspaceSize() reported (" +
            std::to_string(*workspaceSize_) + ")");
    return plan::execute(handle.getContext(), activePlan, args, workspacePtr);
  }

  // ---- builders ---------------------------------------------------------------
  std::shared_ptr<TensorAttr> tensor(const TensorAttr &t) {
    FUSILLI_LOG_LABEL_ENDL("INFO: Adding input tensor '" << t.getName()
                                                         << "' to Graph inputs");
    auto p = std::make_shared<TensorAttr>(t);
    fullGraphInputs_.insert(p);
    return p;
  }

  std::shared_ptr<TensorAttr> convFProp(const TensorPtr &x, const TensorPtr &w,
                                        ConvFPropAttr &attr) {
    nameNode(attr, "conv_fprop");
    nameTensor(x, attr, "X");
    nameTensor(w, attr, "W");
    attr.setX(x).setW(w);
    auto y = outputTensor(attr.getName() + "_Y");
    attr.setY(y);
    subNodes_.emplace_back(
        std::make_shared<ConvFPropNode>(std::move(attr), context));
    return y;
  }

  // graph.h:795-824 of the reference: DW's dims are set by the caller on the
  // returned tensor (the filter's channel extent fixes the group count).
  std::shared_ptr<TensorAttr> convWGrad(const TensorPtr &dy, const TensorPtr &x,
                                        ConvWGradAttr &attr) {
    nameNode(attr, "conv_wgrad");
    nameTensor(dy, attr, "DY");
    nameTensor(x, attr, "X");
    attr.setDY(dy).setX(x);
    auto dw = outputTensor(attr.getName() + "_DW");
    attr.setDW(dw);
    subNodes_.emplace_back(
        std::make_shared<ConvWGradNode>(std::move(attr), context));
    return dw;
  }

  // graph.h:826-855 of the reference: DX's dims are set by the caller.
  std::shared_ptr<TensorAttr> convDGrad(const TensorPtr &dy, const TensorPtr &w,
                                        ConvDGradAttr &attr) {
    nameNode(attr, "conv_dgrad");
    nameTensor(dy, attr, "DY");
    nameTensor(w, attr, "W");
    attr.setDY(dy).setW(w);
    auto dx = outputTensor(attr.getName() + "_DX");
    attr.setDX(dx);
    subNodes_.emplace_back(
        std::make_shared<ConvDGradNode>(std::move(attr), context));
    return dx;
  }

  std::shared_ptr<TensorAttr> matmul(const TensorPtr &a, const TensorPtr &b,
                                     MatmulAttr &attr) {
    nameNode(attr, "matmul");
    nameTensor(a, attr, "A");
    nameTensor(b, attr, "B");
    attr.setA(a).setB(b);
    auto c = outputTensor(attr.getName() + "_C");
    attr.setC(c);
    subNodes_.emplace_back(
        std::make_shared<MatmulNode>(std::move(attr), context));
    return c;
  }

  std::shared_ptr<TensorAttr> pointwise(const TensorPtr &in,
                                        PointwiseAttr &attr) {
    return pointwiseImpl({in}, attr);
  }
  std::shared_ptr<TensorAttr> pointwise(const TensorPtr &in0,
                                        const TensorPtr &in1,
                                        PointwiseAttr &attr) {
    return pointwiseImpl({in0, in1}, attr);
  }
  std::shared_ptr<TensorAttr> pointwise(const TensorPtr &in0,
                                        const TensorPtr &in1,
                                        const TensorPtr &in2,
                                        PointwiseAttr &attr) {
    return pointwiseImpl({in0, in1, in2}, attr);
  }

  std::shared_ptr<TensorAttr> reduction(const TensorPtr &x,
                                        ReductionAttr &attr) {
    nameNode(attr, "reduction");
    nameTensor(x, attr, "X");
    attr.setX(x);
    auto y = outputTensor(attr.getName() + "_Y");
    attr.setY(y);
    subNodes_.emplace_back(
        std::make_shared<ReductionNode>(std::move(attr), context));
    return y;
  }

  std::shared_ptr<TensorAttr> sdpa(const TensorPtr &q, const TensorPtr &k,
                                   const TensorPtr &v, const TensorPtr &mask,
                                   SdpaAttr &attr) {
    nameNode(attr, "sdpa");
    nameTensor(q, attr, "Q");
    nameTensor(k, attr, "K");
    nameTensor(v, attr, "V");
    nameTensor(mask, attr, "MASK");
    attr.setQ(q).setK(k).setV(v);
    if (mask)
      attr.setMASK(mask);
    auto o = outputTensor(attr.getName() + "_O");
    attr.setO(o);
    subNodes_.emplace_back(std::make_shared<SdpaNode>(std::move(attr), context));
    return o;
  }

  // Returns {Y, INV_RMS}; INV_RMS is null outside the training phase.
  std::array<std::shared_ptr<TensorAttr>, 2>
  rmsnorm(const TensorPtr &x, const TensorPtr &scale, RmsnormAttr &attr) {
    nameNode(attr, "rmsnorm");
    nameTensor(x, attr, "X");
    nameTensor(scale, attr, "SCALE");
    nameTensor(attr.getEpsilon(), attr, "EPSILON");
    attr.setX(x);
    attr.setSCALE(scale);
    auto y = outputTensor(attr.getName() + "_Y");
    attr.setY(y);
    std::shared_ptr<TensorAttr> r;
    if (attr.getForwardPhase() == NormFwdPhase::TRAINING)
      r = outputTensor(attr.getName() + "_INV_RMS");
    attr.setINV_RMS(r);
    subNodes_.emplace_back(
        std::make_shared<RmsNormNode>(std::move(attr), context));
    return {y, r};
  }

  // Returns {Y, MEAN, INV_VARIANCE}; the statistics are null outside training.
  std::array<std::shared_ptr<TensorAttr>, 3>
  layernorm(const TensorPtr &x, const TensorPtr &scale, const TensorPtr &bias,
            LayernormAttr &attr) {
    nameNode(attr, "layernorm");
    nameTensor(x, attr, "X");
    nameTensor(scale, attr, "SCALE");
    nameTensor(bias, attr, "BIAS");
    nameTensor(attr.getEpsilon(), attr, "EPSILON");
    attr.setX(x);
    attr.setSCALE(scale);
    attr.setBIAS(bias);
    auto y = outputTensor(attr.getName() + "_Y");
    std::shared_ptr<TensorAttr> m, v;
    if (attr.getForwardPhase() == NormFwdPhase::TRAINING) {
      m = outputTensor(attr.getName() + "_MEAN");
      v = outputTensor(attr.getName() + "_INV_VARIANCE");
    }
    attr.setY(y);
    attr.setMEAN(m);
    attr.setINV_VARIANCE(v);
    subNodes_.emplace_back(
        std::make_shared<LayerNormNode>(std::move(attr), context));
    return {y, m, v};
  }

  // graph.h:860-913 of the reference.  SAVED_MEAN and SAVED_INV_VARIANCE are
  // null outside the training phase.
  std::array<std::shared_ptr<TensorAttr>, 3>
  batchnorm(const TensorPtr &x, const TensorPtr &scale, const TensorPtr &bias,
            const TensorPtr &mean, const TensorPtr &var, BatchnormAttr &attr) {
    nameNode(attr, "batchnorm");
    nameTensor(x, attr, "X");
    nameTensor(scale, attr, "SCALE");
    nameTensor(bias, attr, "BIAS");
    nameTensor(mean, attr, "MEAN");
    nameTensor(var, attr, "VAR");
    nameTensor(attr.getEpsilon(), attr, "EPSILON");
    nameTensor(attr.getMomentum(), attr, "MOMENTUM");
    attr.setX(x);
    attr.setSCALE(scale);
    attr.setBIAS(bias);
    attr.setMEAN(mean);
    attr.setVAR(var);
    auto y = outputTensor(attr.getName() + "_Y");
    std::shared_ptr<TensorAttr> m, v;
    if (attr.getForwardPhase() == NormFwdPhase::TRAINING) {
      m = outputTensor(attr.getName() + "_SAVED_MEAN");
      v = outputTensor(attr.getName() + "_SAVED_INV_VARIANCE");
    }
    attr.setY(y);
    attr.setSAVED_MEAN(m);
    attr.setSAVED_INV_VARIANCE(v);
    subNodes_.emplace_back(
        std::make_shared<BatchNormNode>(std::move(attr), context));
    return {y, m, v};
  }

  // Number of kernel launches the loaded plan performs (the analogue of the
  // dispatch count the reference reads from IREE's compile statistics).
  std::optional<size_t> getKernelCount() const {
    if (!loadedPlan_)
      return std::nullopt;
    return loadedPlan_->steps.size();
  }

private:
  template <typename Attr> void nameNode(Attr &attr, const char *prefix) {
    if (attr.getName().empty())
      attr.setName(std::string(prefix) + "_" + std::to_string(subNodes_.size()));
  }
  template <typename Attr>
  static void nameTensor(const TensorPtr &t, const Attr &attr,
                         const char *suffix) {
    if (t && t->getName().empty())
      t->setName(attr.getName() + "_" + suffix);
  }

  std::shared_ptr<TensorAttr>
  pointwiseImpl(std::initializer_list<TensorPtr> ins, PointwiseAttr &attr) {
    nameNode(attr, "pointwise");
    int i = 0;
    for (const TensorPtr &t : ins) {
      nameTensor(t, attr, ("IN_" + std::to_string(i)).c_str());
      attr.setInput(static_cast<PointwiseAttr::InputNames>(i), t);
      ++i;
    }
    auto out = outputTensor(attr.getName() + "_OUT_0");
    attr.setOUT_0(out);
    subNodes_.emplace_back(
        std::make_shared<PointwiseNode>(std::move(attr), context));
    return out;
  }

  // Node outputs start virtual; setOutput(true) makes them graph outputs.
  std::shared_ptr<TensorAttr> outputTensor(const std::string &name) {
    auto t = std::make_shared<TensorAttr>();
    t->setName(name).setIsVirtual(true);
    fullGraphOutputs_.insert(t);
    return t;
  }

  // Input, output and node names share one namespace (graph/graph.h:655-677).
  ErrorObject preValidateNode() const override final {
    std::unordered_set<std::string> used;
    for (const auto *set : {&fullGraphInputs_, &fullGraphOutputs_})
      for (const auto &t : *set) {
        FUSILLI_RETURN_ERROR_IF(used.contains(t->getName()),
                                ErrorCode::InvalidAttribute,
                                "Symbol name '" + t->getName() +
                                    "' already in use");
        used.insert(t->getName());
      }
    FUSILLI_CHECK_ERROR(checkNodeNamesAreUnique(used));
    return ok();
  }

  ErrorObject inferPropertiesNode() override final {
    fullGraphInputsSorted_.insert(fullGraphInputs_.begin(),
                                  fullGraphInputs_.end());
    fullGraphOutputsSorted_.insert(fullGraphOutputs_.begin(),
                                   fullGraphOutputs_.end());
    return ok();
  }

  void clearRuntimeState() {
    loadedPlan_.reset();
    loadedBackend_.reset();
    workspaceSize_.reset();
    dynamicPlans_.clear();
  }

  // ---- dynamic dims (reference samples/dynamic_shapes/*.cpp) --------------------
  // A tensor marked with setDynamicDims() is declared at the extents compile()
  // plans for; execute() may be given buffers whose shape differs in those
  // dims.  The plan for a new set of extents is built on first use and kept.
  // Every tensor whose extents change must be in the variant pack (a virtual
  // tensor's extents cannot be read from a buffer).

  // Puts back the dims, strides and dynamic-dim marks it replaced.
  class ShapeOverride {
  public:
    ShapeOverride() = default;
    ShapeOverride(const ShapeOverride &) = delete;
    ShapeOverride &operator=(const ShapeOverride &) = delete;
    void set(const std::shared_ptr<TensorAttr> &t, std::vector<int64_t> dims) {
      saved_.push_back({t, t->getDim(), t->getStride()});
      // dense strides in the tensor's own dim order; broadcast dims stay 0
      const auto perm = t->getLogicalToPhysicalPermuteOrder();
      const std::vector<int64_t> oldDim = t->getDim(), oldStride = t->getStride();
      std::vector<int64_t> stride(dims.size(), 1);
      int64_t run = 1;
      for (size_t i = dims.size(); i-- > 0;) {
        const size_t src = static_cast<size_t>(perm[i]);
        if (oldDim[src] > 1 && oldStride[src] == 0) {
          stride[src] = 0;
        } else {
          stride[src] = run;
          run *= dims[src];
        }
      }
      t->setDim(dims).setStride(stride);
    }
    ~ShapeOverride() {
      for (auto it = saved_.rbegin(); it != saved_.rend(); ++it)
        it->t->setDim(it->dim).setStride(it->stride);
    }

  private:
    struct Saved {
      std::shared_ptr<TensorAttr> t;
      std::vector<int64_t> dim, stride;
    };
    std::vector<Saved> saved_;
  };

  // The loaded plan, or the plan specialised to the extents of the buffers
  // bound to tensors with dynamic dims.
  ErrorOr<const plan::Plan *> planForBuffers(
      const Handle &handle,
      const std::unordered_map<std::shared_ptr<TensorAttr>,
                               std::shared_ptr<Buffer>> &variantPack) const {
    std::vector<int64_t> key;
    std::vector<std::pair<std::shared_ptr<TensorAttr>, std::vector<int64_t>>>
        changed;
    auto visit = [&](const std::shared_ptr<TensorAttr> &t) -> ErrorObject {
      if (!t->hasDynamicDims())
        return ok();
      auto it = variantPack.find(t);
      if (it == variantPack.end() || !it->second)
        return ok(); // reported by the variant-pack checks
      const std::vector<size_t> &shape = it->second->getShape();
      const std::vector<int64_t> &dim = t->getDim();
      if (shape.size() != dim.size())
        return ok(); // an untyped / imported buffer carries no extents
      const auto perm = t->getLogicalToPhysicalPermuteOrder();
      std::vector<int64_t> now = dim;
      for (size_t i = 0; i < dim.size(); ++i) {
        const size_t src = static_cast<size_t>(perm[i]);
        if (dim[src] > 1 && t->getStride()[src] == 0)
          continue; // broadcast dims occupy one element
        now[src] = static_cast<int64_t>(shape[i]);
      }
      const auto &dyn = t->getDynamicDims();
      for (size_t i = 0; i < dim.size(); ++i)
        FUSILLI_RETURN_ERROR_IF(
            now[i] != dim[i] &&
                std::find(dyn.begin(), dyn.end(), i) == dyn.end(),
            ErrorCode::VariantPackError,
            "Buffer for tensor '" + t->getName() + "' has extent " +
                std::to_string(now[i]) + " in dim " + std::to_string(i) +
                ", which is not a dynamic dim (expected " +
                std::to_string(dim[i]) + ")");
      for (size_t i = 0; i < dim.size(); ++i)
        FUSILLI_RETURN_ERROR_IF(now[i] < 1, ErrorCode::VariantPackError,
                                "Buffer for tensor '" + t->getName() +
                                    "' has an empty dynamic dim");
      key.insert(key.end(), now.begin(), now.end());
      if (now != dim)
        changed.emplace_back(t, std::move(now));
      return ok();
    };
    for (const auto &out : fullGraphOutputsSorted_)
      if (!out->isVirtual())
        FUSILLI_CHECK_ERROR(visit(out));
    for (const auto &in : fullGraphInputsSorted_)
      if (!in->isScalar())
        FUSILLI_CHECK_ERROR(visit(in));
    if (changed.empty())
      return ok(&*loadedPlan_);
    if (auto it = dynamicPlans_.find(key); it != dynamicPlans_.end())
      return ok(&it->second);
    ShapeOverride scope;
    for (auto &[t, dims] : changed)
      scope.set(t, dims);
    plan::Planner planner(subNodes_, fullGraphInputsSorted_,
                          fullGraphOutputsSorted_, handle.getBackend());
    FUSILLI_ASSIGN_OR_RETURN(plan::Plan p, planner.run());
    return ok(&dynamicPlans_.emplace(std::move(key), std::move(p)).first->second);
  }

  bool isValidated_ = false;
  std::optional<plan::Plan> loadedPlan_;
  // this instance's cache files; never shared between instances
  std::optional<CachedAssets> cache_;
  std::optional<Backend> loadedBackend_;
  std::optional<size_t> workspaceSize_;
  // plans for buffer extents that differ from the declared ones
  mutable std::map<std::vector<int64_t>, plan::Plan> dynamicPlans_;

  std::unordered_set<std::shared_ptr<TensorAttr>> fullGraphInputs_;
  std::unordered_set<std::shared_ptr<TensorAttr>> fullGraphOutputs_;
  // Name-sorted views, filled by validate(); they fix the argument order.
  std::set<std::shared_ptr<TensorAttr>, TensorAttrSortByName>
      fullGraphInputsSorted_;
  std::set<std::shared_ptr<TensorAttr>, TensorAttrSortByName>
      fullGraphOutputsSorted_;
};

} // namespace fusilli

#endif // FUSILLI_GRAPH_H
