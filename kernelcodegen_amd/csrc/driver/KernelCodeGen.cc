// KernelCodeGenerator::optimize / evaluate (declared in include/KernelCodeGen.h;
// reference: src/KernelCodeGen.cc:8-120).
#include "KernelCodeGen.h"

#include <algorithm>
#include <cmath>
#include <sstream>

#include "kcg_hip.h"

namespace KernelCodeGen {

Log KCGLog::level = Log::Release;

namespace {
struct ConfigSlot {
  const char* name;
  KernelCodeGenerator::ConfigList KernelCodeGenerator::*unused;
};
}  // namespace

const KernelCodeGenerator::ConfigList* KernelCodeGenerator::getConfigs(const std::string& n) const {
  if (n == "Matmul") return &matmulConfigs;
  if (n == "BatchMatmul") return &batchMatmulConfigs;
  if (n == "ElementWise") return &elementWiseConfigs;
  if (n == "LayerNorm") return &layerNormConfigs;
  if (n == "FMHA") return &fmhaConfigs;
  if (n == "Binary") return &binaryConfigs;
  if (n == "Gather") return &gatherConfigs;
  if (n == "Softmax") return &softmaxConfigs;
  return nullptr;
}

bool KernelCodeGenerator::setConfigs(const std::string& n, const ConfigList& configs) {
  auto* slot = const_cast<ConfigList*>(getConfigs(n));
  if (!slot) return false;
  *slot = configs;
  return true;
}

// For every optimizer the user pushed: try each of its configurations on a
// fresh copy of the module, keep the best result.  Optimizers are applied
// one after the other, each starting from the best module of the previous one.
// A candidate is better when it schedules more of the graph's operators (a
// configuration that one operator's shape does not fit leaves that operator
// without a kernel, and what it does emit would otherwise measure "faster"),
// and among those that schedule the same number, when it is faster.
mlir::ModuleOp& KernelCodeGenerator::optimize(ComputeDAG& graph_) {
  graph = graph_;
  mlir::ModuleOp module = graph.module.clone();
  saveBestModule(module);
  evaluationLog.clear();

  auto staticConfigOf = [](const std::string& n) -> std::map<std::string, int>* {
    if (n == "Matmul") return &MatmulOptimizer::matmulConfig;
    if (n == "BatchMatmul") return &BatchMatmulOptimizer::batchMatmulConfig;
    if (n == "ElementWise") return &ElementWiseOptimizer::elementWiseConfig;
    if (n == "LayerNorm") return &LayerNormOptimizer::layerNormConfig;
    if (n == "FMHA") return &FMHAOptimizer::fmhaConfig;
    if (n == "Binary") return &BinaryOptimizer::binaryConfig;
    if (n == "Gather") return &GatherOptimizer::gatherConfig;
    if (n == "Softmax") return &SoftmaxOptimizer::softmaxConfig;
    return nullptr;
  };

  for (auto& opt : opts) {
    // each optimizer competes only against its own candidates
    minLatency = FLT_MAX;
    int bestKernels = -1;
    module = bestModule.clone();
    backupModule(module);
    const ConfigList* configs = getConfigs(opt->name);
    std::map<std::string, int>* active = staticConfigOf(opt->name);
    auto tryOnce = [&](int configIndex) {
      Evaluation ev;
      ev.optimizer = opt->name;
      ev.configIndex = configIndex;
      if (active) ev.config = *active;
      if (!opt->applicable(module)) {
        ev.note = "not applicable";
        evaluationLog.push_back(ev);
        return;
      }
      opt->applyOptimzer(module, builder);
      lowerOnly = !(configs && active && configs->size() > 1);
      ev.latencyMs = evaluate(module, &ev.kernels, &ev.note);
      lowerOnly = false;
      // The first applicable candidate is kept whatever its measurement says (a schedule the backend cannot
      // lower still is the scheduled IR, as in the reference, whose evaluate() returns 0 for everything);
      // a later one replaces it when it emits more kernels or the same number of faster ones.
      const bool better = ev.kernels > bestKernels || (ev.kernels == bestKernels && ev.latencyMs < minLatency);
      if (bestKernels < 0 || (ev.latencyMs != FLT_MAX && better)) {
        minLatency = ev.latencyMs;
        bestKernels = ev.kernels;
        saveBestModule(module);
        ev.kept = true;
        for (auto& other : evaluationLog)
          if (other.optimizer == ev.optimizer) other.kept = false;
      }
      if (KCGLog::level == Log::Debug)
        llvm::errs() << "optimize: " << ev.optimizer << " config " << ev.configIndex << ": " << ev.kernels << " kernels, "
                     << ev.latencyMs << " ms" << (ev.note.empty() ? "" : " (" + ev.note + ")") << "\n";
      evaluationLog.push_back(ev);
    };
    if (configs && active) {
      int index = 0;
      for (auto& config : *configs) {
        *active = config;
        resetModule(module);
        tryOnce(index++);
      }
    } else {
      tryOnce(0);
    }
  }
  return bestModule;
}

namespace {

// Device buffers of one kernel launch, filled with seeded synthetic operands.
struct BufferSet {
  std::vector<void*> buffers;
  std::vector<float> scalars;
  std::vector<void*> argPtrs;
  ~BufferSet() {
    for (void* b : buffers)
      if (b) kcg_hip_free(b);
  }
};

// Fills a device buffer with `count` elements of `dtype` drawn from U(lo, hi) (stream `stream` of the seeded
// host generator).  The host makes at most 4 Mi elements; longer buffers repeat them.
bool fillDevice(void* dst, int64_t bytes, int dtype, double lo, double hi, uint64_t stream) {
  const size_t esize = kcg_dtype_size(dtype);
  if (esize == 0 || bytes <= 0) return false;
  const size_t count = (size_t)bytes / esize;
  const size_t chunk = std::min<size_t>(count, (size_t)4 << 20);
  std::vector<char> host(chunk * esize);
  // e4m3 operands are spread over the format's range; their per-tensor scales bring the products back
  const float scale = dtype == KCG_DT_F8E4M3 ? 448.0f / (float)std::max(std::fabs(lo), std::fabs(hi)) : 1.0f;
  if (kcg_host_fill(host.data(), chunk, dtype, KCG_DIST_UNIFORM, 0x4B4347ull, stream, (float)lo, (float)hi, scale) != KCG_OK)
    return false;
  for (size_t done = 0; done < count; done += chunk) {
    const size_t n = std::min(chunk, count - done);
    if (kcg_hip_memcpy_h2d((char*)dst + done * esize, host.data(), n * esize) != KCG_OK) return false;
  }
  return true;
}

}  // namespace

float KernelCodeGenerator::evaluate(mlir::ModuleOp& module) { return evaluate(module, nullptr, nullptr); }

float KernelCodeGenerator::evaluate(mlir::ModuleOp& module, int* numKernels, std::string* note) {
  auto fail = [&](const std::string& why) {
    if (note) *note = why;
    if (KCGLog::level == Log::Debug) llvm::errs() << "evaluate: " << why << "\n";
    return FLT_MAX;
  };
  if (numKernels) *numKernels = 0;
  std::vector<KernelLaunchInfo> infos;
  std::vector<std::string> skipped;
  std::string error;
  applyLowering(module);
  std::string source = HIPGen(module, infos, &error, &skipped);
  if (!error.empty()) return fail("no source: " + error);
  if (numKernels) *numKernels = (int)infos.size();
  if (note && !skipped.empty()) {
    *note = "not scheduled:";
    for (auto& f : skipped) *note += " " + f;
  }
  if (lowerOnly) {
    if (note) *note += std::string(note->empty() ? "" : "; ") + "only candidate, not timed";
    return infos.empty() ? fail("no kernel was emitted") : 0.0f;
  }
  int devices = 0;
  if (kcg_hip_device_count(&devices) != KCG_OK || devices <= 0) return 0.0f;      // no GPU: every candidate ties
  if (infos.empty()) return fail("no kernel was emitted");
  if (kcg_hip_init(0) != KCG_OK) return fail("the device could not be initialised");
  kcg_module_t mod = nullptr;
  std::vector<char> log(1 << 16);
  if (int rc = kcg_hip_compile_cached(source.c_str(), nullptr, 0, &mod, log.data(), log.size())) {
    llvm::errs() << "evaluate: generated source does not compile:\n" << log.data() << "\n";
    return fail(std::string("compile: ") + kcg_hip_strerror(rc));
  }
  float total = 0.0f;
  std::string why;
  for (auto& info : infos) {
    kcg_kernel_t kernel = nullptr;
    if (int rc = kcg_hip_get_kernel(mod, info.name.c_str(), &kernel)) { why = info.name + ": " + kcg_hip_strerror(rc); break; }
    const uint32_t numBuffers = info.numArgs - info.numScalars;      // the trailing arguments are fp32 scalars
    if (info.argBytes.size() != numBuffers || info.argTypes.size() != numBuffers) { why = info.name + ": argument table mismatch"; break; }
    // Operand sets used in turn, so that a launch finds its operands in HBM and not in the 256 MB last-level
    // cache: three, or as many as 6 GiB hold.
    int64_t setBytes = 0;
    for (auto b : info.argBytes) setBytes += b;
    const int numSets = (int)std::max<int64_t>(1, std::min<int64_t>(3, ((int64_t)6 << 30) / std::max<int64_t>(1, setBytes)));
    std::vector<BufferSet> sets((size_t)numSets);
    for (int s = 0; s < numSets && why.empty(); ++s) {
      BufferSet& set = sets[(size_t)s];
      set.buffers.assign(numBuffers, nullptr);
      // per-tensor scales of an fp8 product undo the spread that fillDevice gives its operands
      set.scalars.assign(info.numScalars, (float)(std::max(std::fabs(info.fillLo), std::fabs(info.fillHi)) / 448.0));
      for (uint32_t i = 0; i < numBuffers && why.empty(); ++i) {
        if (int rc = kcg_hip_malloc(&set.buffers[i], (size_t)info.argBytes[i])) { why = info.name + ": " + kcg_hip_strerror(rc); break; }
        // every buffer gets data, the result buffer too (it is overwritten; an in-place operator reads it)
        const bool ok = (int)i == info.workspaceArg
                            ? kcg_hip_memset(set.buffers[i], 0, (size_t)info.argBytes[i]) == KCG_OK
                            : fillDevice(set.buffers[i], info.argBytes[i], info.argTypes[i], info.fillLo, info.fillHi,
                                         (uint64_t)(16 * s + i + 1));
        if (!ok) why = info.name + ": could not fill an operand";
      }
      for (auto& b : set.buffers) set.argPtrs.push_back(&b);
      for (auto& sc : set.scalars) set.argPtrs.push_back(&sc);
    }
    if (!why.empty()) break;
    std::vector<void**> argSets;
    for (auto& set : sets) argSets.push_back(set.argPtrs.data());
    // 30 ms of untimed launches bring the clocks up (the first candidate would otherwise be timed at idle
    // clocks); then the median of seven groups of three launches.
    float median = 0.0f;
    if (int rc = kcg_hip_time_rotating(kernel, info.grid, info.block, info.ldsBytes, nullptr, argSets.data(), numSets,
                                       3, 30.0f, 7, 3, &median, nullptr)) {
      why = info.name + ": " + kcg_hip_strerror(rc);
      break;
    }
    total += median;
  }
  kcg_hip_module_destroy(mod);
  if (!why.empty()) return fail(why);
  return total;
}

}  // namespace KernelCodeGen
