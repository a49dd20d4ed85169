// KernelCodeGenerator::optimize / evaluate (declared in include/KernelCodeGen.h;
// reference: src/KernelCodeGen.cc:8-120).
#include "KernelCodeGen.h"

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
// fresh copy of the module, keep the fastest result.  Optimizers are applied
// one after the other, each starting from the best module of the previous one.
mlir::ModuleOp& KernelCodeGenerator::optimize(ComputeDAG& graph_) {
  graph = graph_;
  mlir::ModuleOp module = graph.module.clone();
  saveBestModule(module);

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
    module = bestModule.clone();
    backupModule(module);
    const ConfigList* configs = getConfigs(opt->name);
    std::map<std::string, int>* active = staticConfigOf(opt->name);
    auto tryOnce = [&]() {
      if (!opt->applicable(module)) return;
      opt->applyOptimzer(module, builder);
      const float latency = evaluate(module);
      if (latency < minLatency) {
        minLatency = latency;
        saveBestModule(module);
      }
    };
    if (configs && active) {
      for (auto& config : *configs) {
        *active = config;
        resetModule(module);
        tryOnce();
      }
    } else {
      tryOnce();
    }
  }
  return bestModule;
}

float KernelCodeGenerator::evaluate(mlir::ModuleOp& module) {
  int devices = 0;
  if (kcg_hip_device_count(&devices) != KCG_OK || devices <= 0) return 0.0f;
  std::vector<KernelLaunchInfo> infos;
  std::string error;
  std::string source = HIPGen(module, infos, &error);
  if (source.empty() || infos.empty()) return infos.empty() && error.empty() ? 0.0f : FLT_MAX;
  if (kcg_hip_init(0) != KCG_OK) return 0.0f;
  kcg_module_t mod = nullptr;
  char log[4096];
  if (kcg_hip_compile(source.c_str(), nullptr, 0, &mod, log, sizeof log) != KCG_OK) {
    llvm::errs() << "evaluate: generated source does not compile:\n" << log << "\n";
    return FLT_MAX;
  }
  float total = 0.0f;
  bool ok = true;
  for (auto& info : infos) {
    kcg_kernel_t kernel = nullptr;
    if (kcg_hip_get_kernel(mod, info.name.c_str(), &kernel) != KCG_OK) { ok = false; break; }
    const uint32_t numBuffers = info.numArgs - info.numScalars;      // the trailing arguments are fp32 scalars
    if (info.argBytes.size() != numBuffers) { ok = false; break; }
    std::vector<void*> buffers(numBuffers, nullptr);
    std::vector<void*> argPtrs;
    std::vector<float> scalars(info.numScalars, 1.0f);
    for (uint32_t i = 0; i < numBuffers && ok; ++i) {
      ok = kcg_hip_malloc(&buffers[i], (size_t)info.argBytes[i]) == KCG_OK &&
           kcg_hip_memset(buffers[i], 0, (size_t)info.argBytes[i]) == KCG_OK;
    }
    for (auto& b : buffers) argPtrs.push_back(&b);
    for (auto& s : scalars) argPtrs.push_back(&s);
    float ms = 0.0f;
    if (ok) ok = kcg_hip_time_launches(kernel, info.grid, info.block, info.ldsBytes, nullptr, argPtrs.data(), 2, 10, &ms) == KCG_OK;
    for (auto b : buffers) if (b) kcg_hip_free(b);
    if (!ok) break;
    total += ms;
  }
  kcg_hip_module_destroy(mod);
  return ok ? total : FLT_MAX;
}

}  // namespace KernelCodeGen
