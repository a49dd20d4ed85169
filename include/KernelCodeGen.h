#pragma once
// Entry point of the library: build a graph of operators, schedule it with the
// per-operator optimizers, generate gfx950 HIP source.
//
//   KernelCodeGenerator generator("ROCm");
//   auto graph = generator.createGraph("demo");
//   generator.opts.push_back(std::make_unique<MatmulOptimizer>());
//   auto A = graph.create<PlaceHolder>(std::vector<int64_t>{m, k}, std::string{"float32"});
//   auto B = graph.create<PlaceHolder>(std::vector<int64_t>{k, n}, std::string{"float32"});
//   auto C = graph.create<Matmul>(A, B);
//   auto module = generator.optimize(graph);
//   auto source = generator.codegen(module);
//
// The class keeps the members of the reference's KernelCodeGenerator
// (include/KernelCodeGen.h:25-165).  Differences: the platform is "ROCm" (also
// accepted: "HIP", "gfx950"); any other platform makes codegen() report an
// error instead of falling off the end of the function; the configuration
// tables hold gfx950 tile sizes (64-wide wavefronts); evaluate() times the
// generated kernels when a GPU is present.

#include <cfloat>
#include <climits>
#include <fstream>
#include <initializer_list>
#include <memory>
#include <sstream>
#include <string>

#include "Backend/HIP.h"
#include "Frontend/Operators.h"
#include "Optimizer/Optimizer.h"
#include "log.h"

namespace KernelCodeGen {

class KernelCodeGenerator {
public:
  using ConfigList = std::vector<std::map<std::string, int>>;

  KernelCodeGenerator(const std::string& platform_ = {"ROCm"}) : builder(&context), graph(builder), platform(platform_) {
    initMLIRContext();
    // Tile sizes for gfx950.  A config with DTYPE_BITS applies to operands of
    // that width only; optimize() tries the configs of an operator in order.
    matmulConfigs = {
        {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 8},
         {"THREAD_SIZE_N", 8}, {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 32}},
        {{"BLOCK_SIZE_M", 256}, {"BLOCK_SIZE_N", 256}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 8},
         {"THREAD_SIZE_N", 8}, {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 32}},
        {{"BLOCK_SIZE_M", 64}, {"BLOCK_SIZE_N", 64}, {"BLOCK_SIZE_K", 32}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 4},
         {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 32}},
        {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 32}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 4},
         {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 32}},
        {{"BLOCK_SIZE_M", 256}, {"BLOCK_SIZE_N", 256}, {"BLOCK_SIZE_K", 64}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 16},
         {"THREAD_SIZE_N", 8}, {"VECTORIZE_WIDTH", 8}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 16}},
        {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 64}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 8},
         {"THREAD_SIZE_N", 8}, {"VECTORIZE_WIDTH", 8}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 16}},
        {{"BLOCK_SIZE_M", 256}, {"BLOCK_SIZE_N", 256}, {"BLOCK_SIZE_K", 128}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 16},
         {"THREAD_SIZE_N", 16}, {"VECTORIZE_WIDTH", 16}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 8}},
        // f64 (v_mfma_f64_16x16x4_f64 family; two doubles per 16-byte access in the schedule)
        {{"BLOCK_SIZE_M", 64}, {"BLOCK_SIZE_N", 64}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 4},
         {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 2}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 64}},
        {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 4},
         {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 2}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 64}},
        {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 256}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 4},
         {"THREAD_SIZE_N", 8}, {"VECTORIZE_WIDTH", 2}, {"WARP_SIZE", 64}, {"DTYPE_BITS", 64}},
    };
    binaryConfigs = {{{"BLOCK_SIZE_M", 64}, {"BLOCK_SIZE_N", 64}, {"THREAD_SIZE_M", 4}, {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 4}}};
    elementWiseConfigs = {{{"BLOCK_SIZE_M", 64}, {"BLOCK_SIZE_N", 64}, {"THREAD_SIZE_M", 4}, {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 4}}};
    // teams of 512, 256 and 1024 threads per normalised row (BLOCK_SIZE / THREAD_SIZE): which is fastest depends on
    // the row length, so with a device present optimize() measures them
    layerNormConfigs = {{{"BLOCK_SIZE", 2048}, {"THREAD_SIZE", 4}, {"VECTORIZE_WIDTH", 4}},
                        {{"BLOCK_SIZE", 1024}, {"THREAD_SIZE", 4}, {"VECTORIZE_WIDTH", 4}},
                        {{"BLOCK_SIZE", 4096}, {"THREAD_SIZE", 4}, {"VECTORIZE_WIDTH", 4}}};
    gatherConfigs = {{{"BLOCK_SIZE_M", 64}, {"BLOCK_SIZE_N", 64}, {"THREAD_SIZE_M", 4}, {"THREAD_SIZE_N", 4}, {"VECTORIZE_WIDTH", 4}}};
    softmaxConfigs = {{{"BLOCK_SIZE", 1024}, {"THREAD_SIZE", 4}, {"VECTORIZE_WIDTH", 4}},
                      {{"BLOCK_SIZE", 2048}, {"THREAD_SIZE", 4}, {"VECTORIZE_WIDTH", 4}},
                      {{"BLOCK_SIZE", 512}, {"THREAD_SIZE", 4}, {"VECTORIZE_WIDTH", 4}}};
    // The reference's tiled attention schedule (its include/KernelCodeGen.h:51-54) with 64-lane layout units; what it
    // does not fit (16-bit operands, ragged sequence lengths) gets one query row per thread, ROW_BLOCK_SIZE queries per
    // workgroup.  CAUSAL and SCALE_RSQRT_D are this build's.
    fmhaConfigs = {{{"BLOCK_SIZE", 128}, {"HdxBr", 128 * 64}, {"BrxBc", 128 * 64}, {"WarpX_O", 2}, {"Slice", 8}, {"BrTileS", 8},
                    {"BcTileS", 8}, {"BrTileO", 8}, {"HdTileO", 8}, {"Width", 4}, {"WARP_SIZE", 64}, {"ROW_BLOCK_SIZE", 256},
                    {"CAUSAL", 0}, {"SCALE_RSQRT_D", 0}}};
    batchMatmulConfigs = matmulConfigs;
  }

  void initMLIRContext() {
    context.getOrLoadDialect<mlir::AffineDialect>();
    context.getOrLoadDialect<mlir::memref::MemRefDialect>();
    context.getOrLoadDialect<mlir::func::FuncDialect>();
    context.getOrLoadDialect<mlir::arith::ArithmeticDialect>();
    context.getOrLoadDialect<mlir::gpu::GPUDialect>();
    context.getOrLoadDialect<mlir::vector::VectorDialect>();
    context.getOrLoadDialect<mlir::scf::SCFDialect>();
    context.getOrLoadDialect<mlir::math::MathDialect>();
    mlir::registerAllPasses();
  }

  ComputeDAG& createGraph(const std::string& graphName) {
    minLatency = FLT_MAX;
    graph.module = mlir::ModuleOp::create(builder.getUnknownLoc(), mlir::Optional<mlir::StringRef>(graphName));
    graph.builder.setInsertionPointToEnd(graph.module.getBody());
    return graph;
  }

  ComputeDAG& getGraph() { return graph; }

  void dump(mlir::ModuleOp& module, const std::string& info = "") {
    if (KCGLog::level == Log::Release) return;
    llvm::errs() << "----------------------------------------------------------\n";
    llvm::errs() << "           " << info << "\n";
    llvm::errs() << "----------------------------------------------------------\n";
    module->dump();
    if (mlir::failed(mlir::verify(module))) {
      module->emitError("module verification error");
      assert(false);
    }
  }

  // "terminal" writes to stdout.
  void save(const std::string& str, const std::string& file) {
    if (file == "terminal") {
      llvm::outs() << str;
      return;
    }
    std::ofstream fileWriter(file.c_str());
    if (!fileWriter.is_open()) {
      llvm::errs() << "Can't open file \"" << file << "\"\n";
      return;
    }
    fileWriter << str;
  }

  void resetModule(mlir::ModuleOp& module) { module = backupModule_.clone(); }
  void backupModule(mlir::ModuleOp& module) { backupModule_ = module.clone(); }
  void saveBestModule(mlir::ModuleOp& module) { bestModule = module.clone(); }

  mlir::ModuleOp& optimize(ComputeDAG& graph_);

  // Latency in milliseconds of all kernels of `module`: every kernel is launched on seeded synthetic
  // operands (three operand sets used in turn, so that no launch finds its operands in the last-level
  // cache), after 30 ms of warm-up launches, and the median of seven event-timed groups counts; code objects
  // go through the on-disk cache.  0 when no GPU is present (every candidate then ties and the first
  // applicable config is kept, as in the reference, whose evaluate() always returns 0,
  // include/KernelCodeGen.h:134-136).  FLT_MAX when the module emits no kernel, does not compile or does
  // not launch; `note` then says why, and otherwise lists the called operators that are not scheduled.
  float evaluate(mlir::ModuleOp& module);
  float evaluate(mlir::ModuleOp& module, int* numKernels, std::string* note);
  // optimize() sets this while an optimizer has a single configuration to offer: the candidate is still lowered
  // (so that one the backend cannot translate is known), but there is nothing to choose between and no kernel is
  // launched; evaluate() then returns 0 with the note "only candidate, not timed".
  bool lowerOnly = false;

  // One line per candidate of the last optimize(): which optimizer and configuration, how many kernels the
  // candidate emitted, its latency (FLT_MAX: failed, see note) and whether it is the one that was kept.
  struct Evaluation {
    std::string optimizer;
    int configIndex = 0;
    std::map<std::string, int> config;
    int kernels = 0;
    float latencyMs = FLT_MAX;
    bool kept = false;
    std::string note;
  };
  const std::vector<Evaluation>& evaluations() const { return evaluationLog; }

  // HIP source for gfx950; launch geometry of the kernels in launchInfos().
  std::string codegen(mlir::ModuleOp module) {
    if (platform == "ROCm" || platform == "HIP" || platform == "gfx950") {
      std::string error;
      applyLowering(module);
      std::string source = HIPGen(module, lastLaunchInfos, &error, &lastSkipped);
      if (!error.empty()) llvm::errs() << "codegen failed: " << error << "\n";
      for (auto& f : lastSkipped) llvm::errs() << "codegen: " << f << " is called but not scheduled: no kernel for it\n";
      lastError = error;
      return source;
    }
    lastError = "platform \"" + platform + "\" is not supported; this build targets ROCm (gfx950) only";
    llvm::errs() << lastError << "\n";
    lastLaunchInfos.clear();
    lastSkipped.clear();
    return std::string();
  }

  // The lowering asked for with setLowering(), written on the module where the backend reads it.  evaluate() does the
  // same, so that the config search rates the kernels codegen() will emit (schedules printed statement by statement
  // when that was asked for).
  void applyLowering(mlir::ModuleOp module) const {
    if (lowering == "schedule" || lowering == "families-only") module->setAttr("kcg.lowering", mlir::StringAttr::get(nullptr, lowering));
    else if (loweringWasSet) module->removeAttr("kcg.lowering");
  }

  // Host program (plain C over include/kcg_hip.h) for the kernels of the last codegen() call, whose source
  // the caller has saved as `kernelFile`: it compiles that file with hipRTC, fills every kernel's operands
  // from the seeded host generator, launches the kernel, compares a sample of its result with a plain C
  // evaluation of the operator on the same operands ("max rel err", "correctness: Done" or "FAILED"), times
  // it on three operand sets in turn and prints one line per kernel; its exit status is non-zero when a
  // check fails.  It takes the place of the adaptor + out-of-tree harness of the reference's flow
  // (test/test.cc:69-104, performance/output.log).  Build with
  //   cc adaptor.c -I include -L kernelcodegen_amd -lkcg_hip -Wl,-rpath,kernelcodegen_amd -o adaptor
  std::string adaptor(const std::string& kernelFile) const;

  // Which lowering codegen() uses from now on: "families" (a kernel family per recognised operator, the schedule
  // itself for what no family takes) or "schedule" (every function's scheduled body printed statement by statement,
  // as the reference's backend does).  Without a call the module's own "kcg.lowering" attribute decides, families by
  // default.  "families-only" is "families" without the way out: a function that its kernel family refuses is an
  // error of codegen() instead of a (much slower) statement-by-statement kernel.  False for another word.
  bool setLowering(const std::string& mode) {
    if (mode != "families" && mode != "schedule" && mode != "families-only") return false;
    lowering = mode;
    loweringWasSet = true;
    return true;
  }

  const std::vector<KernelLaunchInfo>& launchInfos() const { return lastLaunchInfos; }
  // Operators of the last codegen() that the graph calls but no optimizer has scheduled: they have no kernel.
  const std::vector<std::string>& skippedFunctions() const { return lastSkipped; }
  const std::string& error() const { return lastError; }

  void setLogMode(Log level) { KCGLog::level = level; }

  // Replace the configuration candidates of one optimizer ("Matmul", "BatchMatmul",
  // "ElementWise", "LayerNorm", "FMHA", "Binary", "Gather", "Softmax").  False for an unknown name.
  bool setConfigs(const std::string& optimizerName, const ConfigList& configs);
  const ConfigList* getConfigs(const std::string& optimizerName) const;

public:
  std::vector<std::unique_ptr<Optimizer>> opts;

private:
  mlir::MLIRContext context;
  mlir::OpBuilder builder;
  mlir::ModuleOp backupModule_;
  mlir::ModuleOp bestModule;
  ComputeDAG graph;
  std::string platform;
  float minLatency = FLT_MAX;
  ConfigList matmulConfigs;
  ConfigList fmhaConfigs;
  ConfigList binaryConfigs;
  ConfigList elementWiseConfigs;
  ConfigList gatherConfigs;
  ConfigList softmaxConfigs;
  ConfigList layerNormConfigs;
  ConfigList batchMatmulConfigs;
  std::vector<KernelLaunchInfo> lastLaunchInfos;
  std::vector<std::string> lastSkipped;
  std::string lowering;
  bool loweringWasSet = false;
  std::vector<Evaluation> evaluationLog;
  std::string lastError;
};

}  // namespace KernelCodeGen
