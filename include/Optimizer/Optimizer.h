#pragma once
// Per-operator schedules: each Optimizer recognises its operator's naive nests
// in a module (applicable) and rewrites them into a GPU schedule
// (applyOptimzer [sic]) with the Rewriter primitives, driven by a static
// configuration map.  Interface follows the reference
// (include/Optimizer/Optimizer.h:29-286).

#include <map>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#include "Frontend/Operators.h"
#include "IR/IR.h"
#include "Optimizer/Analyzer.h"
#include "Optimizer/Rewriter.h"

// Shape and operand layouts of one batched matmul, parsed from its function name.
struct BatchMatmulDescriptor {
  int m = 0, n = 0, k = 0;
  bool transA = false, transB = false;
  std::vector<int> batch;
  void log() {
    auto& os = llvm::errs();
    os << "m = " << m << " n = " << n << " k = " << k << "\nbatch = ";
    for (int extent : batch) os << extent << ",";
    os << "\ntrans A = " << transA << " transB = " << transB << "\n";
  }
};

namespace KernelCodeGen {

// Parses "BatchMatmul_<b0>_<b1>.._m<M>_n<N>_k<K>_<N|T><N|T>"; false if the name has another form.
bool identifyBatchMatmul(const std::string& name, BatchMatmulDescriptor& matmul);

struct Optimizer {
  virtual ~Optimizer() = default;
  virtual bool applicable(mlir::ModuleOp& module) = 0;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) = 0;
  bool operator==(const Optimizer& other) { return name == other.name; }
  std::string name;
};

struct MatmulOptimizer : Optimizer {
  MatmulOptimizer() { this->name = "Matmul"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  // "loadTileA", "loadTileB", "storeTileA", "storeTileB", "loadFragA", "loadFragB",
  // "cacheReadA", "cacheReadB", "cacheWriteC"
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder);
  void clear() { matmuls.clear(); matmulLoops.clear(); matmulBuffers.clear(); raggedMatmuls.clear(); }
  std::set<mlir::func::FuncOp, CompareFunc> matmuls;
  // Of those, the products whose extents are not multiples of the tile (the reference's optimizer leaves such a
  // product unscheduled): they get the guarded schedule of applyOptimzer instead of the pipelined one.
  std::set<mlir::func::FuncOp, CompareFunc> raggedMatmuls;
  std::map<mlir::func::FuncOp, std::vector<mlir::AffineForOp>, CompareFunc> matmulLoops;
  struct MemoryBuffer { mlir::Value A, B, C; };
  std::map<mlir::func::FuncOp, MemoryBuffer, CompareFunc> matmulBuffers;
  static std::map<std::string, int> matmulConfig;
};

// Broadcasting fp32 Binary nests (Add, Sub, Mul, Div, Pow, Equal, Greater): collapsed to one dimension, split
// over workgroups and lanes, vectorised along the innermost dimension
// (reference: include/Optimizer/Optimizer.h:98-116).
struct BinaryOptimizer : Optimizer {
  BinaryOptimizer() { this->name = "Binary"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  // Index maps of a 2-d refold of the nest: "MaxLoadOrStore", "MinVectorLoad", "CacheLoadOrStore"
  // (csrc/optimizer/OptimizerMembers.cc describes inputs and `extras`).
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder, const std::vector<int64_t>& extras = {},
                               const int needDims = 0, const int oneDimNums = 0);
  llvm::SmallVector<mlir::Value> getMinLoadOperands(int dim, llvm::SmallVector<mlir::Value> operands, const mlir::Value cst = nullptr);
  // How the smaller operand broadcasts into the larger one.
  enum class BinaryType {
    constant = 0,        // no second tensor
    allOne = 1,          // every extent 1
    allEqual = 2,        // (2, 20, 256), (2, 20, 256)
    hasOneOrder = 3,     // (2, 20, 256), (1, 20, 256)   (2, 20, 256), (1, 256)
    noOneOrder = 4,      // (2, 20, 256), (20, 256)
    hasOneUnorder = 5    // (2, 20, 256), (20, 1)        (2, 20, 256), (1, 20, 1)
  };
  struct BinaryOpData {
    BinaryType type;
    int oneDimNums = 0;
    int needDimNums = 0;
  };
  void getBinaryOpData(mlir::Value max_load, mlir::Value min_load, BinaryOpData& data);
  void clear() { binaryBuffers.clear(); binarys.clear(); binaryLoops.clear(); }
  struct MemoryBuffer { mlir::Value A, B, C; };
  std::map<mlir::func::FuncOp, MemoryBuffer, CompareFunc> binaryBuffers;
  std::set<mlir::func::FuncOp, CompareFunc> binarys;
  std::map<mlir::func::FuncOp, std::vector<mlir::AffineForOp>, CompareFunc> binaryLoops;
  static std::map<std::string, int> binaryConfig;
};

struct ElementWiseOptimizer : Optimizer {
  ElementWiseOptimizer() { this->name = "ElementWise"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  // "load" / "store": (blockIdx.y, blockIdx.x, threadIdx.y, threadIdx.x, row in tile) -> (row, column)
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder, const std::vector<int64_t>& extras = {});
  void clear() { elementWiseBuffers.clear(); elementWises.clear(); elementWiseLoops.clear(); }
  struct MemoryBuffer { mlir::Value input, output; };
  std::map<mlir::func::FuncOp, MemoryBuffer, CompareFunc> elementWiseBuffers;
  std::set<mlir::func::FuncOp, CompareFunc> elementWises;
  std::map<mlir::func::FuncOp, std::vector<mlir::AffineForOp>, CompareFunc> elementWiseLoops;
  static std::map<std::string, int> elementWiseConfig;
};

struct LayerNormOptimizer : Optimizer {
  LayerNormOptimizer() { this->name = "LayerNorm"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder, const std::vector<int64_t>& extras = {});
  // Rewrites on the row passes of a LayerNorm-like nest (csrc/optimizer/OptimizerMembers.cc): merging thread
  // levels, staging loads through a cache, loop fission in front of a reduction, splitting off the store,
  // the wavefront-shuffle reduction tree and the lane-strided unrolling of an element-wise pass.
  mlir::AffineParallelOp combineParallel(std::vector<mlir::AffineParallelOp> pals);
  mlir::AffineForOp write(mlir::AffineForOp forOp, std::vector<mlir::Value> buffers);
  mlir::AffineForOp extractOpsFromLoop(mlir::AffineForOp forOp, std::vector<mlir::Value> buffers);
  std::vector<mlir::AffineForOp> read(mlir::AffineForOp forOp, std::vector<mlir::Value> buffers);
  std::vector<mlir::Operation*> reduceUnrollOptimize(mlir::AffineForOp forOp, mlir::AffineParallelOp pal);
  void elementWiseUnrollOptimize(mlir::AffineForOp forOp, mlir::AffineParallelOp pal);
  void clear() { layerNormBuffers.clear(); layerNorms.clear(); layerNormLoops.clear(); }
  struct MemoryBuffer { mlir::Value input, scale, bias, output; };
  std::map<mlir::func::FuncOp, MemoryBuffer, CompareFunc> layerNormBuffers;
  std::set<mlir::func::FuncOp, CompareFunc> layerNorms;
  // per function: {outer loops, sum nest, variance nest, normalise nest}
  std::map<mlir::func::FuncOp, std::vector<std::vector<mlir::AffineForOp>>, CompareFunc> layerNormLoops;
  static std::map<std::string, int> layerNormConfig;
};

// reference: include/Optimizer/Optimizer.h:185-208, src/Optimizer/Optimizer.cc:1940-2074
struct GatherOptimizer : Optimizer {
  GatherOptimizer() { this->name = "Gather"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  // "VectorLoadOrStore" / "PointLoadOrStore"
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder, const std::vector<int64_t>& extras = {});
  // Hoists the single index load of a one-index gather out of `forOp` to the start of the level `pal`.
  void oneIndexLoad(mlir::AffineForOp forOp, mlir::AffineParallelOp pal);
  void clear() { gatherBuffers.clear(); gathers.clear(); gatherLoops.clear(); }
  struct MemoryBuffer { mlir::Value input, indices, output; };
  std::map<mlir::func::FuncOp, MemoryBuffer, CompareFunc> gatherBuffers;
  std::set<mlir::func::FuncOp, CompareFunc> gathers;
  std::map<mlir::func::FuncOp, std::vector<mlir::AffineForOp>, CompareFunc> gatherLoops;
  static std::map<std::string, int> gatherConfig;
};

// No counterpart class in the reference (it schedules softmax only inside its fused attention); added so that
// a Softmax call that no fusion has taken still becomes a kernel.  Config keys: BLOCK_SIZE / THREAD_SIZE
// (threads per row = their quotient), THREADS_PER_ROW (overrides), VECTORIZE_WIDTH.
struct SoftmaxOptimizer : Optimizer {
  SoftmaxOptimizer() { this->name = "Softmax"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  void clear() { softmaxes.clear(); softmaxLoops.clear(); }
  std::set<mlir::func::FuncOp, CompareFunc> softmaxes;
  // per function: {outer loops, {sum loop}, {store loop}}
  std::map<mlir::func::FuncOp, std::vector<std::vector<mlir::AffineForOp>>, CompareFunc> softmaxLoops;
  static std::map<std::string, int> softmaxConfig;
};

struct FMHAOptimizer : Optimizer {
  FMHAOptimizer() { this->name = "FMHA"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  // The reference's 18 names ("loadTileQ", "loadTileK", "storeTileQ", "storeTileK", "loadFragQ", "loadFragK", "brIdxS",
  // "storeTileP", "readTileS", "loadFactor", "loadTileV", "storeTileV", "loadFragP", "loadFragV", "brIdxO", "storeTileO")
  // and "bcIdxS" while the tiled schedule's keys are in fmhaConfig; else the row-per-thread form's five.
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder);
  // fmhaConfig holds every key of the tiled schedule (the reference's, and the tile extents Hd, Br, Bc)
  static bool tiledConfig();
  // Tile extents Br, Bc of the tiled schedule for a (sequence length, head dim) under fmhaConfig, and whether every
  // layout rule of that schedule holds for them (each tensor tiled exactly once by the index maps); `why` says which not.
  static bool tiledLayout(int64_t seq, int64_t hd, int64_t& br, int64_t& bc, std::string* why = nullptr);
  // Queries per workgroup of the row-per-thread schedule (BLOCK_SIZE, or ROW_BLOCK_SIZE beside the tiled schedule's keys).
  static int rowBlockSize();
  // Fills the empty fused function with the reference's tiled schedule (src/Optimizer/Optimizer.cc:2606-2860).
  void buildTiledSchedule(mlir::func::FuncOp funcOp, mlir::OpBuilder& builder, int64_t batch, int64_t heads, int64_t seq_len,
                          int64_t head_dim, bool causal, bool scaled);
  // One online-softmax step over a score tile (running maximum, running sum, rescale factor).
  void softmaxIR(mlir::OpBuilder& builder, mlir::Value tileS, mlir::Value rowMax, mlir::Value smMax, mlir::Value rowSum,
                 mlir::Value smSum, mlir::Value smFac, mlir::Value zero, mlir::Value flt_min, mlir::Value tid);
  void clear() { uniqueFuncCalls.clear(); call2callsMap.clear(); call2bufferMap.clear(); }
  std::set<mlir::func::CallOp, CompareFuncCall> uniqueFuncCalls;
  // first batched matmul call -> {softmax call, second batched matmul call}
  std::map<mlir::func::CallOp, std::vector<mlir::func::CallOp>, CompareFuncCall> call2callsMap;
  struct MemoryBuffer { mlir::Value Q, K, S, V, O; BatchMatmulDescriptor matmul1; BatchMatmulDescriptor matmul2; };
  std::map<mlir::func::CallOp, MemoryBuffer, CompareFuncCall> call2bufferMap;
  static std::map<std::string, int> fmhaConfig;
};

struct BatchMatmulOptimizer : Optimizer {
  BatchMatmulOptimizer() { this->name = "BatchMatmul"; }
  virtual bool applicable(mlir::ModuleOp& module) override;
  virtual void applyOptimzer(mlir::ModuleOp& module, mlir::OpBuilder& builder) override;
  mlir::AffineMap getAffineMap(const std::string& mapIdentifier, mlir::OpBuilder& builder);
  // One-dimensional thread level -> {threadIdx.y, threadIdx.x} values.
  std::vector<mlir::Value> threadLevelOneToTwo(mlir::AffineParallelOp pal);
  void clear() { batchMatmulBuffers.clear(); batchMatmuls.clear(); batchMatmulLoops.clear(); raggedBatchMatmuls.clear(); }
  // of batchMatmuls, the products whose extents are not multiples of the tile (guarded schedule, as in MatmulOptimizer)
  std::set<mlir::func::FuncOp, CompareFunc> raggedBatchMatmuls;
  struct MemoryBuffer { mlir::Value A, B, C; BatchMatmulDescriptor matmul; };
  std::map<mlir::func::FuncOp, MemoryBuffer, CompareFunc> batchMatmulBuffers;
  std::set<mlir::func::FuncOp, CompareFunc> batchMatmuls;
  std::map<mlir::func::FuncOp, std::vector<mlir::AffineForOp>, CompareFunc> batchMatmulLoops;
  static std::map<std::string, int> batchMatmulConfig;
};

}  // namespace KernelCodeGen
