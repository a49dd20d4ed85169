#pragma once
// Affine rewrite primitives the optimizers script into GPU schedules.
// Signatures follow the reference (include/Optimizer/Rewriter.h:16-273); the
// implementation is in kernelcodegen_amd/csrc/optimizer/Rewriter.cc.

#include <vector>

#include "IR/IR.h"
#include "Optimizer/Analyzer.h"
#include "enum.h"

namespace KernelCodeGen {

struct Rewriter {
  Rewriter() = default;

  static mlir::OpBuilder getBuilder(mlir::AffineForOp op, Position pos) {
    switch (pos) {
      case Position::after: {
        mlir::OpBuilder builder(op->getContext());
        builder.setInsertionPointAfter(op);
        return builder;
      }
      case Position::before: return mlir::OpBuilder(op.getOperation());
      case Position::begin: return mlir::OpBuilder::atBlockBegin(op.getBody());
      case Position::end: return mlir::OpBuilder::atBlockTerminator(op.getBody());
    }
    assert(false);
    return mlir::OpBuilder();
  }

  static std::vector<mlir::Value> getParallelIdx(mlir::AffineParallelOp parallelLevel) { return parallelLevel.getIVs(); }

  // For each index of the level, the result of the first affine.apply that uses it.
  static std::vector<mlir::Value> getElementIdx(mlir::AffineParallelOp parallelLevel) {
    std::vector<mlir::Value> idxes;
    for (auto iv : parallelLevel.getIVs())
      for (auto user : iv.getUsers())
        if (auto mapOp = mlir::dyn_cast<mlir::AffineApplyOp>(user)) {
          idxes.push_back(mapOp.getResult());
          break;
        }
    return idxes;
  }

  // Loop `0..ub step 1` -> nest of num_output loops with steps [.., f2, f1, 1]
  // and extents [ub, .., f2, f1] (factors given innermost first, e.g. {8, 128}).
  // Every use of the old index inside an access map becomes the sum of the new ones.
  static std::vector<mlir::AffineForOp> split(mlir::AffineForOp forOp, uint64_t num_output, std::vector<int64_t>&& factors);

  // The one loop-carried value in `loops` becomes a register array indexed by
  // the listed loops that are nested inside the carrying loop's scope.
  static mlir::Value bufferizeLoopCarryVar(std::vector<mlir::AffineForOp>& loops);

  // Loop interchange to the given order (outermost first); imperfect nests are
  // handled by splitting the outer loop around the inner one.
  static void reorder(const std::vector<mlir::AffineForOp>& forOp);

  // Up to 3 perfectly nested loops -> one affine.parallel, normalised to
  // lower bound 0 / step 1.
  static mlir::AffineParallelOp parallel(const std::vector<mlir::AffineForOp>& forOp);

  template <typename ParentOpType>
  static mlir::Value alloc_buffer(ParentOpType father, MemorySpace ms, const std::vector<int64_t> shape_, mlir::Type dtype) {
    auto type = mlir::MemRefType::get(shape_, dtype, {}, static_cast<int>(ms));
    mlir::OpBuilder builder(father->getContext());
    builder.setInsertionPointToStart(father.getBody());
    return builder.create<mlir::memref::AllocOp>(builder.getUnknownLoc(), type).getResult();
  }

  template <typename ContextOp>
  static mlir::Value alloc_buffer(ContextOp contextOp, Position pos, MemorySpace ms, const std::vector<int64_t> shape_, mlir::Type dtype) {
    auto type = mlir::MemRefType::get(shape_, dtype, {}, static_cast<int>(ms));
    mlir::OpBuilder builder(contextOp->getContext());
    if (pos == Position::before) builder.setInsertionPoint(contextOp.getOperation());
    else if (pos == Position::after) builder.setInsertionPointAfter(contextOp.getOperation());
    else assert(false && "alloc_buffer: position must be before or after");
    return builder.create<mlir::memref::AllocOp>(builder.getUnknownLoc(), type).getResult();
  }

  // Copy loop memory -> register array `dst` (1-d), `width` elements per
  // iteration; the loop index is appended to `operands` as the last map input.
  static mlir::AffineForOp read(mlir::Value src, mlir::Value dst, mlir::AffineMap map, llvm::SmallVector<mlir::Value> operands,
                                int64_t width, mlir::AffineForOp compute_at, Position pos);
  static mlir::AffineForOp read(mlir::OpBuilder& builder, mlir::Value src, mlir::Value dst, mlir::AffineMap map,
                                llvm::SmallVector<mlir::Value> operands, int64_t width);

  // Copy loop register array `src` -> memory.  When the map has two more inputs
  // than `operands`, the copy is element-wise (outer index, index in vector).
  static mlir::AffineForOp write(mlir::Value src, mlir::Value dst, mlir::AffineMap map, llvm::SmallVector<mlir::Value> operands,
                                 int64_t width, mlir::AffineForOp compute_at, Position pos);
  static mlir::AffineForOp write(mlir::OpBuilder& builder, mlir::Value src, mlir::Value dst, mlir::AffineMap map,
                                 llvm::SmallVector<mlir::Value> operands, int64_t width);

  static mlir::gpu::BarrierOp barrier(mlir::AffineForOp compute_at, Position pos);

  // affine.load/store in the loop -> vector forms of `width`, loop step = width.
  static mlir::AffineForOp vectorize(mlir::AffineForOp readOrWrite, int64_t width);

  // Redirect loads (stores) of `src` inside `scope` to `cached` with a new access.
  static void cache_read(mlir::AffineForOp scope, mlir::Value src, mlir::Value cached, mlir::AffineMap map,
                         llvm::SmallVector<mlir::Value> operands);
  static void cache_write(mlir::AffineForOp scope, mlir::Value src, mlir::Value cached, mlir::AffineMap map,
                          llvm::SmallVector<mlir::Value> operands);

  // For every store to `dst` under the level: its enclosing loops, outermost first.
  static std::vector<std::vector<mlir::AffineForOp>> get_write(mlir::AffineParallelOp parallelLevel, mlir::Value dst);

  // Double-buffers `buffer` ([2] + shape) and software-pipelines the copy loops
  // `readBodys` over `compute_at`: a prologue copy for the first iteration in
  // front of the loop, the in-loop copies prefetch iteration i+1 under
  // `ub - 2*step - iv >= 0`, users of the buffer select half (iv / step) mod 2.
  // Returns {prologue copies, in-loop copies}; `buffer` is updated.
  static std::vector<std::vector<mlir::AffineForOp>> pipeline(std::vector<mlir::AffineForOp> readBodys, mlir::Value& buffer,
                                                              mlir::AffineForOp compute_at);

  // Flip the half selected by vector loads of `buffer` inside the scope.
  static void change_double_buffer(mlir::AffineForOp, mlir::Value buffer);

  // Peel the last iteration: the loop loses it, its body is copied after the
  // loop with the index replaced by a constant.
  static void detach_last_loop(mlir::AffineForOp forOp);

  static void schedule(mlir::Operation* srcOp, mlir::Operation* dstOp, Position pos);

  // Copy of `srcOp` in front of `forOp` with forOp's index fixed to `iteration`.
  static void extract_loop(mlir::Operation* srcOp, mlir::AffineForOp forOp, int64_t iteration);

  // Inline affine.if ops that hold over the whole range of their operands /
  // delete those that never hold.
  static void take_off_true_if(mlir::ModuleOp module);
  static void delete_false_if(mlir::ModuleOp module);

  // Full unrolling of the loops the predicate selects; tagging with affine.loop = "unroll".
  static void unroll(mlir::ModuleOp module, mlir::function_ref<bool(mlir::AffineForOp)> unrollCheckFn);
  static void unrollAttribute(mlir::ModuleOp module, mlir::function_ref<bool(mlir::AffineForOp)> unrollCheckFn);

  // Declared by the reference and never implemented there (Rewriter.cc:1615-1622).
  // Here: checks that the module can run on the host interpreter (IR/Interpreter.h).
  static void loweringAffineDialect(mlir::ModuleOp module);

  static void set_buffer(mlir::OpBuilder& builder, mlir::Value mem, mlir::Value targetValue);
  static mlir::AffineForOp create_constant_loop(mlir::OpBuilder& builder, int64_t lowerBound, int64_t upperBound, int64_t step);
  // tileC[i][j] += fragA[i] * fragB[j]; returns the outer loop.
  static mlir::AffineForOp outer_product(mlir::OpBuilder& builder, mlir::Value tileC, mlir::Value fragA, mlir::Value fragB,
                                         int64_t m, int64_t n);

  /*----------------------------------------------------------------*/

  // Collapse a perfect nest to a near-square 2-d nest / to one loop; indices are
  // recovered with floordiv / mod chains inside the access maps.
  static std::vector<mlir::AffineForOp> combineToTowDim(std::vector<mlir::AffineForOp> loops);
  static mlir::AffineForOp combineToOneDim(std::vector<mlir::AffineForOp> loops);

  // Element-wise copy loops (no vector width).
  static mlir::AffineForOp read(mlir::Value src, mlir::Value dst, mlir::AffineMap map, llvm::SmallVector<mlir::Value> operands,
                                mlir::AffineForOp compute_at, Position pos);
  static mlir::AffineForOp write(mlir::Value src, mlir::Value dst, mlir::AffineMap map, llvm::SmallVector<mlir::Value> operands,
                                 mlir::AffineForOp compute_at, Position pos);

  // Ragged 2-d tile: range = {rows, cols, tileRows, tileCols}; the loop nest is
  // cloned under four affine.if regions (interior, bottom edge, right edge, corner).
  static mlir::AffineIfOp irregularMat(mlir::AffineForOp forOp, std::vector<int> range, llvm::SmallVector<mlir::Value> operands);

  // iter_arg -> one-element shared buffer allocated at the start of buildBlock.
  static mlir::Value bufferizeLoopCarryVar(mlir::AffineForOp& loop, mlir::Block* buildBlock);

  static void swapLoops(std::vector<std::vector<mlir::AffineForOp>> loops);

  // Result of a scalar op -> stored to buffer[0], users load it back.
  static void bufferizeOpResult(mlir::Operation* resultOp, mlir::Value buffer);

  static void scheduleOpGridToBlock(mlir::AffineParallelOp gridLevel, mlir::AffineParallelOp blockLevel);
  static void deleteExtraCstOp(mlir::AffineParallelOp blockLevel);
  static mlir::AffineForOp modifyLoopStepToOne(mlir::AffineForOp forOp);
  static std::vector<mlir::Value> blockLevelOneToTwo(mlir::AffineParallelOp pal, int64_t oneDimLen);
};

}  // namespace KernelCodeGen
