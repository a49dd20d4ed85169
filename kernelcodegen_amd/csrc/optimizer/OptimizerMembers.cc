// Public helper members of the per-operator optimizers that a program written against the reference may
// call (reference: include/Optimizer/Optimizer.h:89-108 Binary, :159-164 LayerNorm, :191-192 Gather,
// :221-224 FMHA, :267 BatchMatmul).  The schedules in Optimizer.cc are scripted from the Rewriter primitives
// directly and do not go through these; each helper here is a self-contained rewrite or index map with the
// reference's signature and meaning, usable on any nest of the shape it describes.
#include <algorithm>
#include <cassert>
#include <set>

#include "Optimizer/Optimizer.h"

namespace KernelCodeGen {

using namespace mlir;

namespace {

AffineExpr dim(unsigned i) { return getAffineDimExpr(i); }

// Coordinates of position `flat` of a row-major tensor: extras = {rank, stride of dim 0, ..., stride of
// dim rank-2, extent of the last dim, ...}; appends coordinates first..rank-1 to `out`.
void delinearize(AffineExpr flat, const std::vector<int64_t>& extras, int64_t first, SmallVector<AffineExpr>& out) {
  const int64_t rank = extras[0];
  for (int64_t i = first; i < rank; ++i) {
    if (i == 0) out.push_back(flat.floorDiv(extras[1]));
    else if (i != rank - 1) out.push_back((flat % extras[i]).floorDiv(extras[i + 1]));
    else out.push_back(flat % extras[i + 1]);
  }
}

// New empty loop with the bounds and step of `like`, in front of it.
AffineForOp emptyLoopBefore(AffineForOp like) {
  OpBuilder b(like.getOperation());
  return b.create<AffineForOp>(b.getUnknownLoc(), like.getConstantLowerBound(), like.getConstantUpperBound(), like.getStep(),
                               ValueRange({}), [](OpBuilder& lb, Location loc, Value, ValueRange) {
                                 lb.create<AffineYieldOp>(loc, ValueRange({}));
                               });
}

void replaceOperandOf(Operation* op, Value from, Value to) {
  for (unsigned i = 0; i < op->getNumOperands(); ++i)
    if (op->getOperand(i) == from) op->setOperand(i, to);
}

// Operations of `block` in order, without the terminator.
std::vector<Operation*> bodyOps(Block* block) {
  std::vector<Operation*> ops;
  for (auto& op : block->getOperations())
    if (op.getKind() != OpKind::AffineYield) ops.push_back(&op);
  return ops;
}

}  // namespace

// ===========================================================================
// BinaryOptimizer
// ===========================================================================

// How the smaller operand's shape sits in the larger one's, dimensions aligned at the back:
// needDimNums counts the aligned dimensions that agree, oneDimNums those that do not (broadcast ones).
void BinaryOptimizer::getBinaryOpData(Value max_load, Value min_load, BinaryOpData& data) {
  data.oneDimNums = 0;
  data.needDimNums = 0;
  if (!min_load) {
    data.type = BinaryType::constant;
    return;
  }
  auto big = max_load.getType().cast<MemRefType>().getShape();
  auto small = min_load.getType().cast<MemRefType>().getShape();
  if (std::all_of(small.begin(), small.end(), [](int64_t d) { return d == 1; })) {
    data.type = BinaryType::allOne;
    return;
  }
  const size_t shift = big.size() - small.size();
  bool allAgree = true, seenAgree = false, ordered = true;
  for (size_t i = 0; i < small.size(); ++i) {
    if (small[i] == big[i + shift]) {
      seenAgree = true;
      ++data.needDimNums;
    } else {
      allAgree = false;
      if (seenAgree) ordered = false;      // a broadcast dimension behind one that is carried
      ++data.oneDimNums;
    }
  }
  if (allAgree) {
    data.type = shift == 0 ? BinaryType::allEqual : BinaryType::noOneOrder;
    if (shift == 0) data.oneDimNums = data.needDimNums = 0;
    return;
  }
  data.type = ordered ? BinaryType::hasOneOrder : BinaryType::hasOneUnorder;
}

// Index maps of the 2-d refold (y, x) of a binary nest.  Map inputs are
// (blockIdx.y, threadIdx.y, iv_y, blockIdx.x, threadIdx.x, iv_x), already scaled by their steps except the
// vector index iv_x, which counts vectors of four; `extras` describes the original tensor as `delinearize`
// takes it, with the extent of x appended.
//   "MaxLoadOrStore"   -> coordinates in the full-shape operand / the result;
//   "MinVectorLoad"    -> coordinates in the broadcast operand: its last `needDims` coordinates, behind
//                         `oneDimNums` leading coordinates that take the extra first input (a constant 0);
//   "CacheLoadOrStore" -> position in a per-thread register array.
AffineMap BinaryOptimizer::getAffineMap(const std::string& mapIdentifier, OpBuilder&, const std::vector<int64_t>& extras,
                                        const int needDims, const int oneDimNums) {
  const int64_t width = 4;
  if (mapIdentifier == "CacheLoadOrStore") return AffineMap::get(1, 0, dim(0));
  assert(!extras.empty());
  SmallVector<AffineExpr> exprs;
  if (mapIdentifier == "MaxLoadOrStore") {
    AffineExpr y = dim(0) + dim(1) + dim(2), x = dim(3) + dim(4) + dim(5) * width;
    if (extras[0] == 2) {
      exprs.push_back(y);
      exprs.push_back(x);
    } else {
      delinearize(y * extras.back() + x, extras, 0, exprs);
    }
    return AffineMap::get(6, 0, ArrayRef<AffineExpr>(exprs));
  }
  assert(mapIdentifier == "MinVectorLoad" && "BinaryOptimizer::getAffineMap: unknown map");
  if (extras[0] == 2) {
    if (oneDimNums) {        // a (1, X) operand: constant row, x from the last three inputs
      exprs.push_back(dim(0));
      exprs.push_back(dim(1) + dim(2) + dim(3) * width);
      return AffineMap::get(4, 0, ArrayRef<AffineExpr>(exprs));
    }
    exprs.push_back(dim(0) + dim(1) + dim(2) * width);
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>(exprs));
  }
  const unsigned base = oneDimNums ? 1 : 0;
  for (int i = 0; i < oneDimNums; ++i) exprs.push_back(dim(0));
  AffineExpr y = dim(base) + dim(base + 1) + dim(base + 2), x = dim(base + 3) + dim(base + 4) + dim(base + 5) * width;
  delinearize(y * extras.back() + x, extras, extras[0] - needDims, exprs);
  return AffineMap::get(6 + base, 0, ArrayRef<AffineExpr>(exprs));
}

// Map operands for the broadcast operand's load: a 2-d problem addresses it by the x part alone; `cst`
// (the constant 0 of broadcast dimensions) goes in front when given.
llvm::SmallVector<Value> BinaryOptimizer::getMinLoadOperands(int dim_, llvm::SmallVector<Value> operands, const Value cst) {
  llvm::SmallVector<Value> out;
  if (cst) out.push_back(cst);
  if (dim_ == 2) {
    assert(operands.size() >= 5);
    out.push_back(operands[3]);
    out.push_back(operands[4]);
  } else {
    for (Value v : operands) out.push_back(v);
  }
  return out;
}

// ===========================================================================
// LayerNormOptimizer
// ===========================================================================

// Several one-dimensional thread levels of equal extent that follow each other in one block become the
// first one: the bodies are appended in order with a barrier between them, and the operations that stood
// between two levels (scalar work on the results of the level before) move in as well, executed by thread 0
// under `affine.if (tid == 0)` and followed by a barrier.  Returns the merged level.
AffineParallelOp LayerNormOptimizer::combineParallel(std::vector<AffineParallelOp> pals) {
  assert(!pals.empty());
  AffineParallelOp first = pals[0];
  const auto extent = first.getConstantUpperBounds();
  Value tid = first.getIVs()[0];
  for (size_t p = 1; p < pals.size(); ++p) {
    AffineParallelOp pal = pals[p];
    assert(pal.getConstantUpperBounds() == extent && pal->getBlock() == first->getBlock());
    OpBuilder b = OpBuilder::atBlockTerminator(first.getBody());
    Location loc = b.getUnknownLoc();
    // what stands between the previous level and this one
    std::vector<Operation*> between;
    for (Operation* op = pals[p - 1]->getNextNode(); op && op != pal.getOperation(); op = op->getNextNode()) between.push_back(op);
    std::vector<Operation*> guarded;
    for (Operation* op : between) {
      const bool pure = op->getKind() == OpKind::Constant || op->getKind() == OpKind::Alloc;
      if (pure) op->moveBefore(first.getOperation());
      else guarded.push_back(op);
    }
    b.create<gpu::BarrierOp>(loc);
    if (!guarded.empty()) {
      auto zero = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(dim(0)), ArrayRef<bool>(true));
      auto ifOp = b.create<AffineIfOp>(loc, zero, ValueRange({tid}), false);
      for (Operation* op : guarded) op->moveBefore(ifOp.getBody()->getTerminator());
      b.create<gpu::BarrierOp>(loc);
    }
    pal.getIVs()[0].replaceAllUsesWith(tid);
    for (Operation* op : bodyOps(pal.getBody())) op->moveBefore(first.getBody()->getTerminator());
    pal.erase();
  }
  return first;
}

// buffers = {cache, source}.  The loads of `source` in the body of `forOp` are staged: a copy loop with
// forOp's bounds is created in front of it that moves source[...iv...] to cache[iv] (cache[tid + iv] for a
// two-input "PointLoadOrStore" access when forOp sits inside a thread level), vectorised by the configured
// width when the cache holds at least four elements, and the loads in forOp read the cache instead.
// Returns {copy loop, forOp}.
std::vector<AffineForOp> LayerNormOptimizer::read(AffineForOp forOp, std::vector<Value> buffers) {
  assert(buffers.size() >= 2);
  Value cache = buffers[0], source = buffers[1];
  std::vector<AffineLoadOp> targets;
  for (Operation* op : bodyOps(forOp.getBody()))
    if (auto load = dyn_cast<AffineLoadOp>(op))
      if (load.getMemRef() == source) targets.push_back(load);
  if (targets.empty()) return {forOp};
  AffineForOp copy = emptyLoopBefore(forOp);
  OpBuilder b = OpBuilder::atBlockBegin(copy.getBody());
  Location loc = b.getUnknownLoc();
  SmallVector<Value> from;
  for (Value v : targets[0].getMapOperands()) from.push_back(v == forOp.getInductionVar() ? copy.getInductionVar() : v);
  Value loaded = b.create<AffineLoadOp>(loc, source, targets[0].getAffineMap(), ValueRange(from)).getResult();
  b.create<AffineStoreOp>(loc, loaded, cache, ValueRange({copy.getInductionVar()}));
  for (auto load : targets) {
    OpBuilder lb(load.getOperation());
    Value staged = lb.create<AffineLoadOp>(loc, cache, ValueRange({forOp.getInductionVar()})).getResult();
    load.getResult().replaceAllUsesWith(staged);
    load.erase();
  }
  const int64_t width = layerNormConfig.count("VECTORIZE_WIDTH") ? layerNormConfig["VECTORIZE_WIDTH"] : 4;
  const int64_t trips = (copy.getConstantUpperBound() - copy.getConstantLowerBound()) / copy.getStep();
  if (cache.getType().cast<MemRefType>().getNumElements() >= 4 && width > 1 && copy.getStep() == 1 && trips % width == 0)
    copy = Rewriter::vectorize(copy, width);
  return {copy, forOp};
}

// Loop fission in front of a reduction: the loads of the listed buffers in `forOp` and the arithmetic that
// depends on nothing but them move into a new loop of the same bounds in front of forOp, which leaves the
// value they produce in buffers[0] (at the position the buffers[0] load reads); forOp reads that value back.
// Returns the new loop.
AffineForOp LayerNormOptimizer::extractOpsFromLoop(AffineForOp forOp, std::vector<Value> buffers) {
  assert(!buffers.empty());
  std::vector<AffineLoadOp> loads;
  AffineLoadOp home(nullptr);
  for (Operation* op : bodyOps(forOp.getBody()))
    if (auto load = dyn_cast<AffineLoadOp>(op))
      if (std::find(buffers.begin(), buffers.end(), load.getMemRef()) != buffers.end()) {
        loads.push_back(load);
        if (load.getMemRef() == buffers[0]) home = load;
      }
  assert(home && "extractOpsFromLoop: the loop does not read buffers[0]");
  // arithmetic whose operands all come from the chosen loads (transitively), in body order
  std::set<Operation*> moved;
  for (auto l : loads) moved.insert(l.getOperation());
  std::vector<Operation*> chain;
  for (Operation* op : bodyOps(forOp.getBody())) {
    if (moved.count(op) || isa<AffineStoreOp>(op) || isa<AffineLoadOp>(op) || op->getNumResults() != 1) continue;
    bool local = op->getNumOperands() > 0;
    for (Value v : op->getOperands()) {
      Operation* def = v.getDefiningOp();
      if (def && def->getBlock() == forOp.getBody() && !moved.count(def)) local = false;
      if (!def && v == forOp.getInductionVar()) local = false;
      if (v.isa<BlockArgument>() && v != forOp.getInductionVar() && v.cast<BlockArgument>().getOwner() == forOp.getBody()) local = false;
    }
    if (!local) continue;
    moved.insert(op);
    chain.push_back(op);
  }
  if (chain.empty()) return forOp;
  Operation* last = chain.back();
  AffineForOp front = emptyLoopBefore(forOp);
  // forOp reads the result back from buffers[0]
  OpBuilder rb(forOp->getContext());
  rb.setInsertionPointAfter(last);
  Value back = rb.create<AffineLoadOp>(rb.getUnknownLoc(), buffers[0], home.getAffineMap(), home.getMapOperands()).getResult();
  last->getResult(0).replaceAllUsesWith(back);
  for (auto l : loads) {
    l->moveBefore(front.getBody()->getTerminator());
    replaceOperandOf(l.getOperation(), forOp.getInductionVar(), front.getInductionVar());
  }
  for (Operation* op : chain) op->moveBefore(front.getBody()->getTerminator());
  OpBuilder sb = OpBuilder::atBlockTerminator(front.getBody());
  SmallVector<Value> at;
  for (Value v : home.getMapOperands()) at.push_back(v);
  sb.create<AffineStoreOp>(sb.getUnknownLoc(), last->getResult(0), buffers[0], home.getAffineMap(), ValueRange(at));
  return front;
}

// buffers = {cache, destination}.  The store of a cache value to `destination` inside `forOp` moves into a
// loop of its own (same bounds) in front of forOp.  Returns the new loop.
AffineForOp LayerNormOptimizer::write(AffineForOp forOp, std::vector<Value> buffers) {
  assert(buffers.size() >= 2);
  AffineLoadOp cached(nullptr);
  AffineStoreOp out(nullptr);
  for (Operation* op : bodyOps(forOp.getBody()))
    if (auto load = dyn_cast<AffineLoadOp>(op))
      if (load.getMemRef() == buffers[0])
        for (Operation* user : load.getResult().getUsers())
          if (auto st = dyn_cast<AffineStoreOp>(user))
            if (st.getMemRef() == buffers[1]) { cached = load; out = st; }
  if (!out) return forOp;
  AffineForOp front = emptyLoopBefore(forOp);
  OpBuilder b = OpBuilder::atBlockTerminator(front.getBody());
  SmallVector<Value> at;
  for (Value v : cached.getMapOperands()) at.push_back(v == forOp.getInductionVar() ? front.getInductionVar() : v);
  Value again = b.create<AffineLoadOp>(b.getUnknownLoc(), buffers[0], cached.getAffineMap(), ValueRange(at)).getResult();
  out->moveBefore(front.getBody()->getTerminator());
  replaceOperandOf(out.getOperation(), cached.getResult(), again);
  replaceOperandOf(out.getOperation(), forOp.getInductionVar(), front.getInductionVar());
  return front;
}

// `forOp` (trip count P) sums, per thread of the one-dimensional level `pal` (T threads), the elements
// buffer[tid + i * T] of a shared array and accumulates into a one-element result cell (the loop's two
// loads: the multi-index one names the array, the single-index one the cell).  It is replaced by a tree:
// the P strided elements of a thread are added in registers and stored to buffer[tid]; the array is halved
// with `if (tid < h)` steps and a barrier each while h is at least a 64-wide wavefront; the last 64 partials
// go through gpu.shuffle down (32 ... 1); thread 0 adds the total into the cell.  Bank-conflict free: lanes
// always touch consecutive words.  Returns the operations created, in order.
std::vector<Operation*> LayerNormOptimizer::reduceUnrollOptimize(AffineForOp forOp, AffineParallelOp pal) {
  Value array, cell;
  forOp->walk([&](Operation* op) {
    if (auto load = dyn_cast<AffineLoadOp>(op)) {
      if (load.getMemRefType().getNumElements() > 1) array = load.getMemRef();
      else cell = load.getMemRef();
    }
  }, WalkOrder::PreOrder);
  assert(array && cell && "reduceUnrollOptimize: the loop must read a partials array and a result cell");
  const int64_t wave = 64;
  Value tid = pal.getIVs()[0];
  const int64_t threads = pal.getConstantUpperBounds()[0];
  const int64_t perThread = (forOp.getConstantUpperBound() - forOp.getConstantLowerBound()) / forOp.getStep();
  assert(threads >= wave && (threads & (threads - 1)) == 0);
  Type element = array.getType().cast<MemRefType>().getElementType();
  std::vector<Operation*> created;
  OpBuilder b(forOp.getOperation());
  Location loc = b.getUnknownLoc();
  auto shifted = [&](int64_t by) { return AffineMap::get(1, 0, dim(0) + by); };
  // P strided elements of this thread
  Value sum;
  for (int64_t i = 0; i < perThread; ++i) {
    Value v = b.create<AffineLoadOp>(loc, array, shifted(i * threads), ValueRange({tid})).getResult();
    sum = i == 0 ? v : b.create<arith::AddFOp>(loc, sum, v).getResult();
  }
  created.push_back(b.create<AffineStoreOp>(loc, sum, array, ValueRange({tid})).getOperation());
  created.push_back(b.create<gpu::BarrierOp>(loc).getOperation());
  for (int64_t h = threads / 2; h >= wave; h /= 2) {
    auto below = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(h - 1 - dim(0)), ArrayRef<bool>(false));
    auto ifOp = b.create<AffineIfOp>(loc, below, ValueRange({tid}), false);
    OpBuilder ib = OpBuilder::atBlockTerminator(ifOp.getBody());
    Value x = ib.create<AffineLoadOp>(loc, array, ValueRange({tid})).getResult();
    Value y = ib.create<AffineLoadOp>(loc, array, shifted(h), ValueRange({tid})).getResult();
    ib.create<AffineStoreOp>(loc, ib.create<arith::AddFOp>(loc, x, y).getResult(), array, ValueRange({tid}));
    created.push_back(ifOp.getOperation());
    created.push_back(b.create<gpu::BarrierOp>(loc).getOperation());
  }
  // one wavefront left
  auto inWave = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(wave - 1 - dim(0)), ArrayRef<bool>(false));
  auto waveIf = b.create<AffineIfOp>(loc, inWave, ValueRange({tid}), false);
  created.push_back(waveIf.getOperation());
  {
    OpBuilder wb = OpBuilder::atBlockTerminator(waveIf.getBody());
    Value acc = wb.create<AffineLoadOp>(loc, array, ValueRange({tid})).getResult();
    for (int64_t off = wave / 2; off > 0; off /= 2) {
      auto sh = wb.create<gpu::ShuffleOp>(loc, acc, (int32_t)off, (int32_t)wave, gpu::ShuffleMode::DOWN);
      acc = wb.create<arith::AddFOp>(loc, sh.getShuffleResult(), acc).getResult();
    }
    auto isZero = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(dim(0)), ArrayRef<bool>(true));
    auto first = wb.create<AffineIfOp>(loc, isZero, ValueRange({tid}), false);
    OpBuilder fb = OpBuilder::atBlockTerminator(first.getBody());
    Value zero = fb.create<arith::ConstantIndexOp>(loc, 0).getResult();
    Value old = fb.create<AffineLoadOp>(loc, cell, ValueRange({zero})).getResult();
    fb.create<AffineStoreOp>(loc, fb.create<arith::AddFOp>(loc, old, acc).getResult(), cell, ValueRange({zero}));
  }
  created.push_back(b.create<gpu::BarrierOp>(loc).getOperation());
  (void)element;
  forOp.erase();
  return created;
}

// `forOp` (trip count P, step 1) applies an element-wise body to the elements of shared arrays that one
// thread of the level `pal` (T threads) owns.  It is unrolled so that iteration i of thread t works on
// element t + i * T: consecutive lanes touch consecutive words in every copy of the body.
void LayerNormOptimizer::elementWiseUnrollOptimize(AffineForOp forOp, AffineParallelOp pal) {
  Value tid = pal.getIVs()[0];
  const int64_t threads = pal.getConstantUpperBounds()[0];
  const int64_t lb = forOp.getConstantLowerBound(), ub = forOp.getConstantUpperBound(), step = forOp.getStep();
  OpBuilder b(forOp.getOperation());
  Location loc = b.getUnknownLoc();
  for (int64_t i = 0; lb + i * step < ub; ++i) {
    Value position = b.create<AffineApplyOp>(loc, AffineMap::get(1, 0, dim(0) + i * threads), ValueRange({tid})).getResult();
    BlockAndValueMapping mapping;
    mapping.map(forOp.getInductionVar(), position);
    for (Operation* op : bodyOps(forOp.getBody())) b.clone(*op, mapping);
  }
  forOp.erase();
}

// ===========================================================================
// GatherOptimizer
// ===========================================================================

// "VectorLoadOrStore": (blockIdx.y, threadIdx.y, iv_y, blockIdx.x, threadIdx.x, iv_x) of the 2-d refold ->
// coordinates in the result (`extras` as for BinaryOptimizer::getAffineMap); "PointLoadOrStore": identity on
// one input (a register cell or the index operand).
AffineMap GatherOptimizer::getAffineMap(const std::string& mapIdentifier, OpBuilder&, const std::vector<int64_t>& extras) {
  if (mapIdentifier == "PointLoadOrStore") return AffineMap::get(1, 0, dim(0));
  assert(mapIdentifier == "VectorLoadOrStore" && !extras.empty() && "GatherOptimizer::getAffineMap: unknown map");
  SmallVector<AffineExpr> exprs;
  AffineExpr y = dim(0) + dim(1) + dim(2), x = dim(3) + dim(4) + dim(5) * 4;
  delinearize(y * extras.back() + x, extras, 0, exprs);
  return AffineMap::get(6, 0, ArrayRef<AffineExpr>(exprs));
}

// A gather with a single index reads that index at a constant position in every iteration of `forOp`: the
// constant and the load move to the start of the level `pal`, where they are done once per thread.
void GatherOptimizer::oneIndexLoad(AffineForOp forOp, AffineParallelOp pal) {
  for (Operation* op : bodyOps(forOp.getBody())) {
    auto cst = dyn_cast<arith::ConstantIndexOp>(op);
    if (!cst) continue;
    auto users = cst.getResult().getUsers();
    if (users.empty()) continue;
    auto load = dyn_cast<AffineLoadOp>(users[0]);
    if (!load || load.getMapOperands().size() != 1) continue;
    Operation* front = &pal.getBody()->front();
    cst->moveBefore(front);
    load->moveAfter(cst.getOperation());
    return;
  }
}

// ===========================================================================
// FMHAOptimizer
// ===========================================================================

// Index maps of the fused attention schedule (reference: src/Optimizer/Optimizer.cc:2201-2437, the same 18 names).
//
// The tiled schedule is in force when the config carries the reference's keys (Slice, Width, BrTileS, BcTileS, BrTileO,
// HdTileO, WarpX_O, WARP_SIZE, BLOCK_SIZE) and the tile extents Hd, Br, Bc (applyOptimzer puts those in, as the
// reference's does).  A workgroup of BLOCK_SIZE threads owns Br queries; per key tile of Bc keys it forms the score tile
// S^T [Bc][Br] (a thread holds BcTileS x BrTileS of it), turns it into probabilities (softmaxIR), parks them in shared
// memory and adds P V to its O tile [Br][Hd] (a thread holds BrTileO x HdTileO).  Thread arrangement, "warp" being a
// run of WARP_SIZE consecutive threads (a layout unit only: nothing here depends on the hardware's wavefront width
// beyond Bc / BcTileS <= 64, the widest shuffle):
//   score tile:  warps stacked along the queries; inside one, LaneX_S = Bc / BcTileS lanes along the keys and
//                LaneY_S = WARP_SIZE / LaneX_S along the queries; a thread's BrTileS queries (BcTileS keys) are runs of
//                Width that repeat at a pitch of LaneY_S * Width (LaneX_S * Width);
//   output tile: warps as (warp / WarpX_O, warp % WarpX_O) over (queries, head dim); inside one, LaneX_O = Hd / HdTileO /
//                WarpX_O lanes along the head dim and LaneY_O = WARP_SIZE / LaneX_O along the queries, runs of Width as above.
// Inputs and results, name by name (tid = threadIdx.x, iv = the copy loop's index, as Rewriter::read / write append it):
//   loadTileQ  (b, h, blockIdx.x, tid, hd_outer, iv)      -> Q[b, h, query, d]      a Width-vector of the Q slice
//   loadTileK  (b, h, tid, kv, hd_outer, iv)              -> K[b, h, key, d]
//   storeTileQ (tid, iv, e)                               -> smQ[d in slice, query]   element e of that vector (transposed store)
//   storeTileK (tid, iv, e)                               -> smK[d in slice, key]
//   loadFragQ  (tid, hd_inner, iv)                        -> smQ[hd_inner, query]     Width queries of the thread's BrTileS
//   loadFragK  (tid, hd_inner, iv)                        -> smK[hd_inner, key]
//   brIdxS     (tid, br)                                  -> query in the workgroup's tile of score column br
//   bcIdxS     (tid, bc)                                  -> key in the key tile of score row bc  (not in the reference,
//                                                            which has no mask to apply)
//   readTileS  (bc, br)                                   -> tileS[bc, br]
//   storeTileP (tid, bc, br)                              -> smP[key, query]          br a multiple of Width
//   loadFactor (tid, iv) = brIdxO (tid, iv)               -> query of the thread's output rows iv * Width ...
//   loadTileV  (b, h, tid, kv, bc_outer, iv)              -> V[b, h, key, d]
//   storeTileV (tid, iv)                                  -> smV[key in slice, d]
//   loadFragP  (tid, bc_outer, bc_inner, iv)              -> smP[key, query]
//   loadFragV  (tid, bc_inner, iv)                        -> smV[bc_inner, d]
//   storeTileO (b, h, blockIdx.x, tid, br, hd)            -> O[b, h, query, d]        hd a multiple of Width
// The reference's "storeTileO" takes its thread id from input 0 (blockIdx.z) instead of input 3
// (src/Optimizer/Optimizer.cc:2415); input 3 it is here.
//
// Without those keys the row-per-thread form is in force (BLOCK_SIZE queries per workgroup, a thread owns whole rows):
//   "loadTileQ" / "storeTileO": (b, h, blockIdx.x, tid, row in thread) -> [b, h, query, 0]
//   "loadTileK" / "loadTileV":  (b, h, key) -> [b, h, key, 0];   "score": (tid, key in tile) -> position in the score row.
bool FMHAOptimizer::tiledConfig() {
  for (const char* key : {"Slice", "Width", "BrTileS", "BcTileS", "BrTileO", "HdTileO", "WarpX_O", "WARP_SIZE", "BLOCK_SIZE", "Hd", "Br", "Bc"})
    if (!fmhaConfig.count(key) || fmhaConfig[key] <= 0) return false;
  return true;
}

AffineMap FMHAOptimizer::getAffineMap(const std::string& mapIdentifier, OpBuilder&) {
  if (!tiledConfig()) {
    const int64_t block = fmhaConfig.count("BLOCK_SIZE") ? fmhaConfig["BLOCK_SIZE"] : 128;
    if (mapIdentifier == "loadTileQ" || mapIdentifier == "storeTileO")
      return AffineMap::get(5, 0, ArrayRef<AffineExpr>({dim(0), dim(1), dim(2) * block + dim(3) + dim(4), getAffineConstantExpr(0)}));
    if (mapIdentifier == "loadTileK" || mapIdentifier == "loadTileV")
      return AffineMap::get(3, 0, ArrayRef<AffineExpr>({dim(0), dim(1), dim(2), getAffineConstantExpr(0)}));
    assert(mapIdentifier == "score" && "FMHAOptimizer::getAffineMap: unknown map");
    return AffineMap::get(2, 0, ArrayRef<AffineExpr>({dim(1)}));
  }
  const int64_t BLOCK_SIZE = fmhaConfig["BLOCK_SIZE"], width = fmhaConfig["Width"], slice = fmhaConfig["Slice"];
  const int64_t warp = fmhaConfig["WARP_SIZE"], Hd = fmhaConfig["Hd"], Br = fmhaConfig["Br"], Bc = fmhaConfig["Bc"];
  const int64_t BrTileS = fmhaConfig["BrTileS"], BcTileS = fmhaConfig["BcTileS"], BrTileO = fmhaConfig["BrTileO"],
                HdTileO = fmhaConfig["HdTileO"], WarpX_O = fmhaConfig["WarpX_O"];
  const int64_t LaneX_S = Bc / BcTileS, LaneY_S = warp / LaneX_S;
  const int64_t LaneX_O = Hd / HdTileO / WarpX_O, LaneY_O = warp / LaneX_O;
  (void)BcTileS;
  // a copy of a ROWS x COLS tile by all threads, Width elements each: thread tid takes vector tid + iv * BLOCK_SIZE
  auto vectorOf = [&](AffineExpr tid, AffineExpr iv, int64_t cols, AffineExpr& row, AffineExpr& col) {
    AffineExpr v = tid + iv * BLOCK_SIZE;
    row = v.floorDiv(cols / width);
    col = (v % (cols / width)) * width;
  };
  auto warpOf = [&](AffineExpr tid) { return tid.floorDiv(warp); };
  auto laneOf = [&](AffineExpr tid) { return tid % warp; };
  // element i of a thread's run-structured tile extent: run i / Width at `pitch`, lane offset, element i % Width
  auto runs = [&](AffineExpr i, int64_t lanes, AffineExpr lane) {
    return i.floorDiv(width) * (lanes * width) + lane * width + i % width;
  };
  AffineExpr row, col;
  if (mapIdentifier == "loadTileQ") {
    vectorOf(dim(3), dim(5), slice, row, col);
    return AffineMap::get(6, 0, ArrayRef<AffineExpr>({dim(0), dim(1), dim(2) * Br + row, dim(4) + col}));
  }
  if (mapIdentifier == "loadTileK") {
    vectorOf(dim(2), dim(5), slice, row, col);
    return AffineMap::get(6, 0, ArrayRef<AffineExpr>({dim(0), dim(1), dim(3) + row, dim(4) + col}));
  }
  if (mapIdentifier == "storeTileQ" || mapIdentifier == "storeTileK") {
    vectorOf(dim(0), dim(1), slice, row, col);
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>({col + dim(2), row}));
  }
  if (mapIdentifier == "loadFragQ")
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>({dim(1), warpOf(dim(0)) * (LaneY_S * BrTileS) + dim(2) * (LaneY_S * width) +
                                                               laneOf(dim(0)).floorDiv(LaneX_S) * width}));
  if (mapIdentifier == "loadFragK")
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>({dim(1), dim(2) * (LaneX_S * width) + (laneOf(dim(0)) % LaneX_S) * width}));
  if (mapIdentifier == "brIdxS")
    return AffineMap::get(2, 0, ArrayRef<AffineExpr>({warpOf(dim(0)) * (LaneY_S * BrTileS) + runs(dim(1), LaneY_S, laneOf(dim(0)).floorDiv(LaneX_S))}));
  if (mapIdentifier == "bcIdxS")
    return AffineMap::get(2, 0, ArrayRef<AffineExpr>({runs(dim(1), LaneX_S, laneOf(dim(0)) % LaneX_S)}));
  if (mapIdentifier == "storeTileP")
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>({runs(dim(1), LaneX_S, laneOf(dim(0)) % LaneX_S),
                                                      warpOf(dim(0)) * (LaneY_S * BrTileS) + dim(2) * LaneY_S +
                                                          laneOf(dim(0)).floorDiv(LaneX_S) * width}));
  if (mapIdentifier == "readTileS") return AffineMap::get(2, 0, ArrayRef<AffineExpr>({dim(0), dim(1)}));
  AffineExpr xwarp_o = warpOf(dim(0)) % WarpX_O, ywarp_o = warpOf(dim(0)).floorDiv(WarpX_O);
  AffineExpr ylane_o = laneOf(dim(0)).floorDiv(LaneX_O), xlane_o = laneOf(dim(0)) % LaneX_O;
  if (mapIdentifier == "loadFactor" || mapIdentifier == "brIdxO")
    return AffineMap::get(2, 0, ArrayRef<AffineExpr>({ywarp_o * (LaneY_O * BrTileO) + dim(1) * (LaneY_O * width) + ylane_o * width}));
  if (mapIdentifier == "loadTileV") {
    vectorOf(dim(2), dim(5), Hd, row, col);
    return AffineMap::get(6, 0, ArrayRef<AffineExpr>({dim(0), dim(1), dim(3) + row + dim(4), col}));
  }
  if (mapIdentifier == "storeTileV") {
    vectorOf(dim(0), dim(1), Hd, row, col);
    return AffineMap::get(2, 0, ArrayRef<AffineExpr>({row, col}));
  }
  if (mapIdentifier == "loadFragP")
    return AffineMap::get(4, 0, ArrayRef<AffineExpr>({dim(1) + dim(2), ywarp_o * (LaneY_O * BrTileO) + dim(3) * (width * LaneY_O) + ylane_o * width}));
  if (mapIdentifier == "loadFragV")
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>({dim(1), xwarp_o * (LaneX_O * HdTileO) + dim(2) * (width * LaneX_O) + xlane_o * width}));
  assert(mapIdentifier == "storeTileO" && "FMHAOptimizer::getAffineMap: unknown map");
  {
    AffineExpr tid = dim(3);
    AffineExpr xw = warpOf(tid) % WarpX_O, yw = warpOf(tid).floorDiv(WarpX_O);
    AffineExpr yl = laneOf(tid).floorDiv(LaneX_O), xl = laneOf(tid) % LaneX_O;
    AffineExpr q = yw * (LaneY_O * BrTileO) + runs(dim(4), LaneY_O, yl);
    AffineExpr d = xw * (LaneX_O * HdTileO) + dim(5) * LaneX_O + xl * width;
    return AffineMap::get(6, 0, ArrayRef<AffineExpr>({dim(0), dim(1), dim(2) * Br + q, d}));
  }
}

// One online-softmax step over a score tile, emitted at the builder's position (reference:
// src/Optimizer/Optimizer.cc:2475-2604).  tileS is the thread's [BcTileS][BrTileS] piece (key, query) of the score
// tile; rowMax, rowSum [BrTileS] are registers; smMax, smSum, smFac [Br] the running maximum, the running sum and the
// factor by which the output accumulated so far has to be rescaled; `zero` and `flt_min` the constants 0 and the most
// negative finite value.  After the step tileS holds exp(s - new running max), smMax / smSum are updated and
// smFac = exp(old max - new max).
//
// Tiled form (tiledConfig()): a query's keys are spread over the LaneX_S = Bc / BcTileS threads `tid mod LaneX_S`, so
//   1. every thread reduces its own BcTileS keys per query to (max, sum of exp(s - max)), online;
//   2. the LaneX_S threads combine their pairs with gpu.shuffle down (offsets 1, 2, 4, ...; width LaneX_S);
//   3. the thread with tid mod LaneX_S == 0 folds the tile's pair into the running pair in shared memory and leaves the
//      rescale factor there;
//   4. the new running maximum goes back to all LaneX_S threads (gpu.shuffle idx 0) and tileS becomes exp(s - max).
// The reference's text has three slips that its own fixture shows (doc/pass.md:232, 318-322): step 1 stores the sum into
// rowMax and never updates rowSum (:2500-2501); step 3 rescales by exp(tile max - new max) where the old running
// maximum belongs (:2543-2544).  Neither is reproduced.
// Without the tiled keys a thread owns whole query rows (Br = BrTileS of them, all Bc = BcTileS keys): no shuffle,
// the statistics arrays are indexed by the row; `tid` is not used.
void FMHAOptimizer::softmaxIR(OpBuilder& builder, Value tileS, Value rowMax, Value smMax, Value rowSum, Value smSum, Value smFac,
                              Value zero, Value flt_min, Value tid) {
  const int64_t br = fmhaConfig.count("BrTileS") ? fmhaConfig["BrTileS"] : tileS.getType().cast<MemRefType>().getShape()[1];
  const int64_t bc = fmhaConfig.count("BcTileS") ? fmhaConfig["BcTileS"] : tileS.getType().cast<MemRefType>().getShape()[0];
  const bool tiled = tiledConfig();
  const int64_t lanes = tiled ? fmhaConfig["Bc"] / fmhaConfig["BcTileS"] : 1;
  Location loc = builder.getUnknownLoc();
  OpBuilder::InsertionGuard guard(builder);
  auto expOfDiff = [&](OpBuilder& b, Value x, Value y) {
    return b.create<math::ExpOp>(loc, b.create<arith::SubFOp>(loc, x, y).getResult()).getResult();
  };
  // 1. the thread's own keys: (max, sum) per query, online
  {
    AffineForOp rows = Rewriter::create_constant_loop(builder, 0, br, 1);
    Value r = rows.getInductionVar();
    OpBuilder rb = OpBuilder::atBlockBegin(rows.getBody());
    rb.create<AffineStoreOp>(loc, flt_min, rowMax, ValueRange({r}));
    rb.create<AffineStoreOp>(loc, zero, rowSum, ValueRange({r}));
    AffineForOp cols = Rewriter::create_constant_loop(rb, 0, bc, 1);
    OpBuilder cb = OpBuilder::atBlockBegin(cols.getBody());
    Value m = cb.create<AffineLoadOp>(loc, rowMax, ValueRange({r})).getResult();
    Value s = cb.create<AffineLoadOp>(loc, tileS, ValueRange({cols.getInductionVar(), r})).getResult();
    Value mNew = cb.create<arith::MaxFOp>(loc, m, s).getResult();
    Value l = cb.create<AffineLoadOp>(loc, rowSum, ValueRange({r})).getResult();
    Value kept = cb.create<arith::MulFOp>(loc, expOfDiff(cb, m, mNew), l).getResult();
    Value lNew = cb.create<arith::AddFOp>(loc, kept, expOfDiff(cb, s, mNew)).getResult();
    cb.create<AffineStoreOp>(loc, lNew, rowSum, ValueRange({r}));
    cb.create<AffineStoreOp>(loc, mNew, rowMax, ValueRange({r}));
    builder.setInsertionPointAfter(rows.getOperation());
  }
  // 2. the pairs of the threads that share a query
  if (lanes > 1) {
    AffineForOp rows = Rewriter::create_constant_loop(builder, 0, br, 1);
    Value r = rows.getInductionVar();
    OpBuilder rb = OpBuilder::atBlockBegin(rows.getBody());
    for (int64_t off = 1; off < lanes; off *= 2) {
      Value m1 = rb.create<AffineLoadOp>(loc, rowMax, ValueRange({r})).getResult();
      Value l1 = rb.create<AffineLoadOp>(loc, rowSum, ValueRange({r})).getResult();
      Value m2 = rb.create<gpu::ShuffleOp>(loc, m1, (int32_t)off, (int32_t)lanes, gpu::ShuffleMode::DOWN).getResult(0);
      Value l2 = rb.create<gpu::ShuffleOp>(loc, l1, (int32_t)off, (int32_t)lanes, gpu::ShuffleMode::DOWN).getResult(0);
      Value mNew = rb.create<arith::MaxFOp>(loc, m1, m2).getResult();
      Value a = rb.create<arith::MulFOp>(loc, l1, expOfDiff(rb, m1, mNew)).getResult();
      Value b = rb.create<arith::MulFOp>(loc, l2, expOfDiff(rb, m2, mNew)).getResult();
      rb.create<AffineStoreOp>(loc, rb.create<arith::AddFOp>(loc, a, b).getResult(), rowSum, ValueRange({r}));
      rb.create<AffineStoreOp>(loc, mNew, rowMax, ValueRange({r}));
    }
    builder.setInsertionPointAfter(rows.getOperation());
  }
  // 3. into the running pair; the first of the sharing threads does it
  {
    OpBuilder::InsertionGuard inner(builder);
    AffineMap rowOf = tiled ? getAffineMap("brIdxS", builder) : AffineMap::get(2, 0, ArrayRef<AffineExpr>({dim(1)}));
    if (lanes > 1) {
      auto first = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(dim(0) % lanes), ArrayRef<bool>(true));
      auto ifOp = builder.create<AffineIfOp>(loc, first, ValueRange({tid}), false);
      builder.setInsertionPoint(ifOp.getThenBlock()->getTerminator());
    }
    AffineForOp rows = Rewriter::create_constant_loop(builder, 0, br, 1);
    Value r = rows.getInductionVar();
    OpBuilder rb = OpBuilder::atBlockBegin(rows.getBody());
    Value oldMax = rb.create<AffineLoadOp>(loc, smMax, rowOf, ValueRange({tid, r})).getResult();
    Value oldSum = rb.create<AffineLoadOp>(loc, smSum, rowOf, ValueRange({tid, r})).getResult();
    Value tileMax = rb.create<AffineLoadOp>(loc, rowMax, ValueRange({r})).getResult();
    Value newMax = rb.create<arith::MaxFOp>(loc, oldMax, tileMax).getResult();
    Value factor = expOfDiff(rb, oldMax, newMax);
    rb.create<AffineStoreOp>(loc, newMax, smMax, rowOf, ValueRange({tid, r}));
    rb.create<AffineStoreOp>(loc, factor, smFac, rowOf, ValueRange({tid, r}));
    Value kept = rb.create<arith::MulFOp>(loc, oldSum, factor).getResult();
    Value tileSum = rb.create<AffineLoadOp>(loc, rowSum, ValueRange({r})).getResult();
    Value added = rb.create<arith::MulFOp>(loc, tileSum, expOfDiff(rb, tileMax, newMax)).getResult();
    rb.create<AffineStoreOp>(loc, rb.create<arith::AddFOp>(loc, kept, added).getResult(), smSum, rowOf, ValueRange({tid, r}));
    rb.create<AffineStoreOp>(loc, newMax, rowMax, ValueRange({r}));
  }
  // 4. the new running maximum to every sharing thread, then the probabilities
  if (lanes > 1) {
    AffineForOp rows = Rewriter::create_constant_loop(builder, 0, br, 1);
    Value r = rows.getInductionVar();
    OpBuilder rb = OpBuilder::atBlockBegin(rows.getBody());
    Value mine = rb.create<AffineLoadOp>(loc, rowMax, ValueRange({r})).getResult();
    Value firsts = rb.create<gpu::ShuffleOp>(loc, mine, (int32_t)0, (int32_t)lanes, gpu::ShuffleMode::IDX).getResult(0);
    rb.create<AffineStoreOp>(loc, firsts, rowMax, ValueRange({r}));
    builder.setInsertionPointAfter(rows.getOperation());
  }
  {
    AffineForOp outer = Rewriter::create_constant_loop(builder, 0, bc, 1);
    OpBuilder ob = OpBuilder::atBlockBegin(outer.getBody());
    AffineForOp inner = Rewriter::create_constant_loop(ob, 0, br, 1);
    OpBuilder ib = OpBuilder::atBlockBegin(inner.getBody());
    Value c = outer.getInductionVar(), r = inner.getInductionVar();
    Value s = ib.create<AffineLoadOp>(loc, tileS, ValueRange({c, r})).getResult();
    Value m = ib.create<AffineLoadOp>(loc, rowMax, ValueRange({r})).getResult();
    ib.create<AffineStoreOp>(loc, expOfDiff(ib, s, m), tileS, ValueRange({c, r}));
  }
}

// ===========================================================================
// BatchMatmulOptimizer
// ===========================================================================

// A one-dimensional thread level of BLOCK_SIZE_M/THREAD_SIZE_M x BLOCK_SIZE_N/THREAD_SIZE_N threads seen as
// (threadIdx.y, threadIdx.x): two affine.apply operations at the start of the level, tid floordiv X and
// tid mod X with X = BLOCK_SIZE_N / THREAD_SIZE_N.  The reference declares the member and never defines it
// (include/Optimizer/Optimizer.h:267).
std::vector<Value> BatchMatmulOptimizer::threadLevelOneToTwo(AffineParallelOp pal) {
  auto value = [&](const char* key, int dflt) { return batchMatmulConfig.count(key) ? batchMatmulConfig[key] : dflt; };
  int64_t x = value("BLOCK_SIZE_N", 128) / std::max(1, value("THREAD_SIZE_N", 8));
  const int64_t threads = pal.getConstantUpperBounds()[0];
  if (x <= 0 || threads % x) x = threads;
  return Rewriter::blockLevelOneToTwo(pal, x);
}

}  // namespace KernelCodeGen
