// Affine rewrite primitives (declared in include/Optimizer/Rewriter.h).
//
// Most primitives edit the accesses of an operation "that evaluates an affine
// map on a list of index operands": affine.load / store, their vector forms and
// affine.apply.  MapUser gives those five a common face so that each primitive
// is written once; accesses are edited in place.
#include "Optimizer/Rewriter.h"

#include <algorithm>
#include <cmath>
#include <map>
#include <set>

namespace KernelCodeGen {

using namespace mlir;

namespace {

struct MapUser {
  Operation* op = nullptr;
  unsigned first = 0;  // position of the first map operand

  static bool classify(Operation* o, MapUser& out) {
    switch (o->getKind()) {
      case OpKind::AffineLoad: case OpKind::AffineVectorLoad: out = {o, 1}; return true;
      case OpKind::AffineStore: case OpKind::AffineVectorStore: out = {o, 2}; return true;
      case OpKind::AffineApply: out = {o, 0}; return true;
      default: return false;
    }
  }
  bool isAccess() const { return first != 0; }
  Value memref() const { return op->getOperand(first - 1); }
  AffineMap map() const { return op->getAttr("map").map; }
  std::vector<Value> operands() const {
    return std::vector<Value>(op->getOperands().begin() + first, op->getOperands().end());
  }
  void set(AffineMap m, const std::vector<Value>& mapOperands) {
    assert(m.getNumInputs() == mapOperands.size());
    std::vector<Value> all(op->getOperands().begin(), op->getOperands().begin() + first);
    all.insert(all.end(), mapOperands.begin(), mapOperands.end());
    op->setOperands(all);
    op->setAttr("map", AffineMapAttr::get(m));
  }
  void setMemref(Value v) { op->setOperand(first - 1, v); }
};

// Every occurrence of `oldV` among the map operands is replaced by the values
// `newVs`; inside the map the old dimension becomes `expr`, an expression over
// d0..d(n-1) standing for newVs.
void substituteOperand(MapUser u, Value oldV, const std::vector<Value>& newVs, AffineExpr expr) {
  auto oldOperands = u.operands();
  AffineMap map = u.map();
  assert(map.getNumSymbols() == 0);
  std::vector<Value> operands;
  SmallVector<AffineExpr> dimRepl;
  bool found = false;
  for (Value v : oldOperands) {
    const unsigned base = (unsigned)operands.size();
    if (v == oldV) {
      found = true;
      SmallVector<AffineExpr> shifted;
      for (unsigned i = 0; i < newVs.size(); ++i) shifted.push_back(getAffineDimExpr(base + i));
      dimRepl.push_back(expr.replaceDims(shifted));
      operands.insert(operands.end(), newVs.begin(), newVs.end());
    } else {
      dimRepl.push_back(getAffineDimExpr(base));
      operands.push_back(v);
    }
  }
  if (!found) return;
  u.set(map.replaceDimsAndSymbols(dimRepl, {}, (unsigned)operands.size(), 0), operands);
}

// Applies `fn` to every map user nested in `root` (including root).
void forEachMapUser(Operation* root, const std::function<void(MapUser)>& fn) {
  root->walk([&](Operation* o) {
    MapUser u;
    if (MapUser::classify(o, u)) fn(u);
  }, WalkOrder::PreOrder);
}

// Replaces operand `from` by `to` in `root` and everything nested in it.
void replaceOperandsDeep(Operation* root, Value from, Value to) {
  root->walk([&](Operation* o) { o->replaceUsesOfWith(from, to); }, WalkOrder::PreOrder);
}

// The block of the closest enclosing function, module or affine.parallel.
Block* closestScopeBlock(Operation* op) {
  for (Operation* p = op->getParentOp(); p; p = p->getParentOp()) {
    if (isa<ModuleOp>(p)) return ModuleOp(p).getBody();
    if (isa<func::FuncOp>(p)) return &func::FuncOp(p).front();
    if (isa<AffineParallelOp>(p)) return AffineParallelOp(p).getBody();
  }
  assert(false && "operation is not inside a function");
  return nullptr;
}

// The outermost affine.for / affine.if ancestor chain of `op` below a function,
// module or affine.parallel.
Operation* rootLoopOf(Operation* op) {
  while (true) {
    Operation* parent = op->getParentOp();
    assert(parent && "operation is not inside a function");
    if (isa<ModuleOp>(parent) || isa<func::FuncOp>(parent) || isa<AffineParallelOp>(parent)) return op;
    op = parent;
  }
}

// An index constant placed at the start of the scope block that holds op's root loop.
Value hoistedIndexConstant(Operation* anchor, int64_t value) {
  Operation* root = rootLoopOf(anchor);
  OpBuilder b = OpBuilder::atBlockBegin(root->getBlock());
  return b.create<arith::ConstantIndexOp>(b.getUnknownLoc(), value).getResult();
}

void moveBodyWithoutYield(Block* from, Block* to, Operation* before) {
  Operation* op = from->empty() ? nullptr : &from->front();
  while (op) {
    Operation* next = op->getNextNode();
    if (op->getKind() == OpKind::AffineYield && next == nullptr) break;
    op->moveBefore(to, before);
    op = next;
  }
}

int64_t tripCount(AffineForOp loop) {
  return (loop.getConstantUpperBound() - loop.getConstantLowerBound() + loop.getStep() - 1) / loop.getStep();
}

}  // namespace

// ---------------------------------------------------------------------------
// split (reference: Rewriter.cc:114-243)
// ---------------------------------------------------------------------------
std::vector<AffineForOp> Rewriter::split(AffineForOp forOp, uint64_t num_output, std::vector<int64_t>&& factors) {
  assert(forOp.hasConstantBounds() && forOp.getStep() == 1 && forOp.getConstantLowerBound() == 0 &&
         "split needs a loop 0..ub step 1");
  assert(factors.size() + 1 == num_output && "split: factors.size() must be num_output - 1");
  assert(forOp.getNumIterOperands() == 0 && "split: bufferize the loop-carried value first");
  const int64_t ub = forOp.getConstantUpperBound();
  // factors are given innermost first: {8, 128} -> steps 128, 8, 1 and extents ub, 128, 8
  std::vector<int64_t> steps(factors.rbegin(), factors.rend()), ubs{ub};
  steps.push_back(1);
  for (auto it = factors.rbegin(); it != factors.rend(); ++it) ubs.push_back(*it);
  for (size_t i = 0; i + 1 < steps.size(); ++i)
    assert(steps[i] % steps[i + 1] == 0 && ubs[i] % steps[i] == 0 && "split: factors must divide each other and the extent");

  OpBuilder builder(forOp.getOperation());
  std::vector<AffineForOp> loops;
  std::vector<Value> ivs;
  {
    OpBuilder::InsertionGuard guard(builder);
    for (size_t i = 0; i < steps.size(); ++i) {
      auto loop = builder.create<AffineForOp>(builder.getUnknownLoc(), 0, ubs[i], steps[i]);
      loops.push_back(loop);
      ivs.push_back(loop.getInductionVar());
      builder.setInsertionPointToStart(loop.getBody());
    }
  }
  AffineForOp innermost = loops.back();
  moveBodyWithoutYield(forOp.getBody(), innermost.getBody(), innermost.getBody()->getTerminator());

  AffineExpr sum = getAffineDimExpr(0);
  for (unsigned i = 1; i < ivs.size(); ++i) sum = sum + getAffineDimExpr(i);
  Value oldIv = forOp.getInductionVar();
  // A user that takes the index as a plain value (a memref.load beside a loaded index, as Gather builds for an axis
  // other than the first; arithmetic on the index) gets the sum of the new indices through one affine.apply at the
  // start of the innermost body; users with an affine map get the sum inside their map, as in the reference.
  Value applied;
  auto userList = oldIv.getUsers();
  std::vector<Operation*> users(userList.begin(), userList.end());
  for (Operation* user : users) {
    MapUser u;
    if (MapUser::classify(user, u)) {
      substituteOperand(u, oldIv, ivs, sum);
      continue;
    }
    if (!applied) {
      OpBuilder ab = OpBuilder::atBlockBegin(innermost.getBody());
      applied = ab.create<AffineApplyOp>(ab.getUnknownLoc(), AffineMap::get((unsigned)ivs.size(), 0, sum), ValueRange(ivs)).getResult();
    }
    for (unsigned i = 0; i < user->getNumOperands(); ++i)
      if (user->getOperand(i) == oldIv) user->setOperand(i, applied);
  }
  forOp.erase();
  return loops;
}

// ---------------------------------------------------------------------------
// bufferizeLoopCarryVar (reference: Rewriter.cc:263-370)
// ---------------------------------------------------------------------------
Value Rewriter::bufferizeLoopCarryVar(std::vector<AffineForOp>& loops) {
  AffineForOp carry;
  int carryPos = -1;
  for (size_t i = 0; i < loops.size(); ++i)
    if (loops[i].getNumIterOperands() != 0) {
      if (carry) {
        llvm::errs() << "Can't reorder more than one loops carrying args\n";
        assert(false);
      }
      carry = loops[i];
      carryPos = (int)i;
    }
  if (!carry) return nullptr;
  assert(carry.getNumIterOperands() == 1 && "one loop-carried value is supported");

  // the buffer is indexed by the listed loops that enclose the carrying loop
  std::vector<int64_t> shape;
  std::vector<Value> address;
  for (auto loop : loops)
    if (loop != carry && loop->isProperAncestor(carry)) {
      shape.push_back(tripCount(loop));
      address.push_back(loop.getInductionVar());
      assert(loop.getStep() == 1 && loop.getConstantLowerBound() == 0);
    }
  if (shape.empty()) shape.push_back(1);

  Block* scope = closestScopeBlock(loops[0]);
  OpBuilder builder = OpBuilder::atBlockBegin(scope);
  Value carried = carry.getRegionIterArgs()[0];
  auto bufferType = MemRefType::get(shape, carried.getType(), {}, static_cast<int>(MemorySpace::local));
  Value buffer = builder.create<memref::AllocOp>(builder.getUnknownLoc(), bufferType).getResult();
  Value zeroIdx;
  if (address.empty()) {
    zeroIdx = builder.create<arith::ConstantIndexOp>(builder.getUnknownLoc(), 0).getResult();
    address.push_back(zeroIdx);
  }

  // 1. initialise the cell right after the initial value is defined
  Value init = carry.getIterOperands()[0];
  Operation* initDef = init.getDefiningOp();
  if (initDef) builder.setInsertionPointAfter(initDef);
  else builder.setInsertionPoint(carry.getOperation());
  builder.create<AffineStoreOp>(builder.getUnknownLoc(), init, buffer, ValueRange(address));

  // 2. a loop without iter_args: load the cell, run the old body, store the cell
  builder.setInsertionPointAfter(carry.getOperation());
  auto newLoop = builder.create<AffineForOp>(builder.getUnknownLoc(), carry.getConstantLowerBound(),
                                             carry.getConstantUpperBound(), carry.getStep());
  Operation* newYield = newLoop.getBody()->getTerminator();
  builder.setInsertionPoint(newYield);
  Value cell = builder.create<AffineLoadOp>(builder.getUnknownLoc(), buffer, ValueRange(address)).getResult();
  Operation* oldYield = carry.getBody()->getTerminator();
  Value yielded = oldYield->getOperand(0);
  moveBodyWithoutYield(carry.getBody(), newLoop.getBody(), newYield);
  carry.getInductionVar().replaceAllUsesWith(newLoop.getInductionVar());
  carried.replaceAllUsesWith(cell);
  if (yielded == carried) yielded = cell;
  builder.setInsertionPoint(newYield);
  builder.create<AffineStoreOp>(builder.getUnknownLoc(), yielded, buffer, ValueRange(address));

  // 3. users of the loop result read the cell
  builder.setInsertionPointAfter(newLoop.getOperation());
  Value result = builder.create<AffineLoadOp>(builder.getUnknownLoc(), buffer, ValueRange(address)).getResult();
  carry.getResult(0).replaceAllUsesWith(result);
  carry.erase();
  loops[carryPos] = newLoop;
  return buffer;
}

// ---------------------------------------------------------------------------
// reorder (reference: Rewriter.cc:374-559)
// ---------------------------------------------------------------------------
namespace {

// Interchange `outer` and its direct child `inner`.  Operations of outer's body
// before / after `inner` are peeled into their own copies of `outer`, which is
// legal for the nests the schedules build: an initialisation of a buffer in
// front of the loop and a write-back behind it, each indexed by outer's index.
void interchange(AffineForOp outer, AffineForOp inner) {
  assert(inner->getParentOp() == outer.getOperation());
  Block* body = outer.getBody();
  std::vector<Operation*> before, after;
  bool seen = false;
  for (auto& op : body->getOperations()) {
    if (&op == inner.getOperation()) { seen = true; continue; }
    if (op.getKind() == OpKind::AffineYield) continue;
    (seen ? after : before).push_back(&op);
  }
  auto peel = [&](const std::vector<Operation*>& ops, bool front) {
    if (ops.empty()) return;
    OpBuilder b(outer->getContext());
    if (front) b.setInsertionPoint(outer.getOperation()); else b.setInsertionPointAfter(outer.getOperation());
    auto copy = b.create<AffineForOp>(b.getUnknownLoc(), outer.getLowerBoundOperands(), outer.getLowerBoundMap(),
                                      outer.getUpperBoundOperands(), outer.getUpperBoundMap(), outer.getStep());
    for (auto& kv : outer->getAttrs())
      if (kv.first == "affine.loop") copy->setAttr(kv.first, kv.second);
    for (Operation* op : ops) op->moveBefore(copy.getBody(), copy.getBody()->getTerminator());
    // values defined by the peeled ops must not be used by what stays behind
    for (Operation* op : ops)
      for (Value r : op->getResults())
        for (Operation* user : r.getUsers())
          assert(copy->isAncestor(user) && "reorder: peeled operation feeds the inner loop");
    outer.getInductionVar().replaceUsesWithIf(copy.getInductionVar(),
                                              [&](Operation* user) { return copy->isAncestor(user); });
  };
  peel(before, true);
  peel(after, false);

  // outer { inner { B } }  ->  inner { outer { B } }
  inner->moveBefore(outer.getOperation());
  moveBodyWithoutYield(inner.getBody(), outer.getBody(), outer.getBody()->getTerminator());
  outer->moveBefore(inner.getBody(), inner.getBody()->getTerminator());
}

}  // namespace

void Rewriter::reorder(const std::vector<AffineForOp>& loops) {
  std::map<Operation*, int> priority;  // larger = further out
  int p = (int)loops.size();
  for (auto loop : loops) priority[loop.getOperation()] = p--;
  for (auto loop : loops) assert(loop.getNumIterOperands() == 0 && "reorder: bufferize loop-carried values first");

  auto targetChild = [&](AffineForOp parent) -> AffineForOp {
    for (auto& op : parent.getBody()->getOperations())
      if (isa<AffineForOp>(op) && priority.count(&op)) return AffineForOp(&op);
    return AffineForOp();
  };
  // the outermost listed loop in the nest that holds loops[0]
  auto findTop = [&]() -> AffineForOp {
    AffineForOp top;
    for (Operation* o = loops[0].getOperation(); o; o = o->getParentOp()) {
      if (isa<AffineParallelOp>(o) || isa<func::FuncOp>(o) || isa<ModuleOp>(o)) break;
      if (isa<AffineForOp>(o) && priority.count(o)) top = AffineForOp(o);
    }
    return top;
  };
  bool swapped;
  do {
    swapped = false;
    AffineForOp parent = findTop();
    while (AffineForOp child = targetChild(parent)) {
      if (priority[parent.getOperation()] < priority[child.getOperation()]) {
        interchange(parent, child);
        swapped = true;
        // `child` now encloses `parent`; keep pushing `parent` down
      } else {
        parent = child;
      }
    }
  } while (swapped);
}

void Rewriter::swapLoops(std::vector<std::vector<AffineForOp>> loops) {
  for (auto& pair : loops) {
    assert(pair.size() == 2);
    interchange(pair[0], pair[1]);
  }
}

// ---------------------------------------------------------------------------
// parallel (reference: Rewriter.cc:562-605)
// ---------------------------------------------------------------------------
AffineParallelOp Rewriter::parallel(const std::vector<AffineForOp>& forOps) {
  assert(!forOps.empty() && forOps.size() <= 3 && "at most three dimensions (z, y, x)");
  std::vector<int64_t> lbs, ubs, steps;
  for (size_t i = 0; i < forOps.size(); ++i) {
    auto loop = forOps[i];
    assert(loop.hasConstantBounds() && loop.getNumIterOperands() == 0);
    if (i > 0) assert(loop->getParentOp() == forOps[i - 1].getOperation() && "parallel: loops must be perfectly nested");
    if (i + 1 < forOps.size()) assert(loop.getBody()->getOperations().size() == 2 && "parallel: loops must be perfectly nested");
    lbs.push_back(loop.getConstantLowerBound());
    ubs.push_back(loop.getConstantUpperBound());
    steps.push_back(loop.getStep());
  }
  OpBuilder builder(forOps[0].getOperation());
  auto par = builder.create<AffineParallelOp>(builder.getUnknownLoc(), lbs, ubs, steps);
  AffineForOp innermost = forOps.back();
  moveBodyWithoutYield(innermost.getBody(), par.getBody(), par.getBody()->getTerminator());
  auto ivs = par.getIVs();
  for (size_t i = 0; i < forOps.size(); ++i) forOps[i].getInductionVar().replaceAllUsesWith(ivs[i]);
  AffineForOp(forOps[0]).erase();
  normalizeAffineParallel(par);
  return par;
}

// ---------------------------------------------------------------------------
// read / write / barrier / vectorize (reference: Rewriter.cc:608-810, 2021-2055)
// ---------------------------------------------------------------------------
AffineForOp Rewriter::read(OpBuilder& builder, Value src, Value dst, AffineMap map, SmallVector<Value> operands, int64_t width) {
  auto dstType = dst.getType().cast<MemRefType>();
  assert(dstType.getRank() == 1 && dstType.getShape()[0] % width == 0 && "read: destination is a 1-d register array");
  auto dstMap = AffineMap::get(1, 0, getAffineDimExpr(0) * width);
  auto vecType = VectorType::get(width, dstType.getElementType());
  return builder.create<AffineForOp>(builder.getUnknownLoc(), 0, dstType.getShape()[0] / width, 1, ValueRange({}),
    [&](OpBuilder& b, Location loc, Value iv, ValueRange) {
      SmallVector<Value> all = operands;
      all.push_back(iv);
      Value v = b.create<AffineVectorLoadOp>(loc, vecType, src, map, ValueRange(all)).getResult();
      b.create<AffineVectorStoreOp>(loc, v, dst, dstMap, ValueRange({iv}));
      b.create<AffineYieldOp>(loc);
    });
}

AffineForOp Rewriter::read(Value src, Value dst, AffineMap map, SmallVector<Value> operands, int64_t width,
                           AffineForOp compute_at, Position pos) {
  OpBuilder builder = getBuilder(compute_at, pos);
  return read(builder, src, dst, map, operands, width);
}

AffineForOp Rewriter::write(OpBuilder& builder, Value src, Value dst, AffineMap map, SmallVector<Value> operands, int64_t width) {
  auto srcType = src.getType().cast<MemRefType>();
  assert(srcType.getRank() == 1 && srcType.getShape()[0] % width == 0 && "write: source is a 1-d register array");
  const int64_t extra = (int64_t)map.getNumDims() - (int64_t)operands.size();
  assert((extra == 1 || extra == 2) && "write: map takes the operands plus one or two loop indices");
  const bool elementwise = extra == 2;
  return builder.create<AffineForOp>(builder.getUnknownLoc(), 0, srcType.getShape()[0] / width, 1, ValueRange({}),
    [&](OpBuilder& b, Location loc, Value iv, ValueRange) {
      SmallVector<Value> all = operands;
      all.push_back(iv);
      if (!elementwise) {
        auto vecType = VectorType::get(width, srcType.getElementType());
        auto srcMap = AffineMap::get(1, 0, getAffineDimExpr(0) * width);
        Value v = b.create<AffineVectorLoadOp>(loc, vecType, src, srcMap, ValueRange({iv})).getResult();
        b.create<AffineVectorStoreOp>(loc, v, dst, map, ValueRange(all));
      } else {
        auto vecType = VectorType::get(1, srcType.getElementType());
        auto srcMap = AffineMap::get(2, 0, getAffineDimExpr(0) * width + getAffineDimExpr(1));
        b.create<AffineForOp>(loc, 0, width, 1, ValueRange({}),
          [&](OpBuilder& ib, Location iloc, Value j, ValueRange) {
            SmallVector<Value> inner = all;
            inner.push_back(j);
            Value v = ib.create<AffineVectorLoadOp>(iloc, vecType, src, srcMap, ValueRange({iv, j})).getResult();
            ib.create<AffineVectorStoreOp>(iloc, v, dst, map, ValueRange(inner));
            ib.create<AffineYieldOp>(iloc);
          });
      }
      b.create<AffineYieldOp>(loc);
    });
}

AffineForOp Rewriter::write(Value src, Value dst, AffineMap map, SmallVector<Value> operands, int64_t width,
                            AffineForOp compute_at, Position pos) {
  OpBuilder builder = getBuilder(compute_at, pos);
  return write(builder, src, dst, map, operands, width);
}

AffineForOp Rewriter::read(Value src, Value dst, AffineMap map, SmallVector<Value> operands, AffineForOp compute_at, Position pos) {
  OpBuilder builder = getBuilder(compute_at, pos);
  auto dstType = dst.getType().cast<MemRefType>();
  assert(dstType.getRank() == 1);
  return builder.create<AffineForOp>(builder.getUnknownLoc(), 0, dstType.getShape()[0], 1, ValueRange({}),
    [&](OpBuilder& b, Location loc, Value iv, ValueRange) {
      SmallVector<Value> all = operands;
      all.push_back(iv);
      Value v = b.create<AffineLoadOp>(loc, src, map, ValueRange(all)).getResult();
      b.create<AffineStoreOp>(loc, v, dst, ValueRange({iv}));
      b.create<AffineYieldOp>(loc);
    });
}

AffineForOp Rewriter::write(Value src, Value dst, AffineMap map, SmallVector<Value> operands, AffineForOp compute_at, Position pos) {
  OpBuilder builder = getBuilder(compute_at, pos);
  auto srcType = src.getType().cast<MemRefType>();
  assert(srcType.getRank() == 1);
  return builder.create<AffineForOp>(builder.getUnknownLoc(), 0, srcType.getShape()[0], 1, ValueRange({}),
    [&](OpBuilder& b, Location loc, Value iv, ValueRange) {
      SmallVector<Value> all = operands;
      all.push_back(iv);
      Value v = b.create<AffineLoadOp>(loc, src, ValueRange({iv})).getResult();
      b.create<AffineStoreOp>(loc, v, dst, map, ValueRange(all));
      b.create<AffineYieldOp>(loc);
    });
}

gpu::BarrierOp Rewriter::barrier(AffineForOp compute_at, Position pos) {
  OpBuilder builder = getBuilder(compute_at, pos);
  return builder.create<gpu::BarrierOp>(builder.getUnknownLoc());
}

AffineForOp Rewriter::vectorize(AffineForOp loop, int64_t width) {
  assert(loop.getStep() == 1 && loop.getConstantLowerBound() == 0 && loop.getConstantUpperBound() % width == 0 &&
         "vectorize needs a loop 0..ub step 1 with ub divisible by the width");
  loop.setStep(width);
  std::vector<Operation*> scalarAccesses;
  loop->walk([&](Operation* o) {
    if (o->getKind() == OpKind::AffineLoad || o->getKind() == OpKind::AffineStore) scalarAccesses.push_back(o);
  }, WalkOrder::PreOrder);
  for (Operation* o : scalarAccesses) {
    OpBuilder b(o);
    if (o->getKind() == OpKind::AffineLoad) {
      AffineLoadOp load(o);
      auto vecType = VectorType::get(width, load.getMemRefType().getElementType());
      auto vload = b.create<AffineVectorLoadOp>(b.getUnknownLoc(), vecType, load.getMemRef(), load.getAffineMap(), load.getMapOperands());
      load.getResult().replaceAllUsesWith(vload.getResult());
    } else {
      AffineStoreOp store(o);
      b.create<AffineVectorStoreOp>(b.getUnknownLoc(), store.getValue(), store.getMemRef(), store.getAffineMap(), store.getMapOperands());
    }
    o->erase();
  }
  // elementwise operations between the vector loads and the vector stores (a fused epilogue)
  // now work on vectors: their results take the vector type, scalar operands broadcast
  loop->walk([&](Operation* o) {
    if (o->getNumResults() != 1 || o->getNumRegions() != 0) return;
    if (o->getKind() == OpKind::AffineVectorLoad || o->getKind() == OpKind::AffineApply) return;
    bool vectorOperand = false;
    for (auto v : o->getOperands()) vectorOperand |= v.getType().isa<VectorType>();
    Type rt = o->getResult(0).getType();
    if (vectorOperand && !rt.isa<VectorType>() && (rt.isFloat() || rt.isa<IntegerType>()))
      o->getResult(0).setType(VectorType::get(width, rt));
  }, WalkOrder::PreOrder);
  return loop;
}

// ---------------------------------------------------------------------------
// cache_read / cache_write / get_write (reference: Rewriter.cc:747-786)
// ---------------------------------------------------------------------------
void Rewriter::cache_read(AffineForOp scope, Value src, Value cached, AffineMap map, SmallVector<Value> operands) {
  scope->walk([&](Operation* o) {
    if (o->getKind() == OpKind::AffineLoad && AffineLoadOp(o).getMemRef() == src) AffineLoadOp(o).setAccess(cached, map, ValueRange(operands));
  }, WalkOrder::PreOrder);
}

void Rewriter::cache_write(AffineForOp scope, Value src, Value cached, AffineMap map, SmallVector<Value> operands) {
  scope->walk([&](Operation* o) {
    if (o->getKind() == OpKind::AffineStore && AffineStoreOp(o).getMemRef() == src) AffineStoreOp(o).setAccess(cached, map, ValueRange(operands));
  }, WalkOrder::PreOrder);
}

std::vector<std::vector<AffineForOp>> Rewriter::get_write(AffineParallelOp parallelLevel, Value dst) {
  std::vector<std::vector<AffineForOp>> results;
  parallelLevel->walk([&](Operation* o) {
    if (o->getKind() != OpKind::AffineStore || AffineStoreOp(o).getMemRef() != dst) return;
    std::vector<AffineForOp> nest;
    for (Operation* p = o->getParentOp(); p && isa<AffineForOp>(p); p = p->getParentOp()) nest.push_back(AffineForOp(p));
    std::reverse(nest.begin(), nest.end());
    results.push_back(nest);
  }, WalkOrder::PreOrder);
  return results;
}

// ---------------------------------------------------------------------------
// pipeline (reference: Rewriter.cc:812-1183)
// ---------------------------------------------------------------------------
namespace {

// Prepends a leading subscript to the accesses of `buffer` under `root`,
// switching them to `doubled`.  `select(dimOfIv)` builds that subscript from the
// map dimension bound to `iv` (appended to the operands when absent).
void retargetToDoubleBuffer(Operation* user, Value buffer, Value doubled, Value iv,
                            const std::function<AffineExpr(AffineExpr)>& select) {
  MapUser u;
  if (!MapUser::classify(user, u) || !u.isAccess() || u.memref() != buffer) return;
  auto operands = u.operands();
  AffineMap map = u.map();
  AffineExpr lead;
  if (!iv) {
    lead = getAffineConstantExpr(0);
  } else {
    unsigned dim = 0;
    bool found = false;
    for (; dim < operands.size(); ++dim)
      if (operands[dim] == iv) { found = true; break; }
    if (!found) operands.push_back(iv);
    lead = select(getAffineDimExpr(dim));
  }
  SmallVector<AffineExpr> exprs{lead};
  for (auto e : map.getResults()) exprs.push_back(e);
  u.setMemref(doubled);
  u.set(AffineMap::get((unsigned)operands.size(), 0, ArrayRef<AffineExpr>(exprs)), operands);
}

}  // namespace

std::vector<std::vector<AffineForOp>> Rewriter::pipeline(std::vector<AffineForOp> readBodys, Value& buffer, AffineForOp compute_at) {
  assert(compute_at.hasConstantBounds());
  auto bufferType = buffer.getType().cast<MemRefType>();
  auto allocOp = buffer.getDefiningOp<memref::AllocOp>();
  assert(allocOp && "pipeline: the buffer must come from memref.alloc");
  std::vector<int64_t> shape{2};
  for (auto d : bufferType.getShape()) shape.push_back(d);
  OpBuilder builder(allocOp.getOperation());
  Value doubled = builder.create<memref::AllocOp>(builder.getUnknownLoc(),
      MemRefType::get(shape, bufferType.getElementType(), {}, (int)bufferType.getMemorySpaceAsInt())).getResult();

  const int64_t step = compute_at.getStep(), lb = compute_at.getConstantLowerBound(), ub = compute_at.getConstantUpperBound();
  Value iv = compute_at.getInductionVar();

  // 1. prologue: copies of the read bodies in front of the loop, at iv = lb, filling half 0
  Value lbValue = hoistedIndexConstant(compute_at, lb);
  std::vector<AffineForOp> prologue;
  builder.setInsertionPoint(compute_at.getOperation());
  for (auto body : readBodys) {
    BlockAndValueMapping mapper;
    Operation* copy = builder.clone(*body.getOperation(), mapper);
    replaceOperandsDeep(copy, iv, lbValue);
    copy->walk([&](Operation* o) { retargetToDoubleBuffer(o, buffer, doubled, Value(), nullptr); }, WalkOrder::PreOrder);
    prologue.push_back(AffineForOp(copy));
  }

  // 2. in-loop prefetch of iteration i+1 under "iv + 2*step <= ub"
  AffineExpr d0 = getAffineDimExpr(0);
  auto guard = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(ub - 2 * step - d0), ArrayRef<bool>(false));
  builder.setInsertionPointToStart(compute_at.getBody());
  auto ifOp = builder.create<AffineIfOp>(builder.getUnknownLoc(), guard, ValueRange({iv}), false);
  for (auto body : readBodys) body->moveBefore(ifOp.getThenBlock(), ifOp.getThenBlock()->getTerminator());
  for (auto body : readBodys) {
    std::vector<Operation*> users;
    body->walk([&](Operation* o) { users.push_back(o); }, WalkOrder::PreOrder);
    for (Operation* o : users) {
      MapUser u;
      if (!MapUser::classify(o, u)) continue;
      // accesses of other memories advance to the next iteration: iv -> iv + step
      if (!(u.isAccess() && u.memref() == buffer)) substituteOperand(u, iv, {iv}, d0 + step);
      retargetToDoubleBuffer(o, buffer, doubled, iv, [&](AffineExpr d) { return (d.floorDiv(step) + 1) % 2; });
    }
  }

  // 3. every remaining user of the buffer reads the half of the current iteration
  for (Operation* user : buffer.getUsers()) {
    assert((user->getKind() == OpKind::AffineLoad || user->getKind() == OpKind::AffineVectorLoad) &&
           "pipeline: the buffer may only be read outside the copy loops");
    retargetToDoubleBuffer(user, buffer, doubled, iv, [&](AffineExpr d) { return d.floorDiv(step) % 2; });
  }
  allocOp.erase();
  buffer = doubled;
  return {prologue, readBodys};
}

void Rewriter::change_double_buffer(AffineForOp scope, Value buffer) {
  scope->walk([&](Operation* o) {
    if (o->getKind() != OpKind::AffineVectorLoad || AffineVectorLoadOp(o).getMemRef() != buffer) return;
    AffineVectorLoadOp load(o);
    AffineMap map = load.getAffineMap();
    SmallVector<AffineExpr> exprs(map.getResults());
    auto sel = exprs[0].dyn_cast<AffineBinaryOpExpr>();
    assert(sel && sel.getKind() == AffineExprKind::Mod && sel.getRHS() == 2 && "not a double-buffer access");
    exprs[0] = (sel.getLHS() + 1) % 2;
    load.setMap(AffineMap::get(map.getNumDims(), 0, ArrayRef<AffineExpr>(exprs)));
  }, WalkOrder::PostOrder);
}

// ---------------------------------------------------------------------------
// detach_last_loop / schedule / extract_loop (reference: Rewriter.cc:1185-1296)
// ---------------------------------------------------------------------------
void Rewriter::detach_last_loop(AffineForOp forOp) {
  assert(forOp.hasConstantBounds() && forOp.getNumIterOperands() == 0);
  const int64_t step = forOp.getStep(), ub = forOp.getConstantUpperBound();
  const int64_t last = forOp.getConstantLowerBound() + (tripCount(forOp) - 1) * step;
  (void)ub;
  forOp.setConstantUpperBound(last);
  Value lastIv = hoistedIndexConstant(forOp, last);
  OpBuilder builder = getBuilder(forOp, Position::after);
  BlockAndValueMapping mapper;
  AffineForOp copy(builder.clone(*forOp.getOperation(), mapper));
  replaceOperandsDeep(copy, copy.getInductionVar(), lastIv);
  moveBodyWithoutYield(copy.getBody(), copy->getBlock(), copy.getOperation());
  copy.erase();
}

void Rewriter::schedule(Operation* srcOp, Operation* dstOp, Position pos) {
  switch (pos) {
    case Position::after: srcOp->moveAfter(dstOp); break;
    case Position::before: srcOp->moveBefore(dstOp); break;
    case Position::end: {
      auto loop = dyn_cast<AffineForOp>(dstOp);
      assert(loop && "schedule(end) needs an affine.for destination");
      srcOp->moveBefore(loop.getBody()->getTerminator());
      break;
    }
    case Position::begin: {
      Block* body = nullptr;
      if (auto par = dyn_cast<AffineParallelOp>(dstOp)) body = par.getBody();
      else if (auto loop = dyn_cast<AffineForOp>(dstOp)) body = loop.getBody();
      assert(body && "schedule(begin) needs an affine.for or affine.parallel destination");
      srcOp->moveBefore(&body->front());
      break;
    }
  }
}

void Rewriter::extract_loop(Operation* srcOp, AffineForOp forOp, int64_t iteration) {
  assert(forOp.hasConstantBounds());
  OpBuilder builder(forOp.getOperation());
  BlockAndValueMapping mapper;
  Operation* copy = builder.clone(*srcOp, mapper);
  Value fixed = hoistedIndexConstant(forOp, forOp.getConstantLowerBound() + iteration * forOp.getStep());
  replaceOperandsDeep(copy, forOp.getInductionVar(), fixed);
}

// ---------------------------------------------------------------------------
// affine.if simplification (reference: Rewriter.cc:1298-1507)
// ---------------------------------------------------------------------------
namespace {

// Inclusive range of an index value, when it can be told from its definition.
bool valueRange(Value v, int64_t& lo, int64_t& hi) {
  if (auto arg = v.dyn_cast<BlockArgument>()) {
    Operation* owner = arg.getOwner()->getParentOp();
    if (auto loop = dyn_cast<AffineForOp>(owner)) {
      if (!loop.hasConstantBounds() || arg.getArgNumber() != 0) return false;
      lo = loop.getConstantLowerBound();
      hi = lo + (tripCount(loop) - 1) * loop.getStep();
      return tripCount(loop) > 0;
    }
    if (auto par = dyn_cast<AffineParallelOp>(owner)) {
      auto lbs = par.getConstantLowerBounds(), ubs = par.getConstantUpperBounds();
      auto steps = par.getSteps();
      const unsigned i = arg.getArgNumber();
      lo = lbs[i];
      hi = lbs[i] + ((ubs[i] - lbs[i] - 1) / steps[i]) * steps[i];
      return ubs[i] > lbs[i];
    }
    return false;
  }
  if (auto cst = v.getDefiningOp<arith::ConstantIndexOp>()) { lo = hi = cst.value(); return true; }
  return false;
}

// Range of an affine expression over a box of operand ranges (interval arithmetic).
bool exprRange(AffineExpr e, const std::vector<int64_t>& lo, const std::vector<int64_t>& hi, int64_t& outLo, int64_t& outHi) {
  switch (e.getKind()) {
    case AffineExprKind::Constant: outLo = outHi = e.cast<AffineConstantExpr>().getValue(); return true;
    case AffineExprKind::DimId: { unsigned p = e.cast<AffineDimExpr>().getPosition(); outLo = lo[p]; outHi = hi[p]; return true; }
    case AffineExprKind::SymbolId: return false;
    default: break;
  }
  auto b = e.cast<AffineBinaryOpExpr>();
  int64_t ll, lh, rl, rh;
  if (!exprRange(b.getLHS(), lo, hi, ll, lh) || !exprRange(b.getRHS(), lo, hi, rl, rh)) return false;
  auto fdiv = [](int64_t a, int64_t d) { int64_t q = a / d, r = a % d; return (r != 0 && ((r < 0) != (d < 0))) ? q - 1 : q; };
  switch (e.getKind()) {
    case AffineExprKind::Add: outLo = ll + rl; outHi = lh + rh; return true;
    case AffineExprKind::Mul: {
      int64_t c[4] = {ll * rl, ll * rh, lh * rl, lh * rh};
      outLo = *std::min_element(c, c + 4); outHi = *std::max_element(c, c + 4); return true;
    }
    case AffineExprKind::FloorDiv:
      if (rl != rh || rl <= 0) return false;
      outLo = fdiv(ll, rl); outHi = fdiv(lh, rl); return true;
    case AffineExprKind::CeilDiv:
      if (rl != rh || rl <= 0) return false;
      outLo = -fdiv(-ll, rl); outHi = -fdiv(-lh, rl); return true;
    case AffineExprKind::Mod:
      if (rl != rh || rl <= 0) return false;
      if (fdiv(ll, rl) == fdiv(lh, rl)) { outLo = ll - fdiv(ll, rl) * rl; outHi = lh - fdiv(lh, rl) * rl; }
      else { outLo = 0; outHi = rl - 1; }
      return true;
    default: return false;
  }
}

enum class Truth { Always, Never, Unknown };

Truth classifyIf(AffineIfOp ifOp) {
  std::vector<int64_t> lo, hi;
  for (Value v : ifOp.getOperands()) {
    int64_t l, h;
    if (!valueRange(v, l, h)) return Truth::Unknown;
    lo.push_back(l);
    hi.push_back(h);
  }
  IntegerSet set = ifOp.getIntegerSet();
  bool always = true;
  for (unsigned i = 0; i < set.getNumConstraints(); ++i) {
    int64_t l, h;
    if (!exprRange(set.getConstraint(i), lo, hi, l, h)) return Truth::Unknown;
    if (set.isEq(i)) {
      if (l > 0 || h < 0) return Truth::Never;
      if (!(l == 0 && h == 0)) always = false;
    } else {
      if (h < 0) return Truth::Never;
      if (l < 0) always = false;
    }
  }
  return always ? Truth::Always : Truth::Unknown;
}

}  // namespace

void Rewriter::take_off_true_if(ModuleOp module) {
  std::vector<AffineIfOp> ifs;
  module.walk<WalkOrder::PreOrder>([&](AffineIfOp ifOp) { ifs.push_back(ifOp); });
  for (auto ifOp : ifs) {
    if (classifyIf(ifOp) != Truth::Always) continue;
    moveBodyWithoutYield(ifOp.getThenBlock(), ifOp->getBlock(), ifOp.getOperation());
    ifOp.erase();
  }
}

void Rewriter::delete_false_if(ModuleOp module) {
  std::vector<AffineIfOp> ifs;
  module.walk<WalkOrder::PostOrder>([&](AffineIfOp ifOp) { ifs.push_back(ifOp); });
  for (auto ifOp : ifs) {
    if (classifyIf(ifOp) != Truth::Never) continue;
    if (ifOp.hasElse()) moveBodyWithoutYield(ifOp.getElseBlock(), ifOp->getBlock(), ifOp.getOperation());
    ifOp.erase();
  }
}

// ---------------------------------------------------------------------------
// unroll / unrollAttribute (reference: Rewriter.cc:1509-1613)
// ---------------------------------------------------------------------------
void Rewriter::unroll(ModuleOp module, function_ref<bool(AffineForOp)> unrollCheckFn) {
  std::vector<AffineForOp> loops;
  module.walk<WalkOrder::PostOrder>([&](AffineForOp loop) { loops.push_back(loop); });
  for (auto loop : loops) {
    if (!unrollCheckFn(loop) || !loop.hasConstantBounds() || loop.getNumIterOperands() != 0) continue;
    Operation* root = rootLoopOf(loop);
    Block* scope = root->getBlock();
    // reuse an index constant from the run of constants at the start of the scope block
    auto constantFor = [&](int64_t value) -> Value {
      for (auto& op : scope->getOperations()) {
        auto cst = dyn_cast<arith::ConstantIndexOp>(op);
        if (!cst) break;
        if (cst.value() == value) return cst.getResult();
      }
      OpBuilder b = OpBuilder::atBlockBegin(scope);
      return b.create<arith::ConstantIndexOp>(b.getUnknownLoc(), value).getResult();
    };
    OpBuilder builder(loop.getOperation());
    for (int64_t iv = loop.getConstantLowerBound(); iv < loop.getConstantUpperBound(); iv += loop.getStep()) {
      Value cst = constantFor(iv);
      BlockAndValueMapping mapper;
      AffineForOp copy(builder.clone(*loop.getOperation(), mapper));
      replaceOperandsDeep(copy, copy.getInductionVar(), cst);
      moveBodyWithoutYield(copy.getBody(), copy->getBlock(), copy.getOperation());
      copy.erase();
    }
    loop.erase();
  }
}

void Rewriter::unrollAttribute(ModuleOp module, function_ref<bool(AffineForOp)> unrollCheckFn) {
  module.walk<WalkOrder::PostOrder>([&](AffineForOp loop) {
    if (unrollCheckFn(loop)) loop->setAttr("affine.loop", StringAttr::get(nullptr, "unroll"));
  });
}

void Rewriter::loweringAffineDialect(ModuleOp module) {
  std::string message;
  if (failed(verify(module, &message))) llvm::errs() << "module can't be lowered for the host: " << message << "\n";
}

// ---------------------------------------------------------------------------
// small builders (reference: Rewriter.cc:1655-1702)
// ---------------------------------------------------------------------------
void Rewriter::set_buffer(OpBuilder& builder, Value mem, Value targetValue) {
  auto shape = mem.getType().cast<MemRefType>().getShape().vec();
  buildAffineLoopNest(builder, builder.getUnknownLoc(), std::vector<int64_t>(shape.size(), 0), shape,
                      std::vector<int64_t>(shape.size(), 1),
                      [&](OpBuilder& nb, Location loc, ValueRange ivs) { nb.create<AffineStoreOp>(loc, targetValue, mem, ivs); });
}

AffineForOp Rewriter::create_constant_loop(OpBuilder& builder, int64_t lowerBound, int64_t upperBound, int64_t step) {
  return builder.create<AffineForOp>(builder.getUnknownLoc(), lowerBound, upperBound, step);
}

AffineForOp Rewriter::outer_product(OpBuilder& builder, Value tileC, Value fragA, Value fragB, int64_t m, int64_t n) {
  OpBuilder::InsertionGuard guard(builder);
  auto outer = create_constant_loop(builder, 0, m, 1);
  builder.setInsertionPointToStart(outer.getBody());
  auto inner = create_constant_loop(builder, 0, n, 1);
  builder.setInsertionPointToStart(inner.getBody());
  Location loc = builder.getUnknownLoc();
  Value i = outer.getInductionVar(), j = inner.getInductionVar();
  Value a = builder.create<AffineLoadOp>(loc, fragA, ValueRange({i}));
  Value b = builder.create<AffineLoadOp>(loc, fragB, ValueRange({j}));
  Value c = builder.create<AffineLoadOp>(loc, tileC, ValueRange({i, j}));
  Value mul = builder.create<arith::MulFOp>(loc, a, b);
  Value add = builder.create<arith::AddFOp>(loc, mul, c);
  builder.create<AffineStoreOp>(loc, add, tileC, ValueRange({i, j}));
  return outer;
}

// ---------------------------------------------------------------------------
// nest collapsing (reference: Rewriter.cc:1894-2018, 2103-2193)
// ---------------------------------------------------------------------------
namespace {

// Replaces the perfect nest `loops` by the perfect nest of extents `newUbs`.
// The linear position in the old iteration space equals the linear position in
// the new one; old index i is recovered as (lin floordiv stride_i) mod extent_i.
std::vector<AffineForOp> collapseNest(std::vector<AffineForOp> loops, const std::vector<int64_t>& newUbs) {
  std::vector<int64_t> oldUbs;
  for (size_t i = 0; i < loops.size(); ++i) {
    assert(loops[i].hasConstantBounds() && loops[i].getConstantLowerBound() == 0 && loops[i].getStep() == 1);
    if (i > 0) assert(loops[i]->getParentOp() == loops[i - 1].getOperation() && "collapse: loops must be perfectly nested");
    oldUbs.push_back(loops[i].getConstantUpperBound());
  }
  AffineForOp outerOld = loops.front(), innerOld = loops.back();
  const bool carried = outerOld.getNumIterOperands() != 0;
  for (auto l : loops) assert((l.getNumIterOperands() != 0) == carried && "collapse: all loops or none carry a value");

  OpBuilder builder(outerOld.getOperation());
  std::vector<AffineForOp> fresh;
  std::vector<Value> ivs;
  Value carriedIn = carried ? outerOld.getIterOperands()[0] : Value();
  for (size_t i = 0; i < newUbs.size(); ++i) {
    AffineForOp loop;
    if (carried) {
      loop = builder.create<AffineForOp>(builder.getUnknownLoc(), 0, newUbs[i], 1, ValueRange({carriedIn}),
                                         [](OpBuilder&, Location, Value, ValueRange) {});
      carriedIn = loop.getRegionIterArgs()[0];
    } else {
      loop = builder.create<AffineForOp>(builder.getUnknownLoc(), 0, newUbs[i], 1);
    }
    if (!fresh.empty() && carried) {
      OpBuilder yb = OpBuilder::atBlockEnd(fresh.back().getBody());
      yb.create<AffineYieldOp>(yb.getUnknownLoc(), ValueRange({loop.getResult(0)}));
    }
    fresh.push_back(loop);
    ivs.push_back(loop.getInductionVar());
    if (carried) builder.setInsertionPointToStart(loop.getBody());
    else builder.setInsertionPoint(loop.getBody()->getTerminator());
  }
  AffineForOp innerNew = fresh.back();
  if (carried) {
    // the old innermost body comes with its own yield
    Operation* op = innerOld.getBody()->empty() ? nullptr : &innerOld.getBody()->front();
    while (op) { Operation* next = op->getNextNode(); op->moveBefore(innerNew.getBody(), nullptr); op = next; }
    innerOld.getRegionIterArgs()[0].replaceAllUsesWith(innerNew.getRegionIterArgs()[0]);
    outerOld.getResult(0).replaceAllUsesWith(fresh.front().getResult(0));
  } else {
    moveBodyWithoutYield(innerOld.getBody(), innerNew.getBody(), innerNew.getBody()->getTerminator());
  }

  // linear position over the new indices
  AffineExpr lin = getAffineDimExpr(0);
  for (unsigned i = 1; i < newUbs.size(); ++i) lin = lin * newUbs[i] + getAffineDimExpr(i);
  for (size_t i = 0; i < loops.size(); ++i) {
    int64_t stride = 1;
    for (size_t j = i + 1; j < loops.size(); ++j) stride *= oldUbs[j];
    AffineExpr e = lin.floorDiv(stride);
    if (i != 0) e = e % oldUbs[i];
    Value oldIv = loops[i].getInductionVar();
    for (Operation* user : oldIv.getUsers()) {
      MapUser u;
      if (MapUser::classify(user, u)) {
        substituteOperand(u, oldIv, ivs, e);
      } else {
        // a non-affine user (memref.load index): go through an affine.apply
        OpBuilder ub(user);
        Value applied = ub.create<AffineApplyOp>(ub.getUnknownLoc(), AffineMap::get((unsigned)ivs.size(), 0, e), ValueRange(ivs)).getResult();
        user->replaceUsesOfWith(oldIv, applied);
      }
    }
  }
  outerOld.erase();
  return fresh;
}

}  // namespace

std::vector<AffineForOp> Rewriter::combineToTowDim(std::vector<AffineForOp> loops) {
  int64_t total = 1;
  for (auto l : loops) total *= l.getConstantUpperBound();
  // the divisor of the total closest below its square root becomes the inner extent
  int64_t inner = 1;
  for (int64_t i = (int64_t)std::sqrt((double)total); i > 0; --i)
    if (total % i == 0) { inner = i; break; }
  const int64_t outer = total / inner;
  if (loops.size() == 2 && loops[0].getConstantUpperBound() == outer && loops[1].getConstantUpperBound() == inner) return loops;
  return collapseNest(loops, {outer, inner});
}

AffineForOp Rewriter::combineToOneDim(std::vector<AffineForOp> loops) {
  if (loops.size() == 1) return loops[0];
  int64_t total = 1;
  for (auto l : loops) total *= l.getConstantUpperBound();
  return collapseNest(loops, {total})[0];
}

// ---------------------------------------------------------------------------
// ragged tiles (reference: Rewriter.cc:2057-2101)
// ---------------------------------------------------------------------------
AffineIfOp Rewriter::irregularMat(AffineForOp forOp, std::vector<int> range, SmallVector<Value> operands) {
  assert(range.size() == 4 && operands.size() == 4 && "irregularMat: range = {rows, cols, tileRows, tileCols}, four operands");
  const int rows = range[0], cols = range[1], tr = range[2], tc = range[3];
  // start of the last, partial tile in each direction
  const int edgeY = rows / tr * tr, edgeX = cols / tc * tc;
  OpBuilder builder(forOp.getOperation());
  AffineExpr y = getAffineDimExpr(0) + getAffineDimExpr(2), x = getAffineDimExpr(1) + getAffineDimExpr(3);
  struct Case { SmallVector<AffineExpr> exprs; bool eq[2]; int ubY, ubX; };
  std::vector<Case> cases = {
      {{(rows - tr) - y, (cols - tc) - x}, {false, false}, tr, tc},        // interior: a whole tile fits
      {{y - edgeY, (cols - tc) - x}, {true, false}, rows - edgeY, tc},     // bottom edge
      {{(rows - tr) - y, x - edgeX}, {false, true}, tr, cols - edgeX},     // right edge
      {{y - edgeY, x - edgeX}, {true, true}, rows - edgeY, cols - edgeX},  // corner
  };
  AffineIfOp first;
  for (auto& c : cases) {
    if (c.ubY <= 0 || c.ubX <= 0) continue;
    auto set = IntegerSet::get(4, 0, ArrayRef<AffineExpr>(c.exprs), ArrayRef<bool>(c.eq, 2));
    auto ifOp = builder.create<AffineIfOp>(builder.getUnknownLoc(), set, ValueRange(operands), false);
    if (!first) first = ifOp;
    OpBuilder inner(ifOp.getThenBlock()->getTerminator());
    BlockAndValueMapping mapper;
    AffineForOp copy(inner.clone(*forOp.getOperation(), mapper));
    copy.setConstantUpperBound(c.ubY);
    auto son = dyn_cast<AffineForOp>(&copy.getBody()->front());
    assert(son && "irregularMat: expected a two-deep loop nest");
    son.setConstantUpperBound(c.ubX);
  }
  forOp.erase();
  return first;
}

// ---------------------------------------------------------------------------
// helpers of the LayerNorm schedule (reference: Rewriter.cc:2195-2456)
// ---------------------------------------------------------------------------
Value Rewriter::bufferizeLoopCarryVar(AffineForOp& loop, Block* buildBlock) {
  assert(loop.getNumIterOperands() == 1 && loop.hasConstantBounds());
  OpBuilder builder = OpBuilder::atBlockBegin(buildBlock);
  Value carried = loop.getRegionIterArgs()[0];
  Value buffer = builder.create<memref::AllocOp>(builder.getUnknownLoc(),
      MemRefType::get({1}, carried.getType(), {}, static_cast<int>(MemorySpace::shared))).getResult();
  Value zero = builder.create<arith::ConstantIndexOp>(builder.getUnknownLoc(), 0).getResult();
  Value init = loop.getIterOperands()[0];
  if (Operation* def = init.getDefiningOp()) {
    // the initial value must be visible where the cell is initialised
    if (def->getBlock() == loop->getBlock()) builder.setInsertionPointAfter(def);
    else builder.setInsertionPoint(loop.getOperation());
  } else {
    builder.setInsertionPoint(loop.getOperation());
  }
  builder.create<AffineStoreOp>(builder.getUnknownLoc(), init, buffer, ValueRange({zero}));

  builder.setInsertionPointAfter(loop.getOperation());
  auto newLoop = builder.create<AffineForOp>(builder.getUnknownLoc(), loop.getConstantLowerBound(), loop.getConstantUpperBound(), loop.getStep());
  Operation* newYield = newLoop.getBody()->getTerminator();
  builder.setInsertionPoint(newYield);
  Value cell = builder.create<AffineLoadOp>(builder.getUnknownLoc(), buffer, ValueRange({zero})).getResult();
  Value yielded = loop.getBody()->getTerminator()->getOperand(0);
  moveBodyWithoutYield(loop.getBody(), newLoop.getBody(), newYield);
  loop.getInductionVar().replaceAllUsesWith(newLoop.getInductionVar());
  carried.replaceAllUsesWith(cell);
  if (yielded == carried) yielded = cell;
  builder.setInsertionPoint(newYield);
  builder.create<AffineStoreOp>(builder.getUnknownLoc(), yielded, buffer, ValueRange({zero}));
  builder.setInsertionPointAfter(newLoop.getOperation());
  Value result = builder.create<AffineLoadOp>(builder.getUnknownLoc(), buffer, ValueRange({zero})).getResult();
  loop.getResult(0).replaceAllUsesWith(result);
  loop.erase();
  loop = newLoop;
  return buffer;
}

void Rewriter::bufferizeOpResult(Operation* resultOp, Value buffer) {
  assert(resultOp->getNumResults() == 1);
  Block* scope = closestScopeBlock(resultOp);
  Value zero;
  for (auto& op : scope->getOperations())
    if (auto cst = dyn_cast<arith::ConstantIndexOp>(op))
      if (cst.value() == 0 && (cst->getBlock() != resultOp->getBlock() || cst->isBeforeInBlock(resultOp))) { zero = cst.getResult(); break; }
  if (!zero) {
    OpBuilder b = OpBuilder::atBlockBegin(scope);
    zero = b.create<arith::ConstantIndexOp>(b.getUnknownLoc(), 0).getResult();
  }
  Value result = resultOp->getResult(0);
  for (Operation* user : result.getUsers()) {
    OpBuilder b(user);
    Value loaded = b.create<AffineLoadOp>(b.getUnknownLoc(), buffer, ValueRange({zero})).getResult();
    user->replaceUsesOfWith(result, loaded);
  }
  OpBuilder b(resultOp->getContext());
  b.setInsertionPointAfter(resultOp);
  b.create<AffineStoreOp>(b.getUnknownLoc(), result, buffer, ValueRange({zero}));
}

void Rewriter::scheduleOpGridToBlock(AffineParallelOp gridLevel, AffineParallelOp blockLevel) {
  std::vector<Operation*> constants;
  for (auto& op : gridLevel.getBody()->getOperations())
    if (op.getKind() == OpKind::Constant) constants.push_back(&op);
  Operation* firstInBlock = &blockLevel.getBody()->front();
  for (Operation* op : constants) {
    if (isa<AffineApplyOp>(firstInBlock)) op->moveAfter(firstInBlock);
    else op->moveBefore(&blockLevel.getBody()->front());
  }
}

void Rewriter::deleteExtraCstOp(AffineParallelOp blockLevel) {
  std::vector<Operation*> constants;
  blockLevel->walk([&](Operation* o) { if (o->getKind() == OpKind::Constant) constants.push_back(o); }, WalkOrder::PreOrder);
  std::vector<std::pair<Operation*, Value>> unique;  // representative constant -> hoisted value
  OpBuilder builder = OpBuilder::atBlockBegin(blockLevel.getBody());
  for (Operation* c : constants) {
    Value replacement;
    for (auto& kv : unique)
      if (kv.first->getAttr("value") == c->getAttr("value") && kv.first->getResult(0).getType() == c->getResult(0).getType())
        replacement = kv.second;
    if (!replacement) {
      replacement = builder.create<arith::ConstantOp>(builder.getUnknownLoc(), c->getResult(0).getType(), c->getAttr("value")).getResult();
      unique.emplace_back(c, replacement);
    }
    c->getResult(0).replaceAllUsesWith(replacement);
  }
  for (Operation* c : constants) c->erase();
}

AffineForOp Rewriter::modifyLoopStepToOne(AffineForOp forOp) {
  assert(forOp.hasConstantBounds() && forOp.getNumIterOperands() == 0);
  const int64_t step = forOp.getStep(), lb = forOp.getConstantLowerBound(), ub = forOp.getConstantUpperBound();
  assert(lb % step == 0 && ub % step == 0 && "modifyLoopStepToOne: bounds must be multiples of the step");
  OpBuilder builder(forOp.getOperation());
  auto newLoop = builder.create<AffineForOp>(builder.getUnknownLoc(), lb / step, ub / step, 1);
  moveBodyWithoutYield(forOp.getBody(), newLoop.getBody(), newLoop.getBody()->getTerminator());
  Value oldIv = forOp.getInductionVar();
  for (Operation* user : oldIv.getUsers()) {
    MapUser u;
    if (!MapUser::classify(user, u)) { user->emitError("modifyLoopStepToOne: index used outside an affine map"); assert(false); }
    substituteOperand(u, oldIv, {newLoop.getInductionVar()}, getAffineDimExpr(0) * step);
  }
  forOp.erase();
  return newLoop;
}

std::vector<Value> Rewriter::blockLevelOneToTwo(AffineParallelOp pal, int64_t oneDimLen) {
  OpBuilder builder = OpBuilder::atBlockBegin(pal.getBody());
  Value tid = getParallelIdx(pal)[0];
  AffineExpr d0 = getAffineDimExpr(0);
  Value y = builder.create<AffineApplyOp>(builder.getUnknownLoc(), AffineMap::get(1, 0, d0.floorDiv(oneDimLen)), ValueRange({tid})).getResult();
  Value x = builder.create<AffineApplyOp>(builder.getUnknownLoc(), AffineMap::get(1, 0, d0 % oneDimLen), ValueRange({tid})).getResult();
  return {y, x};
}

}  // namespace KernelCodeGen
