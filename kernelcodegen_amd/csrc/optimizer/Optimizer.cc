// Operator schedules (declared in include/Optimizer/Optimizer.h).
//
// GEMM and batched GEMM share one schedule, gemmSchedule(): the reference has
// two near-identical copies of it (src/Optimizer/Optimizer.cc:406-570 and
// :3290-3445); here the batch indices are a prefix of every access map.
#include "Optimizer/Optimizer.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <sstream>

#include "log.h"

#define DUMP(module)                                  \
  {                                                   \
    if (KCGLog::level == Log::Debug) (module).dump(); \
  }

namespace KernelCodeGen {

using namespace mlir;

std::map<std::string, int> MatmulOptimizer::matmulConfig;
std::map<std::string, int> FMHAOptimizer::fmhaConfig;
std::map<std::string, int> BinaryOptimizer::binaryConfig;
std::map<std::string, int> ElementWiseOptimizer::elementWiseConfig;
std::map<std::string, int> LayerNormOptimizer::layerNormConfig;
std::map<std::string, int> GatherOptimizer::gatherConfig;
std::map<std::string, int> SoftmaxOptimizer::softmaxConfig;
std::map<std::string, int> BatchMatmulOptimizer::batchMatmulConfig;

namespace {

int cfg(const std::map<std::string, int>& m, const std::string& key, int dflt = 0) {
  auto it = m.find(key);
  return it == m.end() ? dflt : it->second;
}

// A config entry may be restricted to one operand width with DTYPE_BITS.
bool configMatchesType(const std::map<std::string, int>& m, Type element) {
  const int bits = cfg(m, "DTYPE_BITS", 0);
  return bits == 0 || bits == (int)element.getIntOrFloatBitWidth();
}

// Records the schedule's parameters on the function so that the backend does
// not have to re-derive them from loop bounds.
void tagFunction(func::FuncOp f, const std::string& op, const std::map<std::string, int>& config, OpBuilder& builder) {
  f->setAttr("func.state", builder.getStringAttr("gpu"));
  f->setAttr("kcg.op", builder.getStringAttr(op));
  for (auto& kv : config) f->setAttr("kcg.cfg." + kv.first, builder.getI64IntegerAttr(kv.second));
}

// ---------------------------------------------------------------------------
// Thread arrangement inside a workgroup of blockDimY x blockDimX threads:
// a wavefront is threadOrg = {ty, tx} threads, the workgroup warpOrg = {wy, wx}
// wavefronts, with ty*wy = blockDimY and tx*wx = blockDimX.  The reference
// hard-codes 8x4 lanes in 2x4 warps for 32-wide warps (Optimizer.cc:306-307);
// 64-wide wavefronts get 8x8 lanes.
// ---------------------------------------------------------------------------
struct ThreadLayout {
  int64_t ty, tx, wy, wx;
  bool ok;
};
ThreadLayout threadLayout(int64_t blockDimY, int64_t blockDimX, int64_t warpSize) {
  ThreadLayout l{};
  l.tx = warpSize >= 64 ? 8 : 4;
  l.ty = warpSize / l.tx;
  l.ok = l.ty > 0 && blockDimY % l.ty == 0 && blockDimX % l.tx == 0;
  if (l.ok) { l.wy = blockDimY / l.ty; l.wx = blockDimX / l.tx; }
  return l;
}

struct GemmMaps {
  const std::map<std::string, int>& c;
  unsigned nb;  // number of batch loop indices among the operands of every global access (0 or 1)
  bool tA = false, tB = false;       // operand stored column-major: A as [k, m], B as [n, k]
  std::vector<int64_t> batchShape;   // leading dims of the memrefs; several are addressed through one collapsed index
  int64_t BM, BN, BK, TM, TN, W, bdy, bdx;
  ThreadLayout L;

  GemmMaps(const std::map<std::string, int>& config, unsigned numBatch, bool transA = false, bool transB = false,
           std::vector<int64_t> batchDims = {})
      : c(config), nb(numBatch), tA(transA), tB(transB), batchShape(std::move(batchDims)) {
    BM = cfg(c, "BLOCK_SIZE_M"); BN = cfg(c, "BLOCK_SIZE_N"); BK = cfg(c, "BLOCK_SIZE_K");
    TM = cfg(c, "THREAD_SIZE_M"); TN = cfg(c, "THREAD_SIZE_N");
    W = cfg(c, "VECTORIZE_WIDTH", 1);
    bdy = BM / TM; bdx = BN / TN;
    L = threadLayout(bdy, bdx, cfg(c, "WARP_SIZE", 64));
  }

  AffineExpr d(unsigned i) const { return getAffineDimExpr(i); }

  // Global accesses carry the batch indices first: operands [b.., ...rest].
  // With several batch dims the one collapsed loop index b addresses them as (b floordiv .., .. mod ..).
  AffineMap withBatch(unsigned restDims, std::vector<AffineExpr> exprs) const {
    std::vector<AffineExpr> all;
    if (nb == 1 && batchShape.size() > 1) {
      int64_t inner = 1;
      std::vector<AffineExpr> idx(batchShape.size());
      for (size_t j = batchShape.size(); j-- > 0;) {
        idx[j] = j == 0 ? d(0).floorDiv(inner) : d(0).floorDiv(inner) % batchShape[j];
        inner *= batchShape[j];
      }
      all = idx;
    } else {
      for (unsigned i = 0; i < nb; ++i) all.push_back(d(i));
    }
    all.insert(all.end(), exprs.begin(), exprs.end());
    return AffineMap::get(nb + restDims, 0, ArrayRef<AffineExpr>(all));
  }

  // A tile copy moves vectors of W elements along the operand's contiguous axis.  Copying along
  // k means the LDS store is transposed (element by element, smA/smB are [k][m|n]); copying along
  // m|n stores the vector as it is.
  // operands: [b.., ty, tx, blockIdx.m, k_outer, iv] -> A[b.., m, k]  (or A[b.., k, m])
  AffineMap loadTileA() const {
    AffineExpr vt = d(nb) * bdx + d(nb + 1) + d(nb + 4) * (bdy * bdx);  // virtual thread id of copy iteration iv
    if (tA) {
      AffineExpr k = vt.floorDiv(BM / W) + d(nb + 3);
      AffineExpr m = (vt % (BM / W)) * W + d(nb + 2) * BM;
      return withBatch(5, {k, m});
    }
    AffineExpr m = vt.floorDiv(BK / W) + d(nb + 2) * BM;
    AffineExpr k = (vt % (BK / W)) * W + d(nb + 3);
    return withBatch(5, {m, k});
  }
  // operands: [b.., ty, tx, k_outer, blockIdx.n, iv] -> B[b.., k, n]  (or B[b.., n, k])
  AffineMap loadTileB() const {
    AffineExpr vt = d(nb) * bdx + d(nb + 1) + d(nb + 4) * (bdy * bdx);
    if (tB) {
      AffineExpr n = vt.floorDiv(BK / W) + d(nb + 3) * BN;
      AffineExpr k = (vt % (BK / W)) * W + d(nb + 2);
      return withBatch(5, {n, k});
    }
    AffineExpr k = vt.floorDiv(BN / W) + d(nb + 2);
    AffineExpr n = (vt % (BN / W)) * W + d(nb + 3) * BN;
    return withBatch(5, {k, n});
  }
  // transposed form, operands: [ty, tx, iv, ivInVector] -> sm[k, m|n]; straight form, operands: [ty, tx, iv]
  AffineMap storeTile(bool alongK, int64_t extent) const {
    AffineExpr vt = d(0) * bdx + d(1) + d(2) * (bdy * bdx);
    if (alongK) return AffineMap::get(4, 0, ArrayRef<AffineExpr>({(vt % (BK / W)) * W + d(3), vt.floorDiv(BK / W)}));
    return AffineMap::get(3, 0, ArrayRef<AffineExpr>({vt.floorDiv(extent / W), (vt % (extent / W)) * W}));
  }
  AffineMap storeTileA() const { return storeTile(!tA, BM); }
  AffineMap storeTileB() const { return storeTile(tB, BN); }
  AffineExpr laneId() const { return (d(0) * bdx + d(1)) % (L.ty * L.tx); }
  AffineExpr warpId() const { return (d(0) * bdx + d(1)).floorDiv(L.ty * L.tx); }
  // index (in vectors of W) of the thread's iv-th group of rows / columns inside the workgroup tile
  AffineExpr rowVector(AffineExpr iv) const { return laneId().floorDiv(L.tx) + (warpId().floorDiv(L.wx) + iv * L.wy) * L.ty; }
  AffineExpr colVector(AffineExpr iv) const { return laneId() % L.tx + (warpId() % L.wx + iv * L.wx) * L.tx; }
  // operands: [ty, tx, k_inner, iv] -> smA[k, m] / smB[k, n]
  AffineMap loadFragA() const { return AffineMap::get(4, 0, ArrayRef<AffineExpr>({d(2), rowVector(d(3)) * W})); }
  AffineMap loadFragB() const { return AffineMap::get(4, 0, ArrayRef<AffineExpr>({d(2), colVector(d(3)) * W})); }
  AffineMap cacheRead() const { return AffineMap::get(1, 0, d(0)); }
  // operands: [b.., ty, tx, blockIdx.m, blockIdx.n, iv0, iv1, iv2, iv3] -> C[b.., m, n]
  AffineMap cacheWriteC() const {
    // shift the thread-id dims behind the batch dims
    SmallVector<AffineExpr> shift;
    for (unsigned i = 0; i < 2; ++i) shift.push_back(d(nb + i));
    AffineExpr rv = rowVector(getAffineDimExpr(2).floorDiv(W));   // iv0 at position 2 of a (ty, tx, iv0) view
    AffineExpr cv = colVector(getAffineDimExpr(2).floorDiv(W));
    SmallVector<AffineExpr> forRows{d(nb), d(nb + 1), d(nb + 4)}, forCols{d(nb), d(nb + 1), d(nb + 5)};
    AffineExpr m = d(nb + 2) * BM + rv.replaceDims(forRows) * W + d(nb + 6);
    AffineExpr n = d(nb + 3) * BN + cv.replaceDims(forCols) * W + d(nb + 7);
    return withBatch(8, {m, n});
  }
};

bool checkGemmConfig(const std::map<std::string, int>& c, int64_t M, int64_t N, int64_t K, std::string& why,
                     bool transA = false, bool transB = false) {
  GemmMaps g(c, 0, transA, transB);
  std::ostringstream os;
  if (g.BM <= 0 || g.BN <= 0 || g.BK <= 0 || g.TM <= 0 || g.TN <= 0 || g.W <= 0) os << "missing tile sizes; ";
  else {
    const int64_t threads = g.bdy * g.bdx;
    if (g.BM % g.TM || g.BN % g.TN) os << "THREAD_SIZE must divide BLOCK_SIZE; ";
    if (M % g.BM || N % g.BN || K % g.BK) os << "problem " << M << "x" << N << "x" << K << " is not a multiple of the tile; ";
    if (!g.L.ok) os << "workgroup of " << g.bdy << "x" << g.bdx << " threads does not split into wavefronts; ";
    if (threads <= 0 || (g.BK * g.BM) % (threads * g.W) || (g.BK * g.BN) % (threads * g.W)) os << "tile copies do not divide over the threads; ";
    if (g.TM % g.W || g.TN % g.W || g.BK % g.W || g.BN % g.W) os << "VECTORIZE_WIDTH must divide the thread tile and BLOCK_SIZE_K/N; ";
    if (transA && g.BM % g.W) os << "VECTORIZE_WIDTH must divide BLOCK_SIZE_M for a column-major A; ";
    if (threads > 1024) os << "more than 1024 threads; ";
  }
  why = os.str();
  return why.empty();
}

// The schedule.  `loops` = batch loops, then M, N, K; A, B, C as seen inside the function.
void gemmSchedule(ModuleOp& module, std::vector<AffineForOp> loops, Value A, Value B, Value C,
                  const std::map<std::string, int>& c, bool transA = false, bool transB = false) {
  // several batch loops become one: the grid has three dimensions, one of them for the batch
  std::vector<int64_t> batchShape;
  for (size_t i = 0; i + 3 < loops.size(); ++i) batchShape.push_back(loops[i].getConstantUpperBound());
  if (batchShape.size() > 1) {
    std::vector<AffineForOp> batchLoops(loops.begin(), loops.end() - 3);
    AffineForOp one = Rewriter::combineToOneDim(batchLoops);
    loops.erase(loops.begin(), loops.end() - 3);
    loops.insert(loops.begin(), one);
    DUMP(module);
  }
  const unsigned nb = (unsigned)loops.size() - 3;
  GemmMaps g(c, nb, transA, transB, batchShape);
  AffineForOp loopM = loops[nb], loopN = loops[nb + 1], loopK = loops[nb + 2];

  // tile M and N for workgroups and threads
  auto mAxes = Rewriter::split(loopM, 3, {(int64_t)g.TM, (int64_t)g.BM});
  auto nAxes = Rewriter::split(loopN, 3, {(int64_t)g.TN, (int64_t)g.BN});
  DUMP(module);
  AffineForOp mOuter = mAxes[0], mMid = mAxes[1], mInner = mAxes[2];
  AffineForOp nOuter = nAxes[0], nMid = nAxes[1], nInner = nAxes[2];
  Rewriter::reorder({mOuter, nOuter, mMid, nMid, mInner, nInner});
  DUMP(module);

  std::vector<AffineForOp> gridLoops(loops.begin(), loops.begin() + nb);
  gridLoops.push_back(mOuter);
  gridLoops.push_back(nOuter);
  AffineParallelOp gridLevel = Rewriter::parallel(gridLoops);
  AffineParallelOp blockLevel = Rewriter::parallel({mMid, nMid});
  DUMP(module);

  // accumulator -> register tile, then k outermost inside the thread
  std::vector<AffineForOp> kmn{loopK, mInner, nInner};
  Rewriter::bufferizeLoopCarryVar(kmn);
  loopK = kmn[0]; mInner = kmn[1]; nInner = kmn[2];
  DUMP(module);
  Rewriter::reorder({loopK, mInner, nInner});
  DUMP(module);
  auto kAxes = Rewriter::split(loopK, 2, {(int64_t)g.BK});
  AffineForOp kOuter = kAxes[0], kInner = kAxes[1];
  DUMP(module);

  int64_t blockThreads;
  Analyzer::getParallelNumber(blockLevel, blockThreads);
  Type elementA = A.getType().cast<MemRefType>().getElementType();
  Type elementB = B.getType().cast<MemRefType>().getElementType();

  Value fragB = Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {g.TN}, elementB);
  Value fragA = Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {g.TM}, elementA);
  Value tileB = Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {g.BK * g.BN / blockThreads}, elementB);
  Value tileA = Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {g.BK * g.BM / blockThreads}, elementA);
  Value smB = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {g.BK, g.BN}, elementB);
  Value smA = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {g.BK, g.BM}, elementA);
  DUMP(module);

  auto blockIdx = Rewriter::getParallelIdx(gridLevel);   // [b.., by, bx]
  auto threadIdx = Rewriter::getParallelIdx(blockLevel); // [ty, tx]
  SmallVector<Value> batchIdx(blockIdx.begin(), blockIdx.begin() + nb);
  Value by = blockIdx[nb], bx = blockIdx[nb + 1], ty = threadIdx[0], tx = threadIdx[1];
  auto withBatch = [&](std::initializer_list<Value> rest) {
    SmallVector<Value> v = batchIdx;
    v.append(rest);
    return v;
  };

  // global -> registers -> LDS, once per k tile
  auto loadTileA = Rewriter::read(A, tileA, g.loadTileA(), withBatch({ty, tx, by, kOuter.getInductionVar()}), g.W, kOuter, Position::begin);
  auto loadTileB = Rewriter::read(B, tileB, g.loadTileB(), withBatch({ty, tx, kOuter.getInductionVar(), bx}), g.W, loadTileA, Position::after);
  auto storeTileA = Rewriter::write(tileA, smA, g.storeTileA(), {ty, tx}, g.W, loadTileB, Position::after);
  auto storeTileB = Rewriter::write(tileB, smB, g.storeTileB(), {ty, tx}, g.W, storeTileA, Position::after);
  auto barrierPrefix = Rewriter::barrier(loadTileA, Position::before);
  auto barrierSuffix = Rewriter::barrier(storeTileB, Position::after);
  DUMP(module);

  // LDS -> fragments, once per k
  auto loadFragA = Rewriter::read(smA, fragA, g.loadFragA(), {ty, tx, kInner.getInductionVar()}, g.W, kInner, Position::begin);
  auto loadFragB = Rewriter::read(smB, fragB, g.loadFragB(), {ty, tx, kInner.getInductionVar()}, g.W, loadFragA, Position::after);
  DUMP(module);
  Rewriter::cache_read(kInner, A, fragA, g.cacheRead(), {mInner.getInductionVar()});
  Rewriter::cache_read(kInner, B, fragB, g.cacheRead(), {nInner.getInductionVar()});
  DUMP(module);

  // write-back of the register tile with the final index map, vectorised along n
  auto writeC = Rewriter::get_write(blockLevel, C);
  assert(writeC.size() == 1 && writeC[0].size() == 2);
  auto mW = Rewriter::split(writeC[0][0], 2, {(int64_t)g.W});
  auto nW = Rewriter::split(writeC[0][1], 2, {(int64_t)g.W});
  Rewriter::reorder({mW[0], nW[0], mW[1], nW[1]});
  DUMP(module);
  Rewriter::cache_write(mW[0], C, C, g.cacheWriteC(),
                        withBatch({ty, tx, by, bx, mW[0].getInductionVar(), nW[0].getInductionVar(),
                                   mW[1].getInductionVar(), nW[1].getInductionVar()}));
  Rewriter::vectorize(nW[1], g.W);
  DUMP(module);

  // double buffering of LDS over k tiles and of the fragments over k
  auto dblTileB = Rewriter::pipeline({loadTileB, storeTileB}, smB, kOuter);
  auto dblTileA = Rewriter::pipeline({loadTileA, storeTileA}, smA, kOuter);
  auto dblFragB = Rewriter::pipeline({loadFragB}, fragB, kInner);
  auto dblFragA = Rewriter::pipeline({loadFragA}, fragA, kInner);
  DUMP(module);
  Rewriter::detach_last_loop(kInner);
  DUMP(module);

  // order: global loads first, LDS stores after the compute, fragment prefetch of the next tile last
  Rewriter::schedule(dblTileA[0][0], dblTileB[0][0], Position::before);
  Rewriter::schedule(dblTileA[0][1], dblTileB[0][1], Position::before);
  Rewriter::schedule(barrierPrefix, dblTileB[0][1], Position::after);
  Rewriter::schedule(dblTileB[1][0], dblTileA[1][0], Position::after);
  Rewriter::schedule(dblTileA[1][1], dblTileB[1][1], Position::before);
  Rewriter::schedule(barrierSuffix, dblTileB[1][1], Position::after);
  Operation* storeIf = dblTileA[1][1]->getParentOp();
  Rewriter::schedule(storeIf, kInner, Position::after);
  Rewriter::extract_loop(dblFragA[0][0], kOuter, /*iteration*/ 0);
  Rewriter::extract_loop(dblFragB[0][0], kOuter, /*iteration*/ 0);
  Rewriter::schedule(dblFragB[0][0], kOuter, Position::end);
  Rewriter::schedule(dblFragA[0][0], kOuter, Position::end);
  DUMP(module);
  Rewriter::change_double_buffer(dblFragA[0][0], smA);
  Rewriter::change_double_buffer(dblFragB[0][0], smB);
  DUMP(module);

  Rewriter::take_off_true_if(module);
  Rewriter::delete_false_if(module);
  DUMP(module);

  const int64_t threshold = std::max<int64_t>(g.BK, std::max(g.TM, g.TN));
  auto trips = [](AffineForOp loop) { return (loop.getConstantUpperBound() - loop.getConstantLowerBound()) / loop.getStep(); };
  // the passes walk the whole module; only loops of this function are touched
  Operation* scope = gridLevel->getParentOp();
  Rewriter::unroll(module, [&](AffineForOp loop) -> bool {
    if (!scope->isAncestor(loop) || !loop.hasConstantBounds()) return false;
    return trips(loop) < std::min<int64_t>(threshold, g.W);
  });
  Rewriter::unrollAttribute(module, [&](AffineForOp loop) -> bool {
    if (!scope->isAncestor(loop) || !loop.hasConstantBounds()) return false;
    return trips(loop) <= threshold;
  });
  DUMP(module);
}

}  // namespace

// ===========================================================================
// MatmulOptimizer (reference: Optimizer.cc:243-570)
// ===========================================================================
bool MatmulOptimizer::applicable(ModuleOp& module) {
  clear();
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "Matmul")) {
    if (f.getSymName().find("BatchMatmul") != std::string::npos) continue;
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;  // already scheduled
    auto loops = Analyzer::collectFuncLoops(f);
    // (A, B), or (A, B, scaleA, scaleB) for a quantised product whose scales are graph values
    if (loops.size() != 3 || f.getNumArguments() != (f->hasAttr("kcg.scales") ? 4u : 2u)) continue;
    Value A = f.getArgument(0);
    if (!configMatchesType(matmulConfig, A.getType().cast<MemRefType>().getElementType())) continue;
    auto shapeA = A.getType().cast<MemRefType>().getShape();
    auto shapeB = f.getArgument(1).getType().cast<MemRefType>().getShape();
    std::string why;
    if (!checkGemmConfig(matmulConfig, shapeA[0], shapeB[1], shapeA[1], why)) {
      // Only the extents' fault?  Then the guarded schedule takes it (RAGGED = 0 leaves it unscheduled, as the
      // reference does with every such product).
      GemmMaps g(matmulConfig, 0);
      auto up = [](int64_t x, int64_t t) { return t > 0 ? (x + t - 1) / t * t : x; };
      std::string other;
      if (!cfg(matmulConfig, "RAGGED", 1) ||
          !checkGemmConfig(matmulConfig, up(shapeA[0], g.BM), up(shapeB[1], g.BN), up(shapeA[1], g.BK), other)) {
        llvm::errs() << "MatmulOptimizer: " << f.getSymName() << " not scheduled: " << why << "\n";
        continue;
      }
      raggedMatmuls.insert(f);
    }
    matmuls.insert(f);
    matmulLoops[f] = loops;
    MemoryBuffer buf;
    buf.A = A;
    buf.B = f.getArgument(1);
    buf.C = f.front().back().getOperand(0);  // the returned memref
    matmulBuffers[f] = buf;
    any = true;
  }
  return any;
}

AffineMap MatmulOptimizer::getAffineMap(const std::string& id, OpBuilder&) {
  GemmMaps g(matmulConfig, 0);
  if (id == "loadTileA") return g.loadTileA();
  if (id == "loadTileB") return g.loadTileB();
  if (id == "storeTileA") return g.storeTileA();
  if (id == "storeTileB") return g.storeTileB();
  if (id == "loadFragA") return g.loadFragA();
  if (id == "loadFragB") return g.loadFragB();
  if (id == "cacheReadA" || id == "cacheReadB") return g.cacheRead();
  if (id == "cacheWriteC") return g.cacheWriteC();
  assert(false && "unknown map identifier");
  return AffineMap();
}

// Matmul whose only consumer is a not yet scheduled in-place Relu call (the fusion the reference
// sketches at test/test.cc:59-63): the Relu moves in front of the store of the finished dot
// product, the Relu call disappears and the Matmul call stands for both.
static bool fuseFollowingRelu(ModuleOp& module, func::FuncOp f, AffineForOp loopK, Value C, OpBuilder& builder) {
  func::CallOp mmCall(nullptr);
  int callsOfF = 0;
  for (auto c : Analyzer::collectFuncCalls(module))
    if (c.getCallee() == f.getName()) {
      mmCall = c;
      ++callsOfF;
    }
  if (callsOfF != 1) return false;
  auto users = mmCall.getResult(0).getUsers();
  if (users.size() != 1) return false;
  auto reluCall = dyn_cast<func::CallOp>(users[0]);
  if (!reluCall || reluCall.getCallee().rfind("Relu_Elementwise_", 0) != 0) return false;
  auto g = Analyzer::getTargetFunction(module, reluCall.getCallee());
  if (!g || g->getAttr("func.state").s != "cpu") return false;
  if (reluCall.getResult(0).getType() != mmCall.getResult(0).getType()) return false;
  int callsOfG = 0;
  for (auto c : Analyzer::collectFuncCalls(module))
    if (c.getCallee() == g.getName()) ++callsOfG;

  // the store of the reduction result follows the k loop
  AffineStoreOp store(nullptr);
  for (Operation* op = loopK->getNextNode(); op; op = op->getNextNode())
    if (auto st = dyn_cast<AffineStoreOp>(op))
      if (st.getMemRef() == C && st.getValue() == loopK.getResult(0)) store = st;
  if (!store) return false;
  OpBuilder b(store->getContext());
  b.setInsertionPoint(store.getOperation());
  Value y = store.getValue();
  store->setOperand(0, ElementWise::relu(b, y, y.getType()));

  reluCall.getResult(0).replaceAllUsesWith(mmCall.getResult(0));
  reluCall.erase();
  if (callsOfG == 1) g.erase();
  f->setAttr("kcg.fused_relu", builder.getI64IntegerAttr(1));
  return true;
}

// A product whose extents are not multiples of the tile.  The loops over m and n run to the next multiple and their
// body stands under `if (m < M && n < N)`; then they are tiled like any other (workgroups of BLOCK_SIZE_M x
// BLOCK_SIZE_N results, THREAD_SIZE_M x THREAD_SIZE_N of them per thread), each thread adding up its dot products
// along the whole of k from global memory.  No shared tiles and no pipeline: those assume full tiles (the
// reference's irregularMat, Rewriter.cc:2057-2101, clones a nest four times for the edges of an elementwise map; a
// pipelined product would need that around every stage).  The gfx950 GEMM families guard their own edges, so the
// kernel such a function gets is as fast as any; the schedule is what the interpreter and the statement-by-statement
// lowering run.
static void raggedGemmSchedule(ModuleOp& module, std::vector<AffineForOp> loops, const std::map<std::string, int>& c, int64_t M, int64_t N) {
  GemmMaps g(c, 0);
  // batch loops in front (a batched product): several become one, which is the grid's third dimension
  if (loops.size() > 4) {
    std::vector<AffineForOp> batchLoops(loops.begin(), loops.end() - 3);
    AffineForOp one = Rewriter::combineToOneDim(batchLoops);
    loops.erase(loops.begin(), loops.end() - 3);
    loops.insert(loops.begin(), one);
    DUMP(module);
  }
  const size_t nb = loops.size() - 3;
  AffineForOp loopM = loops[nb], loopN = loops[nb + 1];
  OpBuilder b = OpBuilder::atBlockBegin(loopN.getBody());
  Location loc = b.getUnknownLoc();
  // the guard reads the indices through affine.apply, which is what split() knows how to rewrite
  AffineMap id = AffineMap::get(1, 0, getAffineDimExpr(0));
  Value m = b.create<AffineApplyOp>(loc, id, ValueRange({loopM.getInductionVar()})).getResult();
  Value n = b.create<AffineApplyOp>(loc, id, ValueRange({loopN.getInductionVar()})).getResult();
  auto inside = IntegerSet::get(2, 0, ArrayRef<AffineExpr>({(M - 1) - getAffineDimExpr(0), (N - 1) - getAffineDimExpr(1)}),
                                ArrayRef<bool>({false, false}));
  auto guard = b.create<AffineIfOp>(loc, inside, ValueRange({m, n}), false);
  for (Operation* op = guard->getNextNode(); op && op->getKind() != OpKind::AffineYield;) {
    Operation* next = op->getNextNode();
    op->moveBefore(guard.getThenBlock()->getTerminator());
    op = next;
  }
  auto up = [](int64_t x, int64_t t) { return (x + t - 1) / t * t; };
  loopM.setConstantUpperBound(up(M, g.BM));
  loopN.setConstantUpperBound(up(N, g.BN));
  DUMP(module);
  auto ms = Rewriter::split(loopM, 3, {g.TM, g.BM});
  auto ns = Rewriter::split(loopN, 3, {g.TN, g.BN});
  Rewriter::reorder({ms[0], ns[0], ms[1], ns[1], ms[2], ns[2]});
  DUMP(module);
  std::vector<AffineForOp> gridLoops(loops.begin(), loops.begin() + nb);
  gridLoops.push_back(ms[0]);
  gridLoops.push_back(ns[0]);
  Rewriter::parallel(gridLoops);
  Rewriter::parallel({ms[1], ns[1]});
  DUMP(module);
}

void MatmulOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : matmuls) {
    tagFunction(f, "Matmul", matmulConfig, builder);
    auto& buf = matmulBuffers[f];
    if (cfg(matmulConfig, "FUSE_RELU", 1)) fuseFollowingRelu(module, f, matmulLoops[f][2], buf.C, builder);
    if (raggedMatmuls.count(f)) {
      auto shape = buf.C.getType().cast<MemRefType>().getShape();
      f->setAttr("kcg.ragged", builder.getI64IntegerAttr(1));
      raggedGemmSchedule(module, matmulLoops[f], matmulConfig, shape[0], shape[1]);
    } else {
      gemmSchedule(module, matmulLoops[f], buf.A, buf.B, buf.C, matmulConfig);
    }
  }
}

// ===========================================================================
// BatchMatmulOptimizer (reference: Optimizer.cc:2863-2893, 3168-3445)
// ===========================================================================
bool identifyBatchMatmul(const std::string& name, BatchMatmulDescriptor& out) {
  std::vector<std::string> parts;
  std::stringstream ss(name);
  std::string item;
  while (std::getline(ss, item, '_')) parts.push_back(item);
  if (!parts.empty() && parts.back() == "scaled") parts.pop_back();      // a product that carries per-tensor scales
  if (parts.size() < 5 || parts[0] != "BatchMatmul") return false;
  const size_t n = parts.size();
  auto number = [](const std::string& s, size_t from, int& v) {
    if (s.size() <= from) return false;
    for (size_t i = from; i < s.size(); ++i) if (!isdigit((unsigned char)s[i])) return false;
    v = std::stoi(s.substr(from));
    return true;
  };
  const std::string& layout = parts[n - 1];
  if (layout.size() != 2 || (layout[0] != 'N' && layout[0] != 'T') || (layout[1] != 'N' && layout[1] != 'T')) return false;
  if (parts[n - 4][0] != 'm' || parts[n - 3][0] != 'n' || parts[n - 2][0] != 'k') return false;
  if (!number(parts[n - 4], 1, out.m) || !number(parts[n - 3], 1, out.n) || !number(parts[n - 2], 1, out.k)) return false;
  out.transA = layout[0] == 'T';
  out.transB = layout[1] == 'T';
  out.batch.clear();
  for (size_t i = 1; i + 4 < n; ++i) {
    int b;
    if (!number(parts[i], 0, b)) return false;
    out.batch.push_back(b);
  }
  return true;
}

bool BatchMatmulOptimizer::applicable(ModuleOp& module) {
  clear();
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "BatchMatmul")) {
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;
    BatchMatmulDescriptor desc;
    if (!identifyBatchMatmul(f.getSymName(), desc)) continue;
    auto loops = Analyzer::collectFuncLoops(f);
    // (A, B, C), or (A, B, C, scaleA, scaleB) for a quantised product whose scales are graph values
    if (loops.size() != desc.batch.size() + 3 || f.getNumArguments() != (f->hasAttr("kcg.scales") ? 5u : 3u)) continue;
    Value A = f.getArgument(0);
    if (!configMatchesType(batchMatmulConfig, A.getType().cast<MemRefType>().getElementType())) continue;
    std::string why;
    if (!checkGemmConfig(batchMatmulConfig, desc.m, desc.n, desc.k, why, desc.transA, desc.transB)) {
      GemmMaps g(batchMatmulConfig, 0);
      auto up = [](int64_t x, int64_t t) { return t > 0 ? (x + t - 1) / t * t : x; };
      std::string other;
      if (!cfg(batchMatmulConfig, "RAGGED", 1) ||
          !checkGemmConfig(batchMatmulConfig, up(desc.m, g.BM), up(desc.n, g.BN), up(desc.k, g.BK), other, desc.transA, desc.transB)) {
        llvm::errs() << "BatchMatmulOptimizer: " << f.getSymName() << " not scheduled: " << why << "\n";
        continue;
      }
      raggedBatchMatmuls.insert(f);
    }
    batchMatmuls.insert(f);
    batchMatmulLoops[f] = loops;
    MemoryBuffer buf;
    buf.A = A;
    buf.B = f.getArgument(1);
    buf.C = f.front().back().getOperand(0);
    buf.matmul = desc;
    batchMatmulBuffers[f] = buf;
    any = true;
  }
  return any;
}

AffineMap BatchMatmulOptimizer::getAffineMap(const std::string& id, OpBuilder&) {
  GemmMaps g(batchMatmulConfig, 1);
  if (id == "loadTileA") return g.loadTileA();
  if (id == "loadTileB") return g.loadTileB();
  if (id == "storeTileA") return g.storeTileA();
  if (id == "storeTileB") return g.storeTileB();
  if (id == "loadFragA") return g.loadFragA();
  if (id == "loadFragB") return g.loadFragB();
  if (id == "cacheReadA" || id == "cacheReadB") return g.cacheRead();
  if (id == "cacheWriteC") return g.cacheWriteC();
  assert(false && "unknown map identifier");
  return AffineMap();
}

void BatchMatmulOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : batchMatmuls) {
    tagFunction(f, "BatchMatmul", batchMatmulConfig, builder);
    auto& buf = batchMatmulBuffers[f];
    if (raggedBatchMatmuls.count(f)) {
      f->setAttr("kcg.ragged", builder.getI64IntegerAttr(1));
      raggedGemmSchedule(module, batchMatmulLoops[f], batchMatmulConfig, buf.matmul.m, buf.matmul.n);
      continue;
    }
    gemmSchedule(module, batchMatmulLoops[f], buf.A, buf.B, buf.C, batchMatmulConfig, buf.matmul.transA, buf.matmul.transB);
  }
}

}  // namespace KernelCodeGen

// ===========================================================================
// BinaryOptimizer (reference: Optimizer.cc:928-991)
//
// X op Y with broadcasting.  The nest is collapsed to one dimension and cut
// into workgroups of threads that each own `width` consecutive elements of the
// flattened result; the broadcast indices stay what the builder made them
// (index 0 along a dimension of extent 1).  Arithmetic results only: the
// comparison forms (Equal, Greater) keep their host nest.
// Config: BLOCK_SIZE_M * BLOCK_SIZE_N / (THREAD_SIZE_M * THREAD_SIZE_N) threads
// per workgroup, VECTORIZE_WIDTH elements per thread, both shrunk to divisors
// of the element count.
// ===========================================================================
namespace KernelCodeGen {

using namespace mlir;

bool BinaryOptimizer::applicable(ModuleOp& module) {
  clear();
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "_Binary")) {
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;
    if (f.getNumArguments() != 2) continue;
    const std::string name = f.getSymName();
    const std::string op = name.substr(0, name.find("_Binary"));
    const bool compare = op == "Equal" || op == "Greater";
    if (!compare && op != "Add" && op != "Sub" && op != "Mul" && op != "Div" && op != "Pow") continue;
    auto outType = f.getFunctionType().getResult(0).cast<MemRefType>();
    auto inType = f.getArgument(0).getType().cast<MemRefType>();
    // two operands of one float type (the broadcast kernel family has fp32 and half forms; f64 and bf16 run as the
    // schedule itself); the result has their type, or is i1 for a comparison
    const Type elem = inType.getElementType();
    if ((!elem.isF32() && !elem.isF16() && !elem.isF64() && !elem.isBF16()) || f.getArgument(1).getType().cast<MemRefType>().getElementType() != elem) continue;
    if (compare ? outType.getElementType() == elem : outType.getElementType() != elem) continue;
    if (!configMatchesType(binaryConfig, inType.getElementType())) continue;
    auto loops = Analyzer::collectFuncLoops(f);
    if ((int64_t)loops.size() != outType.getRank() || loops.empty()) continue;
    binarys.insert(f);
    binaryLoops[f] = loops;
    MemoryBuffer abc;
    abc.A = f.getArgument(0);
    abc.B = f.getArgument(1);
    abc.C = f.front().back().getOperand(0);
    binaryBuffers[f] = abc;
    any = true;
  }
  return any;
}

void BinaryOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : binarys) {
    auto loops = binaryLoops[f];
    int64_t total = 1;
    for (auto l : loops) total *= l.getConstantUpperBound();
    int64_t width = cfg(binaryConfig, "VECTORIZE_WIDTH", 4);
    if (loops.back().getConstantUpperBound() % width) width = 1;
    int64_t threads = cfg(binaryConfig, "BLOCK_SIZE_M", 64) * cfg(binaryConfig, "BLOCK_SIZE_N", 64) /
                      std::max(1, cfg(binaryConfig, "THREAD_SIZE_M", 4) * cfg(binaryConfig, "THREAD_SIZE_N", 4));
    threads = std::min<int64_t>(std::max<int64_t>(threads, 1), 1024);
    while (threads > 1 && (total / width) % threads) --threads;     // largest divisor not above the configured count
    std::map<std::string, int> used = binaryConfig;
    used["THREADS"] = (int)threads;
    used["VECTORIZE_WIDTH"] = (int)width;
    tagFunction(f, "Binary", used, builder);

    AffineForOp flat = Rewriter::combineToOneDim(loops);
    DUMP(module);
    auto parts = Rewriter::split(flat, 3, {width, threads * width});
    DUMP(module);
    AffineParallelOp gridLevel = Rewriter::parallel({parts[0]});
    AffineParallelOp blockLevel = Rewriter::parallel({parts[1]});
    (void)gridLevel;
    (void)blockLevel;
    DUMP(module);
    Rewriter::unrollAttribute(module, [&](AffineForOp loop) -> bool {
      return f->isAncestor(loop) && loop.hasConstantBounds() && loop.getConstantUpperBound() <= 16;
    });
    DUMP(module);
  }
}

// ===========================================================================
// GatherOptimizer (reference: Optimizer.cc:1940-2074).  The nest has one loop per result
// dimension; its body reads the index (affine.load), the element it names (memref.load) and
// stores it.  Schedule: all loops into one, split into per-thread runs of consecutive elements,
// grid and workgroup levels.  The function name carries input shape, index shape and axis.
// ===========================================================================
namespace {

// "Gather_<input dims>_indices_<index dims>_axis_<a>" -> a, or -1
int64_t gatherAxisOf(const std::string& name) {
  const size_t at = name.rfind("_axis_");
  if (name.rfind("Gather_", 0) != 0 || at == std::string::npos) return -1;
  const std::string digits = name.substr(at + 6);
  if (digits.empty() || digits.find_first_not_of("0123456789") != std::string::npos) return -1;
  return std::stoll(digits);
}

}  // namespace

bool GatherOptimizer::applicable(ModuleOp& module) {
  clear();
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "Gather_")) {
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;
    if (f.getNumArguments() != 2 || gatherAxisOf(f.getSymName()) < 0) continue;
    auto outType = f.getFunctionType().getResult(0).cast<MemRefType>();
    auto loops = Analyzer::collectFuncLoops(f);
    if ((int64_t)loops.size() != outType.getRank() || loops.empty()) continue;
    // the body the Frontend builds: one memref.load addressed by a loaded index, one store
    int loads = 0, stores = 0;
    f->walk([&](Operation* op) {
      if (op->getKind() == OpKind::MemLoad) ++loads;
      if (op->getKind() == OpKind::AffineStore) ++stores;
    }, WalkOrder::PreOrder);
    if (loads != 1 || stores != 1) continue;
    MemoryBuffer buf;
    buf.input = f.getArgument(0);
    buf.indices = f.getArgument(1);
    Operation& ret = f.front().back();
    buf.output = ret.getOperand(0);
    gathers.insert(f);
    gatherBuffers[f] = buf;
    gatherLoops[f] = loops;
    any = true;
  }
  return any;
}

void GatherOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : gathers) {
    auto loops = gatherLoops[f];
    int64_t total = 1;
    for (auto l : loops) total *= l.getConstantUpperBound();
    // a thread moves `width` consecutive elements of the result when the innermost result dimension allows
    int64_t width = cfg(gatherConfig, "VECTORIZE_WIDTH", 4);
    if (width < 1 || loops.back().getConstantUpperBound() % width) width = 1;
    int64_t threads = cfg(gatherConfig, "BLOCK_SIZE_M", 64) * cfg(gatherConfig, "BLOCK_SIZE_N", 64) /
                      std::max(1, cfg(gatherConfig, "THREAD_SIZE_M", 4) * cfg(gatherConfig, "THREAD_SIZE_N", 4));
    threads = std::min<int64_t>(std::max<int64_t>(threads, 1), 1024);
    while (threads > 1 && (total / width) % threads) --threads;     // largest divisor not above the configured count
    std::map<std::string, int> used = gatherConfig;
    used["THREADS"] = (int)threads;
    used["VECTORIZE_WIDTH"] = (int)width;
    used["AXIS"] = (int)gatherAxisOf(f.getSymName());
    tagFunction(f, "Gather", used, builder);

    AffineForOp flat = Rewriter::combineToOneDim(loops);
    DUMP(module);
    auto parts = Rewriter::split(flat, 3, {width, threads * width});
    DUMP(module);
    AffineParallelOp gridLevel = Rewriter::parallel({parts[0]});
    AffineParallelOp blockLevel = Rewriter::parallel({parts[1]});
    (void)gridLevel;
    (void)blockLevel;
    DUMP(module);
    Rewriter::unrollAttribute(module, [&](AffineForOp loop) -> bool {
      return f->isAncestor(loop) && loop.hasConstantBounds() && loop.getConstantUpperBound() <= 16;
    });
    DUMP(module);
  }
}

}  // namespace KernelCodeGen

// ===========================================================================
// ElementWiseOptimizer (reference: Optimizer.cc:995-1175)
// ===========================================================================
namespace KernelCodeGen {

using namespace mlir;

namespace {

// Largest divisor of `n` that is <= `limit` and a multiple of `unit` (unit itself must divide n).
int64_t largestDivisor(int64_t n, int64_t limit, int64_t unit) {
  for (int64_t d = std::min(limit, n) / unit * unit; d >= unit; d -= unit)
    if (n % d == 0) return d;
  return unit;
}

// Puts everything a function does before its return into a new loop of one trip (0..1) and returns that loop: an
// operator over a single row then has the outer loop that the schedules turn into the grid level.
AffineForOp wrapBodyInUnitLoop(func::FuncOp f, OpBuilder& builder) {
  Block& body = f.front();
  auto ip = builder.saveInsertionPoint();
  builder.setInsertionPointToStart(&body);
  auto loop = builder.create<AffineForOp>(builder.getUnknownLoc(), 0, 1, 1);
  builder.restoreInsertionPoint(ip);
  Operation* op = loop->getNextNode();
  while (op && op->getKind() != OpKind::Return) {
    Operation* next = op->getNextNode();
    if (op->getKind() == OpKind::Alloc) op->moveBefore(loop.getOperation());      // the result buffer stays in front of the loop
    else op->moveBefore(loop.getBody()->getTerminator());
    op = next;
  }
  return loop;
}

// Replaces `loop` (0..ub step s, no iter_args) by its body executed once with
// the index given by `apply(d0 -> d0 * s)` of `threadIdx`: the loop becomes a
// dimension of the enclosing thread level.
void bindLoopToThread(AffineForOp loop, Value threadIdx) {
  assert(loop.hasConstantBounds() && loop.getConstantLowerBound() == 0 && loop.getNumIterOperands() == 0);
  OpBuilder b(loop.getOperation());
  Value idx = b.create<AffineApplyOp>(b.getUnknownLoc(), AffineMap::get(1, 0, getAffineDimExpr(0) * loop.getStep()),
                                      ValueRange({threadIdx})).getResult();
  loop.getInductionVar().replaceAllUsesWith(idx);
  Operation* op = loop.getBody()->empty() ? nullptr : &loop.getBody()->front();
  while (op) {
    Operation* next = op->getNextNode();
    if (!(op->getKind() == OpKind::AffineYield && !next)) op->moveBefore(loop.getOperation());
    op = next;
  }
  loop.erase();
}

// A reduction pass of a row team: `loop` carries one running sum over the row.  Each of the `tpr` threads
// (index `tid`) accumulates a partial over its own `width`-wide slices, publishes it in `shared`, and after
// a barrier every thread adds up all partials; later users of the loop's result see that total.
// `tree` (a level and a one-element shared cell): the partials are added up the way the reference's LayerNorm
// schedule does it (Optimizer.cc:1623-1749, LayerNormOptimizer::reduceUnrollOptimize): halving steps in shared memory
// down to one wavefront, shuffles inside it, lane 0 adds the total into the cell, everybody reads the cell.  Without it
// every thread adds up all partials itself.
void scheduleTeamReduction(AffineForOp loop, Value shared, Value tid, int64_t width, int64_t tpr, Type element,
                           AffineParallelOp treeLevel = AffineParallelOp(), Value treeCell = Value()) {
  std::vector<AffineForOp> one{loop};
  Value cell = Rewriter::bufferizeLoopCarryVar(one);
  loop = one[0];
  auto parts = Rewriter::split(loop, 3, {width, tpr * width});
  bindLoopToThread(parts[1], tid);
  // the load that follows the loop reads the thread's partial: publish it, then add up all partials
  Operation* after = parts[0]->getNextNode();
  auto partialLoad = dyn_cast<AffineLoadOp>(after);
  assert(partialLoad && partialLoad.getMemRef() == cell);
  OpBuilder rb(partialLoad->getContext());
  rb.setInsertionPointAfter(partialLoad.getOperation());
  Location loc = rb.getUnknownLoc();
  rb.create<AffineStoreOp>(loc, partialLoad.getResult(), shared, ValueRange({tid}));
  if (treeLevel) {
    Value zeroIdx = rb.create<arith::ConstantIndexOp>(loc, 0).getResult();
    Value zero = rb.create<arith::ConstantOp>(loc, rb.getFloatAttr(element, 0)).getResult();
    rb.create<AffineStoreOp>(loc, zero, treeCell, ValueRange({zeroIdx}));      // every thread, the same value
    // one element per thread, accumulated into the cell: the loop shape the tree builder takes
    auto flat = rb.create<AffineForOp>(loc, 0, 1, 1, ValueRange({}),
      [&](OpBuilder& lb, Location lloc, Value i, ValueRange) {
        Value c = lb.create<AffineLoadOp>(lloc, treeCell, ValueRange({zeroIdx})).getResult();
        Value v = lb.create<AffineLoadOp>(lloc, shared, AffineMap::get(2, 0, getAffineDimExpr(0) + getAffineDimExpr(1) * tpr), ValueRange({tid, i})).getResult();
        lb.create<AffineStoreOp>(lloc, lb.create<arith::AddFOp>(lloc, c, v).getResult(), treeCell, ValueRange({zeroIdx}));
        lb.create<AffineYieldOp>(lloc, ValueRange({}));
      });
    auto created = LayerNormOptimizer().reduceUnrollOptimize(flat, treeLevel);
    rb.setInsertionPointAfter(created.back());
    Value total = rb.create<AffineLoadOp>(loc, treeCell, ValueRange({zeroIdx})).getResult();
    partialLoad.getResult().replaceUsesWithIf(total, [&](Operation* user) {
      return user->getKind() != OpKind::AffineStore || AffineStoreOp(user).getMemRef() != shared;
    });
    return;
  }
  rb.create<gpu::BarrierOp>(loc);
  Value zero = rb.create<arith::ConstantOp>(loc, rb.getFloatAttr(element, 0)).getResult();
  auto total = rb.create<AffineForOp>(loc, 0, tpr, 1, ValueRange({zero}),
    [&](OpBuilder& lb, Location lloc, Value j, ValueRange iterArgs) {
      Value p = lb.create<AffineLoadOp>(lloc, shared, ValueRange({j})).getResult();
      Value s = lb.create<arith::AddFOp>(lloc, p, iterArgs[0]).getResult();
      lb.create<AffineYieldOp>(lloc, ValueRange({s}));
    });
  // every later user of the partial uses the total (the store that publishes it keeps the partial)
  partialLoad.getResult().replaceUsesWithIf(total.getResult(0), [&](Operation* user) {
    return user->getKind() != OpKind::AffineStore || AffineStoreOp(user).getMemRef() != shared;
  });
}


}  // namespace

bool ElementWiseOptimizer::applicable(ModuleOp& module) {
  clear();
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "Elementwise")) {
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;
    if (f.getNumArguments() != 1) continue;
    auto loops = Analyzer::collectFuncLoops(f);
    auto inType = f.getArgument(0).getType().cast<MemRefType>();
    if ((int64_t)loops.size() != inType.getRank() || loops.empty()) continue;
    if (!configMatchesType(elementWiseConfig, inType.getElementType())) continue;
    elementWises.insert(f);
    elementWiseLoops[f] = loops;
    MemoryBuffer buf;
    buf.input = f.getArgument(0);
    buf.output = f.front().back().getOperand(0);
    elementWiseBuffers[f] = buf;
    any = true;
  }
  return any;
}

AffineMap ElementWiseOptimizer::getAffineMap(const std::string& id, OpBuilder&, const std::vector<int64_t>& extras) {
  // (blockIdx.y, blockIdx.x, threadIdx.y, threadIdx.x, row in thread tile, vector in thread tile) -> (y, x) of the 2-d view;
  // extras = {BLOCK_SIZE_M, BLOCK_SIZE_N, THREAD_SIZE_M, THREAD_SIZE_N, width}
  assert(extras.size() == 5 && (id == "load" || id == "store"));
  auto d = [](unsigned i) { return getAffineDimExpr(i); };
  AffineExpr y = d(0) * extras[0] + d(2) * extras[2] + d(4);
  AffineExpr x = d(1) * extras[1] + d(3) * extras[3] + d(5) * extras[4];
  return AffineMap::get(6, 0, ArrayRef<AffineExpr>({y, x}));
}

void ElementWiseOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : elementWises) {
    auto loops = elementWiseLoops[f];
    auto& buf = elementWiseBuffers[f];
    auto inType = buf.input.getType().cast<MemRefType>();
    auto outType = buf.output.getType().cast<MemRefType>();

    // N-d nest -> near-square 2-d nest
    auto two = Rewriter::combineToTowDim(loops);
    const int64_t dimY = two[0].getConstantUpperBound(), dimX = two[1].getConstantUpperBound();
    DUMP(module);

    // tile sizes: the configured ones, shrunk to divisors of the 2-d extents
    int64_t width = cfg(elementWiseConfig, "VECTORIZE_WIDTH", 4);
    if (inType.getShape().back() % width || dimX % width || inType.getElementType().getIntOrFloatBitWidth() != 32 ||
        outType.getElementType().getIntOrFloatBitWidth() != 32)
      width = 1;
    int64_t tsn = largestDivisor(dimX, cfg(elementWiseConfig, "THREAD_SIZE_N", 4), width);
    int64_t tsm = largestDivisor(dimY, cfg(elementWiseConfig, "THREAD_SIZE_M", 4), 1);
    int64_t bsn = largestDivisor(dimX, cfg(elementWiseConfig, "BLOCK_SIZE_N", 64), tsn);
    int64_t bsm = largestDivisor(dimY, cfg(elementWiseConfig, "BLOCK_SIZE_M", 64), tsm);
    // Extents with few divisors (a prime number of rows, say) leave thread tiles of one element, and the block tile
    // then holds one thread per element: no workgroup may exceed 1024 threads, so the larger side of the block gives
    // way to its next smaller divisor until it fits.
    while ((bsm / tsm) * (bsn / tsn) > 1024) {
      if (bsm / tsm >= bsn / tsn) bsm = largestDivisor(dimY, bsm - 1, tsm);
      else bsn = largestDivisor(dimX, bsn - 1, tsn);
    }
    std::map<std::string, int> used = elementWiseConfig;
    used["BLOCK_SIZE_M"] = (int)bsm; used["BLOCK_SIZE_N"] = (int)bsn;
    used["THREAD_SIZE_M"] = (int)tsm; used["THREAD_SIZE_N"] = (int)tsn; used["VECTORIZE_WIDTH"] = (int)width;
    tagFunction(f, "ElementWise", used, builder);

    auto ySplit = Rewriter::split(two[0], 3, {tsm, bsm});
    auto xSplit = Rewriter::split(two[1], 3, {tsn, bsn});
    DUMP(module);
    AffineForOp yOuter = ySplit[0], yMid = ySplit[1], yInner = ySplit[2];
    AffineForOp xOuter = xSplit[0], xMid = xSplit[1], xInner = xSplit[2];
    Rewriter::reorder({yOuter, xOuter, yMid, xMid, yInner, xInner});
    auto gridLevel = Rewriter::parallel({yOuter, xOuter});
    auto blockLevel = Rewriter::parallel({yMid, xMid});
    DUMP(module);

    // constants of the per-element computation move to the start of the thread body
    std::vector<Operation*> constants;
    xInner->walk([&](Operation* o) { if (o->getKind() == OpKind::Constant) constants.push_back(o); }, WalkOrder::PreOrder);
    for (Operation* c : constants) Rewriter::schedule(c, blockLevel, Position::begin);

    // stage one row of the thread tile through registers: vector read, compute, vector write
    if (width > 1) {
      // the existing scalar accesses give the index maps: x index of the thread tile -> vector index * width
      AffineLoadOp load;
      AffineStoreOp store;
      xInner->walk([&](Operation* o) {
        if (o->getKind() == OpKind::AffineLoad && AffineLoadOp(o).getMemRef() == buf.input) load = AffineLoadOp(o);
        if (o->getKind() == OpKind::AffineStore && AffineStoreOp(o).getMemRef() == buf.output) store = AffineStoreOp(o);
      }, WalkOrder::PreOrder);
      assert(load && store);
      auto retarget = [&](AffineMap map, ValueRange operands, SmallVector<Value>& outOperands) {
        // every occurrence of the xInner index becomes (vector index * width); the vector index is the
        // last map input, behind the other operands
        for (Value v : operands)
          if (v != xInner.getInductionVar()) outOperands.push_back(v);
        const unsigned last = (unsigned)outOperands.size();
        SmallVector<AffineExpr> repl;
        unsigned next = 0;
        for (Value v : operands) {
          if (v == xInner.getInductionVar()) repl.push_back(getAffineDimExpr(last) * width);
          else repl.push_back(getAffineDimExpr(next++));
        }
        return map.replaceDimsAndSymbols(repl, {}, last + 1, 0);
      };
      SmallVector<Value> loadOperands, storeOperands;
      AffineMap loadMap = retarget(load.getAffineMap(), load.getMapOperands(), loadOperands);
      AffineMap storeMap = retarget(store.getAffineMap(), store.getMapOperands(), storeOperands);
      Value fragIn = Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {tsn}, inType.getElementType());
      Value fragOut = buf.input == buf.output ? fragIn
                                              : Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {tsn}, outType.getElementType());
      Rewriter::read(buf.input, fragIn, loadMap, loadOperands, width, xInner, Position::before);
      Rewriter::write(fragOut, buf.output, storeMap, storeOperands, width, xInner, Position::after);
      AffineMap point = AffineMap::get(1, 0, getAffineDimExpr(0));
      Rewriter::cache_read(xInner, buf.input, fragIn, point, {xInner.getInductionVar()});
      Rewriter::cache_write(xInner, buf.output, fragOut, point, {xInner.getInductionVar()});
      DUMP(module);
    }
    (void)gridLevel;

    auto trips = [](AffineForOp loop) { return (loop.getConstantUpperBound() - loop.getConstantLowerBound()) / loop.getStep(); };
    Rewriter::unroll(module, [&](AffineForOp loop) -> bool {
      return f->isAncestor(loop) && loop.hasConstantBounds() && trips(loop) < 2;
    });
    Rewriter::unrollAttribute(module, [&](AffineForOp loop) -> bool {
      return f->isAncestor(loop) && loop.hasConstantBounds() && trips(loop) <= 64;
    });
    DUMP(module);
  }
}

// ===========================================================================
// LayerNormOptimizer (reference: Optimizer.cc:1179-1930)
//
// Schedule: one workgroup per normalised group (grid = product of the outer
// dims), TPR threads per group.  Each of the three passes over the group is
// split so that thread t handles elements io*(TPR*VW) + t*VW + ii; the two
// reductions keep a per-thread partial in a register cell, publish it to a
// shared array, and after a barrier every thread adds up all TPR partials in
// the same order, so all threads hold the same mean / variance.
// ===========================================================================
bool LayerNormOptimizer::applicable(ModuleOp& module) {
  clear();
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "LayerNorm")) {
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;
    if (f.getNumArguments() != 3) continue;
    auto inType = f.getArgument(0).getType().cast<MemRefType>();
    if (!configMatchesType(layerNormConfig, inType.getElementType())) continue;
    // outer loops: the chain of single-loop bodies from the function body down
    // to the block that holds the three passes
    std::vector<AffineForOp> outer;
    Block* block = &f.front();
    while (true) {
      std::vector<AffineForOp> here;
      for (auto& op : block->getOperations())
        if (isa<AffineForOp>(op)) here.push_back(AffineForOp(&op));
      if (here.size() == 1 && here[0].getNumIterOperands() == 0) { outer.push_back(here[0]); block = here[0].getBody(); continue; }
      if (here.size() != 3) { outer.clear(); block = nullptr; }
      break;
    }
    if (block && outer.empty()) {
      // normalisation over the whole tensor (axis 0): one group; a loop of one trip around the three passes stands for
      // the loop over the groups
      OpBuilder wb(&f.front().front());
      outer.push_back(wrapBodyInUnitLoop(f, wb));
      block = outer[0].getBody();
    }
    if (!block) {
      llvm::errs() << "LayerNormOptimizer: " << f.getSymName() << " not scheduled: the body is not the three-pass nest\n";
      continue;
    }
    std::vector<std::vector<AffineForOp>> groups{outer};
    for (auto& op : block->getOperations())
      if (isa<AffineForOp>(op)) {
        std::vector<AffineForOp> nest;
        op.walk([&](Operation* o) { if (isa<AffineForOp>(o)) nest.push_back(AffineForOp(o)); }, WalkOrder::PreOrder);
        groups.push_back(nest);
      }
    if (groups.size() != 4 || groups[1][0].getNumIterOperands() != 1 || groups[2][0].getNumIterOperands() != 1 ||
        groups[3][0].getNumIterOperands() != 0)
      continue;
    layerNorms.insert(f);
    layerNormLoops[f] = groups;
    MemoryBuffer buf;
    buf.input = f.getArgument(0);
    buf.scale = f.getArgument(1);
    buf.bias = f.getArgument(2);
    buf.output = f.front().back().getOperand(0);
    layerNormBuffers[f] = buf;
    any = true;
  }
  return any;
}

AffineMap LayerNormOptimizer::getAffineMap(const std::string& id, OpBuilder&, const std::vector<int64_t>& extras) {
  // "element": (chunk start, threadIdx, index in vector) -> position in the group; extras = {width}
  assert(id == "element" && extras.size() == 1);
  return AffineMap::get(3, 0, getAffineDimExpr(0) + getAffineDimExpr(1) * extras[0] + getAffineDimExpr(2));
}

// LayerNorm whose only consumer is a not yet scheduled GELU ElementWise call: the GELU moves
// into the LayerNorm's normalise nest (applied to the value about to be stored), the GELU call
// disappears and the LayerNorm call stands for both.  One kernel, one pass over the tensor
// instead of two.  Returns true when the fusion was done.
static bool fuseFollowingGelu(ModuleOp& module, func::FuncOp f, AffineForOp innermostNormLoop, Value output,
                              OpBuilder& builder) {
  func::CallOp lnCall(nullptr);
  int callsOfF = 0;
  for (auto c : Analyzer::collectFuncCalls(module))
    if (c.getCallee() == f.getName()) {
      lnCall = c;
      ++callsOfF;
    }
  if (callsOfF != 1) return false;
  auto users = lnCall.getResult(0).getUsers();
  if (users.size() != 1) return false;
  auto geluCall = dyn_cast<func::CallOp>(users[0]);
  if (!geluCall || geluCall.getCallee().rfind("Gelu_Elementwise_", 0) != 0) return false;
  auto g = Analyzer::getTargetFunction(module, geluCall.getCallee());
  if (!g || g->getAttr("func.state").s != "cpu") return false;
  if (geluCall.getResult(0).getType() != lnCall.getResult(0).getType()) return false;
  int callsOfG = 0;
  for (auto c : Analyzer::collectFuncCalls(module))
    if (c.getCallee() == g.getName()) ++callsOfG;

  // the store of the normalised value is the last store into the output in the normalise nest
  AffineStoreOp store(nullptr);
  for (auto& op : *innermostNormLoop.getBody())
    if (auto st = dyn_cast<AffineStoreOp>(&op))
      if (st.getMemRef() == output) store = st;
  if (!store) return false;
  OpBuilder b(store->getContext());
  b.setInsertionPoint(store.getOperation());
  Value y = store.getValue();
  Value z = ElementWise::gelu(b, y, y.getType());
  store->setOperand(0, z);

  geluCall.getResult(0).replaceAllUsesWith(lnCall.getResult(0));
  geluCall.erase();
  if (callsOfG == 1) g.erase();
  f->setAttr("kcg.fused_gelu", builder.getI64IntegerAttr(1));
  return true;
}

void LayerNormOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : layerNorms) {
    auto groups = layerNormLoops[f];
    auto& buf = layerNormBuffers[f];
    if (cfg(layerNormConfig, "FUSE_GELU", 1)) fuseFollowingGelu(module, f, groups[3].back(), buf.output, builder);
    auto inType = buf.input.getType().cast<MemRefType>();
    int64_t count = 1;
    for (auto l : groups[1]) count *= l.getConstantUpperBound();

    // threads per group and vector width: configured values shrunk until they tile the group
    int64_t width = cfg(layerNormConfig, "VECTORIZE_WIDTH", 4);
    auto sizeOf = [](Value v) { return v.getType().cast<MemRefType>().getNumElements(); };
    if (count % width || sizeOf(buf.scale) % width || sizeOf(buf.bias) % width || inType.getShape().back() % width) width = 1;
    int64_t tpr = cfg(layerNormConfig, "BLOCK_SIZE", 2048) / std::max(1, cfg(layerNormConfig, "THREAD_SIZE", 4));
    if (cfg(layerNormConfig, "THREADS_PER_ROW", 0) > 0) tpr = cfg(layerNormConfig, "THREADS_PER_ROW");
    while (tpr > 1 && count % (tpr * width)) tpr /= 2;
    std::map<std::string, int> used = layerNormConfig;
    used["THREADS_PER_ROW"] = (int)tpr;
    used["VECTORIZE_WIDTH"] = (int)width;
    tagFunction(f, "LayerNorm", used, builder);

    // rows -> grid
    AffineForOp rowLoop = Rewriter::combineToOneDim(groups[0]);
    AffineForOp sumLoop = Rewriter::combineToOneDim(groups[1]);
    AffineForOp varLoop = Rewriter::combineToOneDim(groups[2]);
    AffineForOp normLoop = Rewriter::combineToOneDim(groups[3]);
    DUMP(module);
    AffineParallelOp gridLevel = Rewriter::parallel({rowLoop});

    // thread level around the whole body of the group
    OpBuilder b = OpBuilder::atBlockBegin(gridLevel.getBody());
    Operation* firstOld = &gridLevel.getBody()->front();
    AffineParallelOp blockLevel = b.create<AffineParallelOp>(b.getUnknownLoc(), std::vector<int64_t>{0}, std::vector<int64_t>{tpr});
    (void)firstOld;
    {
      Operation* op = blockLevel->getNextNode();
      while (op && op->getKind() != OpKind::AffineYield) {
        Operation* next = op->getNextNode();
        op->moveBefore(blockLevel.getBody()->getTerminator());
        op = next;
      }
    }
    Value tid = blockLevel.getIVs()[0];
    Type element = inType.getElementType();
    Value red1 = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {tpr}, element);
    Value red2 = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {tpr}, element);
    DUMP(module);

    // TREE_REDUCE: the reference's tree over the partials (needs whole wavefronts and a power of two)
    const bool tree = cfg(layerNormConfig, "TREE_REDUCE", 0) && tpr >= 64 && (tpr & (tpr - 1)) == 0;
    auto scheduleReduction = [&](AffineForOp loop, Value shared) {
      if (!tree) return scheduleTeamReduction(loop, shared, tid, width, tpr, element);
      Value cell = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {1}, element);
      scheduleTeamReduction(loop, shared, tid, width, tpr, element, blockLevel, cell);
    };
    scheduleReduction(sumLoop, red1);
    DUMP(module);
    scheduleReduction(varLoop, red2);
    DUMP(module);
    auto normParts = Rewriter::split(normLoop, 3, {width, tpr * width});
    bindLoopToThread(normParts[1], tid);
    DUMP(module);

    auto trips = [](AffineForOp loop) { return (loop.getConstantUpperBound() - loop.getConstantLowerBound()) / loop.getStep(); };
    Rewriter::unrollAttribute(module, [&](AffineForOp loop) -> bool {
      return f->isAncestor(loop) && loop.hasConstantBounds() && trips(loop) <= 16;
    });
    DUMP(module);
  }
}

// ===========================================================================
// SoftmaxOptimizer: a Softmax call that no attention fusion has taken (the reference schedules
// softmax only inside its fused attention, Optimizer.cc:2113-2860, and has no class for it).
// Nest (Operators.cc:462-578): outer loops over the leading dimensions; a loop that sums exp(x)
// over the row; a loop that stores exp(x) / sum back in place.  Schedule, like LayerNorm's:
// rows -> grid, a team of threads per row, the sum through per-thread partials and a shared cell
// per thread, the second loop dealt over the team.
// ===========================================================================
bool SoftmaxOptimizer::applicable(ModuleOp& module) {
  clear();
  std::set<std::string> called;
  for (auto call : Analyzer::collectFuncCalls(module)) called.insert(call.getCallee());
  bool any = false;
  for (auto f : Analyzer::collectFunctions(module, "Softmax_")) {
    const std::string name = f.getSymName();
    if (name.rfind("Softmax_", 0) != 0 || !called.count(name)) continue;
    auto state = f->getAttr("func.state");
    if (state && state.s != "cpu") continue;
    if (f.getNumArguments() != 1) continue;
    auto type = f.getArgument(0).getType().cast<MemRefType>();
    const Type elem = type.getElementType();
    if ((!elem.isF32() && !elem.isF16() && !elem.isF64() && !elem.isBF16()) || type.getRank() < 1) continue;
    // outer perfect nest of rank-1 loops, then exactly two row loops: the sum (one carried value) and the store
    std::vector<AffineForOp> outer;
    Block* body = &f.front();
    bool ok = true;
    for (int64_t d = 0; d + 1 < type.getRank() && ok; ++d) {
      AffineForOp loop;
      for (auto& op : body->getOperations())
        if (auto l = dyn_cast<AffineForOp>(op)) { if (loop) ok = false; loop = l; }
      if (!loop || !loop.hasConstantBounds() || loop.getNumIterOperands() != 0) { ok = false; break; }
      outer.push_back(loop);
      body = loop.getBody();
    }
    if (!ok) continue;
    std::vector<AffineForOp> rowLoops;
    for (auto& op : body->getOperations())
      if (auto l = dyn_cast<AffineForOp>(op)) rowLoops.push_back(l);
    if (rowLoops.size() != 2 || rowLoops[0].getNumIterOperands() != 1 || rowLoops[1].getNumIterOperands() != 0) continue;
    softmaxes.insert(f);
    softmaxLoops[f] = {outer, {rowLoops[0]}, {rowLoops[1]}};
    any = true;
  }
  return any;
}

void SoftmaxOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto f : softmaxes) {
    auto groups = softmaxLoops[f];
    auto type = f.getArgument(0).getType().cast<MemRefType>();
    const int64_t count = type.getShape().back();
    int64_t width = cfg(softmaxConfig, "VECTORIZE_WIDTH", 4);
    if (width < 1 || count % width) width = 1;
    int64_t tpr = cfg(softmaxConfig, "BLOCK_SIZE", 1024) / std::max(1, cfg(softmaxConfig, "THREAD_SIZE", 4));
    if (cfg(softmaxConfig, "THREADS_PER_ROW", 0) > 0) tpr = cfg(softmaxConfig, "THREADS_PER_ROW");
    while (tpr > 1 && count % (tpr * width)) tpr /= 2;
    std::map<std::string, int> used = softmaxConfig;
    used["THREADS_PER_ROW"] = (int)tpr;
    used["VECTORIZE_WIDTH"] = (int)width;
    tagFunction(f, "Softmax", used, builder);

    // a vector is a single row: a loop of one trip around the whole body stands for the loop over the rows
    if (groups[0].empty()) groups[0].push_back(wrapBodyInUnitLoop(f, builder));
    AffineForOp rowLoop = Rewriter::combineToOneDim(groups[0]);
    AffineForOp sumLoop = groups[1][0], storeLoop = groups[2][0];
    DUMP(module);
    AffineParallelOp gridLevel = Rewriter::parallel({rowLoop});
    // thread level around the whole body of the row
    OpBuilder b = OpBuilder::atBlockBegin(gridLevel.getBody());
    AffineParallelOp blockLevel = b.create<AffineParallelOp>(b.getUnknownLoc(), std::vector<int64_t>{0}, std::vector<int64_t>{tpr});
    {
      Operation* op = blockLevel->getNextNode();
      while (op && op->getKind() != OpKind::AffineYield) {
        Operation* next = op->getNextNode();
        op->moveBefore(blockLevel.getBody()->getTerminator());
        op = next;
      }
    }
    Value tid = blockLevel.getIVs()[0];
    Type element = type.getElementType();
    Value red = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {tpr}, element);
    DUMP(module);
    if (cfg(softmaxConfig, "TREE_REDUCE", 0) && tpr >= 64 && (tpr & (tpr - 1)) == 0) {
      Value cell = Rewriter::alloc_buffer(gridLevel, MemorySpace::shared, {1}, element);
      scheduleTeamReduction(sumLoop, red, tid, width, tpr, element, blockLevel, cell);
    } else {
      scheduleTeamReduction(sumLoop, red, tid, width, tpr, element);
    }
    DUMP(module);
    // a thread stores exactly the elements its own partial sum read, so the in-place update needs no further barrier
    auto parts = Rewriter::split(storeLoop, 3, {width, tpr * width});
    bindLoopToThread(parts[1], tid);
    DUMP(module);
    auto trips = [](AffineForOp loop) { return (loop.getConstantUpperBound() - loop.getConstantLowerBound()) / loop.getStep(); };
    Rewriter::unrollAttribute(module, [&](AffineForOp loop) -> bool {
      return f->isAncestor(loop) && loop.hasConstantBounds() && trips(loop) <= 16;
    });
    DUMP(module);
  }
}

}  // namespace KernelCodeGen

// ===========================================================================
// FMHAOptimizer (reference: Optimizer.cc:2113-2860)
//
// Matches BatchMatmul(Q, K^T) -> Softmax -> BatchMatmul(P, V) with single-use
// intermediate results and replaces the three calls by one call of a fused
// function Fused_Multi_Head_Attention_<b>_<h>_SL<S>_HD<D>(Q, K, V, O) that never
// materialises the S x S matrix.  Two schedules of the fused function:
//
//  * the reference's tiled one (buildTiledSchedule; Optimizer.cc:2606-2860, structure fixture doc/pass.md:136-405),
//    taken for fp32 graphs when the config carries its keys (Slice, Width, BrTileS, BcTileS, BrTileO, HdTileO, WarpX_O,
//    WARP_SIZE, BLOCK_SIZE = threads, HdxBr, BrxBc) and the shape fits its layout rules (tiledLayout): grid
//    (batch, head, S / Br), Q / K / V slices and the probabilities staged in shared memory, 8 x 8 register tiles fed
//    by outer products, the online softmax of softmaxIR with wavefront shuffles;
//  * one query row per thread (everything else: 16-bit graphs, ragged sequence lengths, a config without those
//    keys): grid (batch, head, S / Br), Br threads, a loop over the keys with the running maximum, running sum and
//    the output row rescaled on the fly.
// The reference's text has slips that its own fixture shows: the row pass of the softmax stores the sum into the
// maximum (Optimizer.cc:2500-2501), the running sum is rescaled by the wrong factor (:2543-2544), the output store
// uses blockIdx.z as the thread id (:2415), the probability tile is allocated [Br][Bc] and indexed [bc][br] (:2695),
// the V slice [Slice][Bc] and indexed [.][hd] (:2694), applicable() has no return.  None is reproduced; both schedules
// are checked against the three unfused nests on the host interpreter (with its barrier audit) and on the device.
// Config beyond the reference's: SCALE_RSQRT_D = 1 multiplies the scores by 1/sqrt(D); CAUSAL = 1 keeps keys j <= i;
// ROW_BLOCK_SIZE = queries per workgroup of the row-per-thread form when BLOCK_SIZE means the tiled form's threads.
// ===========================================================================
namespace KernelCodeGen {

using namespace mlir;

// Queries per workgroup of the row-per-thread form.
int FMHAOptimizer::rowBlockSize() {
  if (fmhaConfig.count("Slice") && fmhaConfig["Slice"] > 0)       // BLOCK_SIZE is the tiled form's thread count then
    return fmhaConfig.count("ROW_BLOCK_SIZE") ? fmhaConfig["ROW_BLOCK_SIZE"] : 256;
  return fmhaConfig.count("BLOCK_SIZE") ? fmhaConfig["BLOCK_SIZE"] : 128;
}

bool FMHAOptimizer::tiledLayout(int64_t seq, int64_t hd, int64_t& br, int64_t& bc, std::string* why) {
  auto no = [&](const std::string& text) { if (why) *why = text; return false; };
  auto cfg = [&](const char* key) -> int64_t { return fmhaConfig.count(key) ? fmhaConfig[key] : 0; };
  const int64_t threads = cfg("BLOCK_SIZE"), slice = cfg("Slice"), width = cfg("Width"), warp = cfg("WARP_SIZE");
  const int64_t brS = cfg("BrTileS"), bcS = cfg("BcTileS"), brO = cfg("BrTileO"), hdO = cfg("HdTileO"), warpX = cfg("WarpX_O");
  for (int64_t v : {threads, slice, width, warp, brS, bcS, brO, hdO, warpX, cfg("HdxBr"), cfg("BrxBc")})
    if (v <= 0) return no("a key of the tiled schedule is missing from the config");
  if (hd <= 0 || cfg("HdxBr") % hd) return no("HdxBr is no multiple of the head dim");
  br = cfg("HdxBr") / hd;
  if (br <= 0 || cfg("BrxBc") % br) return no("BrxBc is no multiple of Br");
  bc = cfg("BrxBc") / br;
  if (seq % br || seq % bc) return no("the sequence length is no multiple of Br and Bc");
  if (hd % slice || bc % slice || slice % width) return no("Slice must divide Hd and Bc, Width must divide Slice");
  if (threads % warp) return no("BLOCK_SIZE is no multiple of WARP_SIZE");
  // every thread copies whole Width-vectors, the same number each
  for (int64_t elems : {slice * br, slice * bc, slice * hd})
    if (elems % (threads * width)) return no("a slice does not split into Width-vectors over the threads");
  if (hd % width) return no("Width must divide the head dim");
  // the score tile [Bc][Br] over the threads
  if (threads * brS * bcS != br * bc || brS % width || bcS % width || bc % bcS) return no("BrTileS x BcTileS tiles do not cover the score tile");
  const int64_t laneXS = bc / bcS;
  if (laneXS > 64 || (laneXS & (laneXS - 1)) || warp % laneXS) return no("Bc / BcTileS must be a power of two that divides WARP_SIZE");
  if ((threads / warp) * (warp / laneXS) * brS != br) return no("the warps' score rows do not add up to Br");
  // the output tile [Br][Hd]
  if (threads * brO * hdO != br * hd || brO % width || hdO % width || hd % (hdO * warpX)) return no("BrTileO x HdTileO tiles do not cover the output tile");
  const int64_t laneXO = hd / hdO / warpX;
  if (laneXO <= 0 || warp % laneXO || (threads / warp) % warpX) return no("the output tile's lanes and warps do not fit WARP_SIZE / WarpX_O");
  if ((threads / warp / warpX) * (warp / laneXO) * brO != br) return no("the warps' output rows do not add up to Br");
  return true;
}

// The reference's tiled attention schedule (src/Optimizer/Optimizer.cc:2606-2860), scripted with the same Rewriter
// primitives in the same order, its slips repaired (see the head of this section).  fp32 throughout.
void FMHAOptimizer::buildTiledSchedule(func::FuncOp funcOp, OpBuilder& builder, int64_t batch, int64_t heads, int64_t seq_len,
                                       int64_t head_dim, bool causal, bool scaled) {
  OpBuilder::InsertionGuard whole(builder);
  Location loc = builder.getUnknownLoc();
  Block& body = funcOp.front();
  Value Q = body.getArgument(0), K = body.getArgument(1), V = body.getArgument(2), O = body.getArgument(3);
  Type elementType = Q.getType().cast<MemRefType>().getElementType();
  builder.setInsertionPointToStart(&body);
  auto returnOp = builder.create<func::ReturnOp>(loc, ValueRange({O}));
  builder.setInsertionPoint(returnOp.getOperation());

  int64_t Br = 0, Bc = 0;
  const bool fits = tiledLayout(seq_len, head_dim, Br, Bc);
  assert(fits && "buildTiledSchedule: the caller checks the layout");
  (void)fits;
  const int64_t Hd = head_dim, Slice = fmhaConfig["Slice"], BLOCK_SIZE = fmhaConfig["BLOCK_SIZE"], Width = fmhaConfig["Width"];
  fmhaConfig["Hd"] = (int)Hd;
  fmhaConfig["Br"] = (int)Br;
  fmhaConfig["Bc"] = (int)Bc;
  const int64_t BrTileS = fmhaConfig["BrTileS"], BcTileS = fmhaConfig["BcTileS"], BrTileO = fmhaConfig["BrTileO"], HdTileO = fmhaConfig["HdTileO"];

  std::vector<int64_t> bounds{batch, heads, seq_len / Br, BLOCK_SIZE};
  buildAffineLoopNest(builder, loc, std::vector<int64_t>(4, 0), bounds, std::vector<int64_t>(4, 1),
                      [&](OpBuilder&, Location, ValueRange) {});
  auto loops = Analyzer::collectFuncLoops(funcOp);
  auto gridLevel = Rewriter::parallel({loops[0], loops[1], loops[2]});
  auto blockLevel = Rewriter::parallel({loops[3]});
  funcOp->setAttr("func.state", builder.getStringAttr("gpu"));
  Value bz = gridLevel.getIVs()[0], by = gridLevel.getIVs()[1], bx = gridLevel.getIVs()[2], tid = blockLevel.getIVs()[0];

  // shared tiles: a slice of Q, K (both stored transposed: [d][row]) and V, the probabilities [key][query], the
  // running statistics per query
  Value smQ = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Slice, Br}, elementType);
  Value smK = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Slice, Bc}, elementType);
  Value smV = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Slice, Hd}, elementType);
  Value smP = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Bc, Br}, elementType);
  Value smMax = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Br}, elementType);
  Value smSum = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Br}, elementType);
  Value smFac = Rewriter::alloc_buffer(blockLevel, MemorySpace::shared, {Br}, elementType);
  Value tileO = Rewriter::alloc_buffer(blockLevel, MemorySpace::local, {BrTileO, HdTileO}, elementType);

  builder.setInsertionPointAfter(Analyzer::getLastOp<memref::AllocOp>(blockLevel).getOperation());
  Value zero = builder.create<arith::ConstantOp>(loc, builder.getFloatAttr(elementType, 0)).getResult();
  Value flt_min = builder.create<arith::ConstantOp>(loc, builder.getFloatAttr(elementType, -FLT_MAX)).getResult();
  Value scale;
  if (scaled) scale = builder.create<arith::ConstantOp>(loc, builder.getFloatAttr(elementType, 1.0 / std::sqrt((double)Hd))).getResult();
  Rewriter::set_buffer(builder, tileO, zero);

  AffineExpr d0 = getAffineDimExpr(0), d1 = getAffineDimExpr(1);
  // running sum 0, running maximum the most negative finite value; thread tid takes queries tid, tid + BLOCK_SIZE, ...
  {
    auto init = Rewriter::create_constant_loop(builder, 0, Br, BLOCK_SIZE);
    OpBuilder ib = OpBuilder::atBlockBegin(init.getBody());
    auto inRange = IntegerSet::get(2, 0, ArrayRef<AffineExpr>((Br - 1) - d0 - d1), ArrayRef<bool>(false));
    auto ifOp = ib.create<AffineIfOp>(loc, inRange, ValueRange({tid, init.getInductionVar()}), false);
    OpBuilder tb(ifOp.getThenBlock()->getTerminator());
    AffineMap at = AffineMap::get(2, 0, ArrayRef<AffineExpr>(d0 + d1));
    tb.create<AffineStoreOp>(loc, zero, smSum, at, ValueRange({tid, init.getInductionVar()}));
    tb.create<AffineStoreOp>(loc, flt_min, smMax, at, ValueRange({tid, init.getInductionVar()}));
    builder.setInsertionPointAfter(init.getOperation());
  }

  auto outer_reduce = Rewriter::create_constant_loop(builder, 0, seq_len, Bc);
  Value kv = outer_reduce.getInductionVar();
  builder.setInsertionPointToStart(outer_reduce.getBody());
  if (causal) {
    // a key tile that starts behind the workgroup's last query concerns none of its threads: the same decision in
    // every thread, so the barriers inside are reached by all of them or by none
    auto set = IntegerSet::get(2, 0, ArrayRef<AffineExpr>(d0 * Br + (Br - 1) - d1), ArrayRef<bool>(false));
    auto ifOp = builder.create<AffineIfOp>(loc, set, ValueRange({bx, kv}), false);
    builder.setInsertionPoint(ifOp.getThenBlock()->getTerminator());
  }
  // everything below is built in program order at the builder's position (inside the key-tile loop)
  Value ldgQ = builder.create<memref::AllocOp>(loc, MemRefType::get({Slice * Br / BLOCK_SIZE}, elementType, {}, (int)MemorySpace::local)).getResult();
  Value ldgK = builder.create<memref::AllocOp>(loc, MemRefType::get({Slice * Bc / BLOCK_SIZE}, elementType, {}, (int)MemorySpace::local)).getResult();
  Value tileS = builder.create<memref::AllocOp>(loc, MemRefType::get({BcTileS, BrTileS}, elementType, {}, (int)MemorySpace::local)).getResult();
  Rewriter::set_buffer(builder, tileS, zero);

  // ---- S^T = K Q^T, a slice of the head dim at a time ----
  {
    auto hd_outer = Rewriter::create_constant_loop(builder, 0, Hd, Slice);
    auto bar1 = Rewriter::barrier(hd_outer, Position::begin);
    OpBuilder hb(hd_outer.getBody()->getTerminator());
    (void)bar1;
    Rewriter::read(hb, Q, ldgQ, getAffineMap("loadTileQ", hb), {bz, by, bx, tid, hd_outer.getInductionVar()}, Width);
    Rewriter::read(hb, K, ldgK, getAffineMap("loadTileK", hb), {bz, by, tid, kv, hd_outer.getInductionVar()}, Width);
    Rewriter::write(hb, ldgQ, smQ, getAffineMap("storeTileQ", hb), {tid}, Width);
    auto writeSmK = Rewriter::write(hb, ldgK, smK, getAffineMap("storeTileK", hb), {tid}, Width);
    auto bar2 = Rewriter::barrier(writeSmK, Position::after);
    Value fragQ = Rewriter::alloc_buffer(bar2, Position::after, MemorySpace::local, {BrTileS}, elementType);
    Value fragK = Rewriter::alloc_buffer(fragQ.getDefiningOp<memref::AllocOp>(), Position::after, MemorySpace::local, {BcTileS}, elementType);
    auto hd_inner = Rewriter::create_constant_loop(hb, 0, Slice, 1);
    OpBuilder ib(hd_inner.getBody()->getTerminator());
    Rewriter::read(ib, smQ, fragQ, getAffineMap("loadFragQ", ib), {tid, hd_inner.getInductionVar()}, Width);
    Rewriter::read(ib, smK, fragK, getAffineMap("loadFragK", ib), {tid, hd_inner.getInductionVar()}, Width);
    Rewriter::outer_product(ib, tileS, fragK, fragQ, BcTileS, BrTileS);
    builder.setInsertionPointAfter(hd_outer.getOperation());
  }
  // ---- scale and mask (not in the reference, whose attention has neither) ----
  if (scaled || causal) {
    auto outer = Rewriter::create_constant_loop(builder, 0, BcTileS, 1);
    OpBuilder ob(outer.getBody()->getTerminator());
    auto inner = Rewriter::create_constant_loop(ob, 0, BrTileS, 1);
    OpBuilder ib(inner.getBody()->getTerminator());
    Value c = outer.getInductionVar(), r = inner.getInductionVar();
    if (scaled) {
      Value s = ib.create<AffineLoadOp>(loc, tileS, ValueRange({c, r})).getResult();
      ib.create<AffineStoreOp>(loc, ib.create<arith::MulFOp>(loc, s, scale).getResult(), tileS, ValueRange({c, r}));
    }
    if (causal) {
      // (kv, tid, bc, bx, br): key kv + bcIdxS(tid, bc) lies behind query bx * Br + brIdxS(tid, br)
      AffineExpr key = getAffineMap("bcIdxS", ib).getResult(0).replaceDims({getAffineDimExpr(1), getAffineDimExpr(2)}) + d0;
      AffineExpr query = getAffineMap("brIdxS", ib).getResult(0).replaceDims({getAffineDimExpr(1), getAffineDimExpr(4)}) + getAffineDimExpr(3) * Br;
      auto behind = IntegerSet::get(5, 0, ArrayRef<AffineExpr>(key - query - 1), ArrayRef<bool>(false));
      auto ifOp = ib.create<AffineIfOp>(loc, behind, ValueRange({kv, tid, c, bx, r}), false);
      OpBuilder tb(ifOp.getThenBlock()->getTerminator());
      tb.create<AffineStoreOp>(loc, flt_min, tileS, ValueRange({c, r}));
    }
    builder.setInsertionPointAfter(outer.getOperation());
  }
  // ---- online softmax of the tile; probabilities to shared memory ----
  Value rowMax = builder.create<memref::AllocOp>(loc, MemRefType::get({BrTileS}, elementType, {}, (int)MemorySpace::local)).getResult();
  Value rowSum = builder.create<memref::AllocOp>(loc, MemRefType::get({BrTileS}, elementType, {}, (int)MemorySpace::local)).getResult();
  softmaxIR(builder, tileS, rowMax, smMax, rowSum, smSum, smFac, zero, flt_min, tid);
  AffineForOp storeP = Rewriter::create_constant_loop(builder, 0, BcTileS, 1);
  {
    OpBuilder ob(storeP.getBody()->getTerminator());
    auto inner = Rewriter::create_constant_loop(ob, 0, BrTileS, Width);
    OpBuilder ib(inner.getBody()->getTerminator());
    Value c = storeP.getInductionVar(), r = inner.getInductionVar();
    auto vectorType = VectorType::get(Width, elementType);
    Value p = ib.create<AffineVectorLoadOp>(loc, vectorType, tileS, getAffineMap("readTileS", ib), ValueRange({c, r})).getResult();
    ib.create<AffineVectorStoreOp>(loc, p, smP, getAffineMap("storeTileP", ib), ValueRange({tid, c, r}));
  }
  auto bar3 = Rewriter::barrier(storeP, Position::after);
  // ---- O = factor * O + P V ----
  Value factor = Rewriter::alloc_buffer(bar3, Position::after, MemorySpace::local, {BrTileO}, elementType);
  builder.setInsertionPointAfter(factor.getDefiningOp());
  Rewriter::read(builder, smFac, factor, getAffineMap("loadFactor", builder), {tid}, Width);
  auto perElementOfO = [&](Value perRow, bool divide) {
    auto outer = Rewriter::create_constant_loop(builder, 0, BrTileO, 1);
    OpBuilder ob(outer.getBody()->getTerminator());
    auto inner = Rewriter::create_constant_loop(ob, 0, HdTileO, 1);
    OpBuilder ib(inner.getBody()->getTerminator());
    Value r = outer.getInductionVar(), d = inner.getInductionVar();
    Value o = ib.create<AffineLoadOp>(loc, tileO, ValueRange({r, d})).getResult();
    Value f = ib.create<AffineLoadOp>(loc, perRow, ValueRange({r})).getResult();
    Value res = divide ? ib.create<arith::DivFOp>(loc, o, f).getResult() : ib.create<arith::MulFOp>(loc, o, f).getResult();
    ib.create<AffineStoreOp>(loc, res, tileO, ValueRange({r, d}));
    builder.setInsertionPointAfter(outer.getOperation());
  };
  perElementOfO(factor, false);
  {
    auto bc_outer = Rewriter::create_constant_loop(builder, 0, Bc, Slice);
    Value ldgV = Rewriter::alloc_buffer(bc_outer, Position::before, MemorySpace::local, {Slice * Hd / BLOCK_SIZE}, elementType);
    auto bar4 = Rewriter::barrier(bc_outer, Position::begin);
    (void)bar4;
    OpBuilder vb(bc_outer.getBody()->getTerminator());
    Rewriter::read(vb, V, ldgV, getAffineMap("loadTileV", vb), {bz, by, tid, kv, bc_outer.getInductionVar()}, Width);
    auto writeSmV = Rewriter::write(vb, ldgV, smV, getAffineMap("storeTileV", vb), {tid}, Width);
    auto bar5 = Rewriter::barrier(writeSmV, Position::after);
    Value fragP = Rewriter::alloc_buffer(bar5, Position::after, MemorySpace::local, {BrTileO}, elementType);
    Value fragV = Rewriter::alloc_buffer(fragP.getDefiningOp<memref::AllocOp>(), Position::after, MemorySpace::local, {HdTileO}, elementType);
    auto bc_inner = Rewriter::create_constant_loop(vb, 0, Slice, 1);
    OpBuilder ib(bc_inner.getBody()->getTerminator());
    Rewriter::read(ib, smP, fragP, getAffineMap("loadFragP", ib), {tid, bc_outer.getInductionVar(), bc_inner.getInductionVar()}, Width);
    Rewriter::read(ib, smV, fragV, getAffineMap("loadFragV", ib), {tid, bc_inner.getInductionVar()}, Width);
    Rewriter::outer_product(ib, tileO, fragP, fragV, BrTileO, HdTileO);
  }

  // ---- after the last key tile: O / running sum, to global memory ----
  Value rowSumO = Rewriter::alloc_buffer(outer_reduce, Position::after, MemorySpace::local, {BrTileO}, elementType);
  builder.setInsertionPointAfter(rowSumO.getDefiningOp());
  Rewriter::read(builder, smSum, rowSumO, getAffineMap("brIdxO", builder), {tid}, Width);
  perElementOfO(rowSumO, true);
  {
    auto outer = Rewriter::create_constant_loop(builder, 0, BrTileO, 1);
    OpBuilder ob(outer.getBody()->getTerminator());
    auto inner = Rewriter::create_constant_loop(ob, 0, HdTileO, Width);
    OpBuilder ib(inner.getBody()->getTerminator());
    Value r = outer.getInductionVar(), d = inner.getInductionVar();
    auto vectorType = VectorType::get(Width, elementType);
    Value o = ib.create<AffineVectorLoadOp>(loc, vectorType, tileO, ValueRange({r, d})).getResult();
    ib.create<AffineVectorStoreOp>(loc, o, O, getAffineMap("storeTileO", ib), ValueRange({bz, by, bx, tid, r, d}));
  }
  std::map<std::string, int> used = fmhaConfig;
  used["CAUSAL"] = causal;
  used["SCALE_RSQRT_D"] = scaled;
  used["TILED"] = 1;
  tagFunction(funcOp, "FMHA", used, builder);
}

bool FMHAOptimizer::applicable(ModuleOp& module) {
  clear();
  auto calls = Analyzer::collectFuncCalls(module);
  auto stateOf = [&](const std::string& name) {
    auto f = Analyzer::getTargetFunction(module, name);
    return f ? f->getAttr("func.state").s : std::string();
  };
  for (auto first : calls) {
    BatchMatmulDescriptor m1, m2;
    if (!identifyBatchMatmul(first.getCallee(), m1) || m1.transA || !m1.transB) continue;
    if (stateOf(first.getCallee()) != "cpu") continue;
    Value s = first.getResult(0);
    auto sUsers = s.getUsers();
    if (sUsers.size() != 1) continue;
    auto softmax = dyn_cast<func::CallOp>(sUsers[0]);
    if (!softmax || softmax.getCallee().rfind("Softmax", 0) != 0 || stateOf(softmax.getCallee()) != "cpu") continue;
    Value p = softmax.getResult(0);
    auto pUsers = p.getUsers();
    if (pUsers.size() != 1) continue;
    auto second = dyn_cast<func::CallOp>(pUsers[0]);
    if (!second || !identifyBatchMatmul(second.getCallee(), m2) || m2.transA || m2.transB) continue;
    if (stateOf(second.getCallee()) != "cpu" || second.getOperand(0) != p) continue;
    // Q [b.., S, D] x K [b.., S, D]^T -> S [b.., S, S];  P x V [b.., S, D] -> O [b.., S, D]
    if (m1.batch != m2.batch || m1.batch.size() != 2 || m1.m != m1.n || m2.m != m1.m || m2.k != m1.n || m2.n != m1.k) continue;
    if (uniqueFuncCalls.count(first)) continue;
    const int br = rowBlockSize();
    // A sequence length that BLOCK_SIZE does not divide gets one more, partly filled workgroup whose surplus threads
    // do nothing (RAGGED = 0 leaves such a graph unfused, as the reference's full-tile schedule would).
    const bool raggedOk = !fmhaConfig.count("RAGGED") || fmhaConfig["RAGGED"];
    if (br <= 0 || (m1.m % br && !raggedOk)) {
      llvm::errs() << "FMHAOptimizer: sequence length " << m1.m << " is not a multiple of BLOCK_SIZE " << br << "\n";
      continue;
    }
    uniqueFuncCalls.insert(first);
    call2callsMap[first] = {softmax, second};
    MemoryBuffer buf;
    buf.Q = first.getOperand(0);
    buf.K = first.getOperand(1);
    buf.S = first.getOperand(2);
    buf.V = second.getOperand(1);
    buf.O = second.getOperand(2);
    buf.matmul1 = m1;
    buf.matmul2 = m2;
    call2bufferMap[first] = buf;
  }
  return !uniqueFuncCalls.empty();
}

void FMHAOptimizer::applyOptimzer(ModuleOp& module, OpBuilder& builder) {
  for (auto first : uniqueFuncCalls) {
    auto& buf = call2bufferMap[first];
    func::CallOp softmax = call2callsMap[first][0], second = call2callsMap[first][1];
    const int64_t batch = buf.matmul1.batch[0], heads = buf.matmul1.batch[1], seq = buf.matmul1.m, hd = buf.matmul1.k;
    const int64_t br = rowBlockSize();
    const bool causal = fmhaConfig.count("CAUSAL") && fmhaConfig["CAUSAL"];
    const bool scaled = fmhaConfig.count("SCALE_RSQRT_D") && fmhaConfig["SCALE_RSQRT_D"];
    auto typeQ = buf.Q.getType().cast<MemRefType>(), typeK = buf.K.getType().cast<MemRefType>();
    auto typeV = buf.V.getType().cast<MemRefType>(), typeO = buf.O.getType().cast<MemRefType>();
    Type f32 = builder.getF32Type();

    std::string name = "Fused_Multi_Head_Attention_" + std::to_string(batch) + "_" + std::to_string(heads) + "_SL" +
                       std::to_string(seq) + "_HD" + std::to_string(hd);
    if (causal) name += "_causal";
    if (scaled) name += "_scaled";
    auto ip = builder.saveInsertionPoint();
    auto funcOp = buildFuction(module, builder, name, {typeQ, typeK, typeV, typeO}, {typeO});
    Block& body = funcOp.front();
    int64_t tiledBr = 0, tiledBc = 0;
    std::string whyNot;
    const bool wantTiled = fmhaConfig.count("Slice") && fmhaConfig["Slice"] > 0 && (!fmhaConfig.count("TILED") || fmhaConfig["TILED"]);
    const bool allF32 = typeQ.getElementType().isF32() && typeK.getElementType().isF32() && typeV.getElementType().isF32() &&
                        typeO.getElementType().isF32();
    if (body.empty() && wantTiled && allF32 && tiledLayout(seq, hd, tiledBr, tiledBc, &whyNot)) {
      buildTiledSchedule(funcOp, builder, batch, heads, seq, hd, causal, scaled);
    } else if (body.empty()) {
      if (wantTiled && allF32 && KCGLog::debug())
        llvm::errs() << "FMHAOptimizer: " << name << " takes the row-per-thread schedule (" << whyNot << ")\n";
      builder.setInsertionPointToStart(&body);
      Location loc = builder.getUnknownLoc();
      Value Q = body.getArgument(0), K = body.getArgument(1), V = body.getArgument(2), O = body.getArgument(3);
      const bool ragged = seq % br != 0;
      auto grid = builder.create<AffineParallelOp>(loc, std::vector<int64_t>{0, 0, 0},
                                                   std::vector<int64_t>{batch, heads, (seq + br - 1) / br});
      builder.create<func::ReturnOp>(loc, ValueRange({O}));
      builder.setInsertionPoint(grid.getBody()->getTerminator());
      auto block = builder.create<AffineParallelOp>(loc, std::vector<int64_t>{0}, std::vector<int64_t>{br});
      builder.setInsertionPoint(block.getBody()->getTerminator());
      auto gidx = grid.getIVs();
      Value b = gidx[0], h = gidx[1], rb = gidx[2], t = block.getIVs()[0];
      AffineExpr d0 = getAffineDimExpr(0), d1 = getAffineDimExpr(1), d2 = getAffineDimExpr(2), d3 = getAffineDimExpr(3),
                 d4 = getAffineDimExpr(4);
      // (b, h, rb, t, d) -> [b, h, rb*Br + t, d]
      AffineMap rowMap = AffineMap::get(5, 0, ArrayRef<AffineExpr>({d0, d1, d2 * br + d3, d4}));
      auto widenTo = [&](OpBuilder& ob, Value v) -> Value {
        return v.getType() == f32 ? v : ob.create<arith::ExtFOp>(ob.getUnknownLoc(), f32, v).getResult();
      };
      if (ragged) {
        // (rb, t): the thread's query row rb*Br + t exists; everything a thread does sits under this condition (and
        // the keys are then read from global memory: a barrier must not stand under a condition that differs
        // between the threads of a workgroup)
        auto rowExists = IntegerSet::get(2, 0, ArrayRef<AffineExpr>((seq - 1) - d0 * br - d1), ArrayRef<bool>(false));
        auto ifOp = builder.create<AffineIfOp>(loc, rowExists, ValueRange({rb, t}), false);
        builder.setInsertionPoint(ifOp.getThenBlock()->getTerminator());
      }

      Value zeroIdx = builder.create<arith::ConstantIndexOp>(loc, 0).getResult();
      Value zero = builder.create<arith::ConstantOp>(loc, builder.getFloatAttr(f32, 0)).getResult();
      Value negInf = builder.create<arith::ConstantOp>(loc, builder.getFloatAttr(f32, -INFINITY)).getResult();
      Value scale = builder.create<arith::ConstantOp>(loc, builder.getFloatAttr(f32, 1.0 / std::sqrt((double)hd))).getResult();
      Value rowMax = Rewriter::alloc_buffer(block, MemorySpace::local, {1}, f32);
      Value rowSum = Rewriter::alloc_buffer(block, MemorySpace::local, {1}, f32);
      Value acc = Rewriter::alloc_buffer(block, MemorySpace::local, {hd}, f32);
      Value qRow = Rewriter::alloc_buffer(block, MemorySpace::local, {hd}, f32);
      builder.create<AffineStoreOp>(loc, negInf, rowMax, ValueRange({zeroIdx}));
      builder.create<AffineStoreOp>(loc, zero, rowSum, ValueRange({zeroIdx}));
      Rewriter::set_buffer(builder, acc, zero);
      // the query row stays in registers
      builder.create<AffineForOp>(loc, 0, hd, 1, ValueRange({}), [&](OpBuilder& lb, Location lloc, Value d, ValueRange) {
        Value q = widenTo(lb, lb.create<AffineLoadOp>(lloc, Q, rowMap, ValueRange({b, h, rb, t, d})).getResult());
        lb.create<AffineStoreOp>(lloc, q, qRow, ValueRange({d}));
        lb.create<AffineYieldOp>(lloc);
      });
      // Keys.  A workgroup walks them in tiles of Bc rows of K and V that its threads copy into shared memory together
      // (thread t takes elements t, t + Br, ... of the tile, row-major), one barrier after the copy and one after
      // the tile's last use; every thread then runs its own query row's online softmax over the tile from there.
      // (The reference's attention schedule stages Q, K, V and P tiles in shared memory,
      // src/Optimizer/Optimizer.cc:2201-2437; the query row and the probabilities of a thread's own row stay in
      // registers here.)  Without a tile length that the threads can share out evenly the keys are read from global
      // memory one by one.
      int64_t bc = fmhaConfig.count("BLOCK_SIZE_KV") ? fmhaConfig["BLOCK_SIZE_KV"] : 0;
      if (bc <= 0)
        for (int64_t c : {64, 32, 16, 8, 4, 2, 1})
          if (seq % c == 0 && (c * hd) % br == 0) { bc = c; break; }
      const bool tiled = !ragged && bc > 0 && seq % bc == 0 && (bc * hd) % br == 0;
      Value smK, smV;
      if (tiled) {
        smK = Rewriter::alloc_buffer(grid, MemorySpace::shared, {bc, hd}, typeK.getElementType());
        smV = Rewriter::alloc_buffer(grid, MemorySpace::shared, {bc, hd}, typeV.getElementType());
      }
      auto tileLoop = builder.create<AffineForOp>(loc, 0, seq, tiled ? bc : seq);
      {
        OpBuilder tb(tileLoop.getBody()->getTerminator());
        Value jt = tileLoop.getInductionVar();
        if (tiled && causal) {
          // a tile whose first key lies behind the workgroup's last query concerns none of its threads (the same
          // decision in every thread, so the barriers inside are reached by all of them or by none)
          auto set = IntegerSet::get(2, 0, ArrayRef<AffineExpr>(d0 * br + (br - 1) - d1), ArrayRef<bool>(false));
          auto ifOp = tb.create<AffineIfOp>(loc, set, ValueRange({rb, jt}), false);
          tb.setInsertionPoint(ifOp.getThenBlock()->getTerminator());
        }
        if (tiled) {
          // (jt, c, t) -> tile row (c*Br + t) floordiv hd, column (c*Br + t) mod hd
          AffineExpr flat = d1 * br + d2;
          AffineMap fromGlobal = AffineMap::get(5, 0, ArrayRef<AffineExpr>({d3, d4, d0 + flat.floorDiv(hd), flat % hd}));
          AffineMap toShared = AffineMap::get(3, 0, ArrayRef<AffineExpr>({flat.floorDiv(hd), flat % hd}));
          tb.create<AffineForOp>(loc, 0, bc * hd / br, 1, ValueRange({}), [&](OpBuilder& lb, Location lloc, Value c, ValueRange) {
            Value kv = lb.create<AffineLoadOp>(lloc, K, fromGlobal, ValueRange({jt, c, t, b, h})).getResult();
            lb.create<AffineStoreOp>(lloc, kv, smK, toShared, ValueRange({jt, c, t}));
            Value vv = lb.create<AffineLoadOp>(lloc, V, fromGlobal, ValueRange({jt, c, t, b, h})).getResult();
            lb.create<AffineStoreOp>(lloc, vv, smV, toShared, ValueRange({jt, c, t}));
            lb.create<AffineYieldOp>(lloc);
          });
          gpu::BarrierOp::create(tb, loc);
        }
        auto keyLoop = tb.create<AffineForOp>(loc, 0, tiled ? bc : seq, 1);
        if (tiled) gpu::BarrierOp::create(tb, loc);      // the next tile overwrites what this one's last key still reads
        OpBuilder kb(keyLoop.getBody()->getTerminator());
        Value jj = keyLoop.getInductionVar();
        // the key's row in K and V: global (b, h, jt + jj, d) or shared (jj, d)
        AffineMap keyRow = AffineMap::get(5, 0, ArrayRef<AffineExpr>({d0, d1, d2 + d3, d4}));
        auto loadKey = [&](OpBuilder& lb, Location lloc, Value global, Value shared, Value d) -> Value {
          if (tiled) return lb.create<AffineLoadOp>(lloc, shared, ValueRange({jj, d})).getResult();
          return lb.create<AffineLoadOp>(lloc, global, keyRow, ValueRange({b, h, jt, jj, d})).getResult();
        };
        if (causal) {
          // (rb, t, jt, jj): rb*Br + t - (jt + jj) >= 0
          auto set = IntegerSet::get(4, 0, ArrayRef<AffineExpr>(d0 * br + d1 - d2 - d3), ArrayRef<bool>(false));
          auto ifOp = kb.create<AffineIfOp>(loc, set, ValueRange({rb, t, jt, jj}), false);
          kb.setInsertionPoint(ifOp.getThenBlock()->getTerminator());
        }
        auto dot = kb.create<AffineForOp>(loc, 0, hd, 1, ValueRange({zero}),
          [&](OpBuilder& lb, Location lloc, Value d, ValueRange iterArgs) {
            Value q = lb.create<AffineLoadOp>(lloc, qRow, ValueRange({d})).getResult();
            Value k = widenTo(lb, loadKey(lb, lloc, K, smK, d));
            Value mul = lb.create<arith::MulFOp>(lloc, q, k).getResult();
            Value add = lb.create<arith::AddFOp>(lloc, mul, iterArgs[0]).getResult();
            lb.create<AffineYieldOp>(lloc, ValueRange({add}));
          });
        Value s = dot.getResult(0);
        if (scaled) s = kb.create<arith::MulFOp>(loc, s, scale).getResult();
        Value mOld = kb.create<AffineLoadOp>(loc, rowMax, ValueRange({zeroIdx})).getResult();
        Value lOld = kb.create<AffineLoadOp>(loc, rowSum, ValueRange({zeroIdx})).getResult();
        Value mNew = kb.create<arith::MaxFOp>(loc, mOld, s).getResult();
        Value p = kb.create<math::ExpOp>(loc, kb.create<arith::SubFOp>(loc, s, mNew).getResult()).getResult();
        Value alpha = kb.create<math::ExpOp>(loc, kb.create<arith::SubFOp>(loc, mOld, mNew).getResult()).getResult();
        Value lNew = kb.create<arith::AddFOp>(loc, kb.create<arith::MulFOp>(loc, lOld, alpha).getResult(), p).getResult();
        kb.create<AffineStoreOp>(loc, mNew, rowMax, ValueRange({zeroIdx}));
        kb.create<AffineStoreOp>(loc, lNew, rowSum, ValueRange({zeroIdx}));
        kb.create<AffineForOp>(loc, 0, hd, 1, ValueRange({}), [&](OpBuilder& lb, Location lloc, Value d, ValueRange) {
          Value o = lb.create<AffineLoadOp>(lloc, acc, ValueRange({d})).getResult();
          Value v = widenTo(lb, loadKey(lb, lloc, V, smV, d));
          Value scaledO = lb.create<arith::MulFOp>(lloc, o, alpha).getResult();
          Value pv = lb.create<arith::MulFOp>(lloc, p, v).getResult();
          lb.create<AffineStoreOp>(lloc, lb.create<arith::AddFOp>(lloc, scaledO, pv).getResult(), acc, ValueRange({d}));
          lb.create<AffineYieldOp>(lloc);
        });
      }
      // O = acc / sum
      Value lFinal = builder.create<AffineLoadOp>(loc, rowSum, ValueRange({zeroIdx})).getResult();
      builder.create<AffineForOp>(loc, 0, hd, 1, ValueRange({}), [&](OpBuilder& lb, Location lloc, Value d, ValueRange) {
        Value o = lb.create<AffineLoadOp>(lloc, acc, ValueRange({d})).getResult();
        Value r = lb.create<arith::DivFOp>(lloc, o, lFinal).getResult();
        if (typeO.getElementType() != f32) r = lb.create<arith::TruncFOp>(lloc, typeO.getElementType(), r).getResult();
        lb.create<AffineStoreOp>(lloc, r, O, rowMap, ValueRange({b, h, rb, t, d}));
        lb.create<AffineYieldOp>(lloc);
      });
      std::map<std::string, int> used = fmhaConfig;
      for (const char* key : {"Hd", "Br", "Bc"}) used.erase(key);     // a tiled function's extents, left by an earlier one
      used["BLOCK_SIZE"] = (int)br;
      used["CAUSAL"] = causal;
      used["SCALE_RSQRT_D"] = scaled;
      used["BLOCK_SIZE_KV"] = tiled ? (int)bc : 0;
      used["TILED"] = 0;
      tagFunction(funcOp, "FMHA", used, builder);
    }
    // one fused call replaces the three calls
    builder.setInsertionPointAfter(second.getOperation());
    auto fused = builder.create<func::CallOp>(builder.getUnknownLoc(), funcOp, ValueRange({buf.Q, buf.K, buf.V, buf.O}));
    second.getResult(0).replaceAllUsesWith(fused.getResult(0));
    second.erase();
    softmax.erase();
    func::CallOp(first).erase();
    // the S placeholder and the unfused functions stay in the module, unused, as in the reference
    builder.restoreInsertionPoint(ip);
    DUMP(module);
  }
}

}  // namespace KernelCodeGen
