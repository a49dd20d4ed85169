// Unit checks of the IR, the Analyzer and every Rewriter primitive.  Each
// rewrite is applied to a small nest and judged by what it must preserve: the
// function computes the same values on the host interpreter before and after
// (bit for bit unless a summation order changes), the module still verifies,
// and the structural effect (loop bounds, steps, buffer shapes, sets) is the
// documented one.  Prints one "ok <name>" line per check; exits non-zero on the
// first failure.
#include <cmath>
#include <cstdio>
#include <functional>
#include <random>
#include <sstream>

#include "IR/Interpreter.h"
#include "KernelCodeGen.h"

using namespace KernelCodeGen;
using namespace mlir;

static int failures = 0;
#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) {                                                           \
      printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                 \
      ++failures;                                                            \
      return;                                                                \
    }                                                                        \
  } while (0)

static std::mt19937 rng(7);
static HostTensor randomTensor(std::vector<int64_t> shape, OpBuilder& b) {
  HostTensor t{shape, b.getF32Type(), {}};
  std::uniform_real_distribution<float> U(-1, 1);
  for (int64_t i = 0; i < t.numElements(); ++i) t.data.push_back((double)U(rng));
  return t;
}
static double maxDiff(const HostTensor& a, const HostTensor& b) {
  if (a.data.size() != b.data.size()) return 1e30;
  double m = 0;
  for (size_t i = 0; i < a.data.size(); ++i) m = std::max(m, std::fabs(a.data[i] - b.data[i]));
  return m;
}

struct Fixture {
  KernelCodeGenerator gen{"ROCm"};
  ComputeDAG* graph;
  OpBuilder builder;
  Fixture() { graph = &gen.createGraph("t"); }
  ModuleOp module() { return graph->module; }
  std::vector<HostTensor> run(std::vector<HostTensor> in) {
    Interpreter I(graph->module);
    return I.runGraph(in);
  }
  bool verifies() {
    std::string msg;
    bool ok = succeeded(verify(graph->module, &msg));
    if (!ok) printf("  verify: %s\n", msg.c_str());
    return ok;
  }
};

static void run(const char* name, const std::function<void()>& fn) {
  int before = failures;
  fn();
  if (failures == before) printf("ok %s\n", name);
  fflush(stdout);
}

// ---------------------------------------------------------------------------
static void testAffineAlgebra() {
  AffineExpr d0 = getAffineDimExpr(0), d1 = getAffineDimExpr(1);
  AffineExpr e = (d0 * 16 + d1).floorDiv(32) + ((d0 * 16 + d1) % 32) * 4;
  CHECK(e.evaluate({3, 5}) == (53 / 32) + (53 % 32) * 4);
  CHECK((d0 - 7).evaluate({3}) == -4);
  CHECK(((d0 - 7) % 4).evaluate({3}) == 0);            // mod is non-negative
  CHECK(((d0 - 7).floorDiv(4)).evaluate({2}) == -2);   // floor, not truncation
  CHECK(((d0 - 7).ceilDiv(4)).evaluate({2}) == -1);
  CHECK(d0 + 0 == d0 && d0 * 1 == d0 && (d0 * 0) == 0);
  CHECK((getAffineConstantExpr(6) * 7) == 42);
  CHECK(d0 + d1 == d0 + d1);                            // interned: structural equality is pointer equality
  AffineMap m = AffineMap::get(2, 0, ArrayRef<AffineExpr>({d0 + d1, d0 * 2}));
  CHECK(m.getNumDims() == 2 && m.getNumResults() == 2 && !m.isConstant());
  auto r = m.evaluate({3, 4});
  CHECK(r[0] == 7 && r[1] == 6);
  CHECK(AffineMap::getConstantMap(5).getSingleConstantResult() == 5);
  AffineExpr sub = e.replaceDims({d1, d0});
  CHECK(sub.evaluate({5, 3}) == e.evaluate({3, 5}));
  IntegerSet s = IntegerSet::get(1, 0, ArrayRef<AffineExpr>(1008 - d0), ArrayRef<bool>(false));
  CHECK(s.contains({1008}) && !s.contains({1009}));
  std::ostringstream os;
  s.print(os);
  CHECK(os.str() == "(d0) : (-d0 + 1008 >= 0)");       // the guard of the reference's Matmul dump (doc/pass.md:55)
}

static void testIRBasics() {
  Fixture f;
  auto A = f.graph->create<PlaceHolder>(std::vector<int64_t>{4, 4}, std::string{"float32"});
  auto B = f.graph->create<PlaceHolder>(std::vector<int64_t>{4, 4}, std::string{"float32"});
  auto C = f.graph->create<Matmul>(A, B);
  CHECK(C && C.getType().cast<MemRefType>().getShape()[0] == 4);
  auto m = f.module();
  auto funcs = Analyzer::collectFunctions(m, "Matmul");
  CHECK(funcs.size() == 1 && funcs[0].getSymName() == "Matmul_m4n4k4");
  CHECK(Analyzer::collectFunctions(m, "Softmax").empty());
  CHECK(Analyzer::getTargetFunction(m, "Matmul_m4n4k4") && !Analyzer::getTargetFunction(m, "Matmul"));
  auto loops = Analyzer::collectFuncLoops(funcs[0]);
  CHECK(loops.size() == 3 && loops[2].getNumIterOperands() == 1);   // pre-order: i, j, k
  CHECK(Analyzer::collectOutermostLoop(m).size() == 1);
  CHECK(Analyzer::collectFuncCalls(m).size() == 1);
  CHECK(Analyzer::getUsersNumber(A.getUsers()) == 1);
  // use lists and replaceAllUsesWith
  auto A2 = f.graph->create<PlaceHolder>(std::vector<int64_t>{4, 4}, std::string{"float32"});
  A2.getDefiningOp()->moveAfter(A.getDefiningOp());
  A.replaceAllUsesWith(A2);
  CHECK(A.use_empty() && A2.hasOneUse());
  // deep clone is independent and prints the same
  auto copy = m.clone();
  std::ostringstream a, b;
  m->print(a);
  copy->print(b);
  CHECK(a.str() == b.str());
  Analyzer::collectFuncLoops(Analyzer::collectFunctions(copy, "Matmul")[0])[2].setStep(2);
  CHECK(loops[2].getStep() == 1);
  copy.destroy();
  CHECK(f.verifies());
  // the verifier catches a use that does not dominate
  Operation* call = Analyzer::collectFuncCalls(m)[0];
  call->moveBefore(&m.getBody()->front());
  std::string msg;
  CHECK(failed(verify(m, &msg)) && msg.find("dominate") != std::string::npos);
}

static void testIdentifyBatchMatmul() {
  BatchMatmulDescriptor d;
  CHECK(identifyBatchMatmul("BatchMatmul_8_32_m2048_n64_k2048_NN", d));
  CHECK(d.m == 2048 && d.n == 64 && d.k == 2048 && !d.transA && !d.transB && d.batch == std::vector<int>({8, 32}));
  CHECK(identifyBatchMatmul("BatchMatmul_16_m1024_n1024_k1024_NT", d) && d.transB && d.batch.size() == 1);
  CHECK(!identifyBatchMatmul("Matmul_m4n4k4", d) && !identifyBatchMatmul("BatchMatmul_m4_n4_k4_XY", d));
}

// A function with a single elementwise nest over [rows, cols]: y = 2*x + 1 written with mulf/addf.
struct EwCase {
  Fixture f;
  func::FuncOp fn;
  std::vector<AffineForOp> loops;
  std::vector<HostTensor> in, ref;
  EwCase(std::vector<int64_t> shape) {
    auto X = f.graph->create<PlaceHolder>(shape, std::string{"float32"});
    f.graph->create<ElementWise>(X, "Gelu", MemorySpace::global);
    auto m = f.module();
    fn = Analyzer::collectFunctions(m, "Elementwise")[0];
    loops = Analyzer::collectFuncLoops(fn);
    in = {randomTensor(shape, f.builder)};
    ref = f.run(in);
  }
  double diff() { return maxDiff(ref[0], f.run(in)[0]); }
};

static void testSplit() {
  EwCase c({24, 16});
  auto parts = Rewriter::split(c.loops[0], 3, {2, 8});
  CHECK(parts.size() == 3);
  CHECK(parts[0].getStep() == 8 && parts[0].getConstantUpperBound() == 24);
  CHECK(parts[1].getStep() == 2 && parts[1].getConstantUpperBound() == 8);
  CHECK(parts[2].getStep() == 1 && parts[2].getConstantUpperBound() == 2);
  CHECK(parts[1]->getParentOp() == parts[0].getOperation() && parts[2]->getParentOp() == parts[1].getOperation());
  CHECK(c.f.verifies() && c.diff() == 0.0);
  // the sum of the new indices sits inside the access map, no affine.apply is created
  std::ostringstream os;
  c.fn->print(os);
  CHECK(os.str().find("affine.apply") == std::string::npos && os.str().find(" + ") != std::string::npos);
}

static void testReorderPerfectAndImperfect() {
  EwCase c({6, 10});
  Rewriter::reorder({c.loops[1], c.loops[0]});
  CHECK(c.loops[0]->getParentOp() == c.loops[1].getOperation());
  CHECK(c.f.verifies() && c.diff() == 0.0);
  // imperfect nest: matmul after bufferisation has init / write-back around the k loop
  Fixture f;
  auto A = f.graph->create<PlaceHolder>(std::vector<int64_t>{8, 6}, std::string{"float32"});
  auto B = f.graph->create<PlaceHolder>(std::vector<int64_t>{6, 4}, std::string{"float32"});
  f.graph->create<Matmul>(A, B);
  std::vector<HostTensor> in{randomTensor({8, 6}, f.builder), randomTensor({6, 4}, f.builder)};
  auto ref = f.run(in);
  auto m = f.module();
  auto loops = Analyzer::collectFuncLoops(Analyzer::collectFunctions(m, "Matmul")[0]);
  std::vector<AffineForOp> kij{loops[2], loops[0], loops[1]};
  Value tile = Rewriter::bufferizeLoopCarryVar(kij);
  CHECK(tile && tile.getType().cast<MemRefType>().getShape().vec() == std::vector<int64_t>({8, 4}));
  CHECK(tile.getType().cast<MemRefType>().getMemorySpaceAsInt() == (unsigned)MemorySpace::local);
  CHECK(kij[0].getNumIterOperands() == 0);
  CHECK(f.verifies() && maxDiff(ref[0], f.run(in)[0]) == 0.0);
  Rewriter::reorder({kij[0], kij[1], kij[2]});   // k outermost: init and write-back nests are peeled off
  CHECK(kij[1]->getParentOp() == kij[0].getOperation() && kij[2]->getParentOp() == kij[1].getOperation());
  CHECK(f.verifies() && maxDiff(ref[0], f.run(in)[0]) == 0.0);
}

static void testParallelAndNormalise() {
  EwCase c({12, 8});
  auto rows = Rewriter::split(c.loops[0], 2, {4});
  auto par = Rewriter::parallel({rows[0]});
  CHECK(par.getNumDims() == 1);
  int64_t total;
  auto dims = Analyzer::getParallelNumber(par, total);
  CHECK(dims == std::vector<int64_t>({3}) && total == 3);            // 12 / 4, normalised to step 1
  CHECK(isa<AffineApplyOp>(&par.getBody()->front()));                 // d0 * 4 at the start of the body
  CHECK(Rewriter::getElementIdx(par).size() == 1 && Rewriter::getParallelIdx(par).size() == 1);
  CHECK(c.f.verifies() && c.diff() == 0.0);
}

static void testReadWriteVectorizeCache() {
  EwCase c({8, 16});
  auto inner = c.loops[1];
  Value X = c.fn.getArgument(0);
  Value Y = c.fn.front().back().getOperand(0);
  Type f32 = c.f.builder.getF32Type();
  // stage a whole row through two register arrays
  Value regIn = Rewriter::alloc_buffer(inner, Position::before, MemorySpace::local, {16}, f32);
  Value regOut = Rewriter::alloc_buffer(inner, Position::before, MemorySpace::local, {16}, f32);
  AffineExpr d0 = getAffineDimExpr(0), d1 = getAffineDimExpr(1);
  AffineMap rowVec = AffineMap::get(2, 0, ArrayRef<AffineExpr>({d0, d1 * 4}));
  auto rd = Rewriter::read(X, regIn, rowVec, {c.loops[0].getInductionVar()}, 4, inner, Position::before);
  auto wr = Rewriter::write(regOut, Y, rowVec, {c.loops[0].getInductionVar()}, 4, inner, Position::after);
  CHECK(rd.getConstantUpperBound() == 4 && wr.getConstantUpperBound() == 4);
  AffineMap point = AffineMap::get(1, 0, d0);
  Rewriter::cache_read(inner, X, regIn, point, {inner.getInductionVar()});
  Rewriter::cache_write(inner, Y, regOut, point, {inner.getInductionVar()});
  CHECK(c.f.verifies() && c.diff() == 0.0);
  std::ostringstream os;
  c.fn->print(os);
  CHECK(os.str().find("affine.vector_load") != std::string::npos && os.str().find("vector<4xf32>") != std::string::npos);
  // element-wise write (two extra map inputs) and the width-free copy loops
  Value reg2 = Rewriter::alloc_buffer(inner, Position::before, MemorySpace::local, {16}, f32);
  AffineMap elem = AffineMap::get(3, 0, ArrayRef<AffineExpr>({d0, d1 * 4 + getAffineDimExpr(2)}));
  auto rd2 = Rewriter::read(Y, reg2, rowVec, {c.loops[0].getInductionVar()}, 4, wr, Position::after);
  auto wr2 = Rewriter::write(reg2, Y, elem, {c.loops[0].getInductionVar()}, 4, rd2, Position::after);
  CHECK(isa<AffineForOp>(&wr2.getBody()->front()));
  AffineMap scalarRow = AffineMap::get(2, 0, ArrayRef<AffineExpr>({d0, d1}));
  auto rd3 = Rewriter::read(Y, reg2, scalarRow, {c.loops[0].getInductionVar()}, wr2, Position::after);
  auto wr3 = Rewriter::write(reg2, Y, scalarRow, {c.loops[0].getInductionVar()}, rd3, Position::after);
  CHECK(rd3.getConstantUpperBound() == 16 && wr3.getConstantUpperBound() == 16);
  CHECK(c.f.verifies() && c.diff() == 0.0);
  // vectorize a scalar copy loop
  Rewriter::vectorize(wr3, 4);
  CHECK(wr3.getStep() == 4);
  CHECK(c.f.verifies() && c.diff() == 0.0);
  auto bar = Rewriter::barrier(wr3, Position::after);
  CHECK(bar && bar->getPrevNode() == wr3.getOperation());
}

static void testIfSimplificationAndUnroll() {
  EwCase c({4, 8});
  auto inner = c.loops[1];
  OpBuilder b = OpBuilder::atBlockBegin(inner.getBody());
  AffineExpr d0 = getAffineDimExpr(0);
  // always true over 0..7, never true, and undecided
  auto always = b.create<AffineIfOp>(b.getUnknownLoc(), IntegerSet::get(1, 0, ArrayRef<AffineExpr>(7 - d0), ArrayRef<bool>(false)),
                                     ValueRange({inner.getInductionVar()}));
  auto never = b.create<AffineIfOp>(b.getUnknownLoc(), IntegerSet::get(1, 0, ArrayRef<AffineExpr>(d0 - 8), ArrayRef<bool>(false)),
                                    ValueRange({inner.getInductionVar()}));
  auto maybe = b.create<AffineIfOp>(b.getUnknownLoc(), IntegerSet::get(1, 0, ArrayRef<AffineExpr>(3 - d0), ArrayRef<bool>(false)),
                                    ValueRange({inner.getInductionVar()}));
  // move the real body under `always`; put a wrong store under `never`
  std::vector<Operation*> bodyOps;
  for (auto& op : inner.getBody()->getOperations())
    if (!isa<AffineIfOp>(op) && op.getKind() != OpKind::AffineYield) bodyOps.push_back(&op);
  for (auto* op : bodyOps) op->moveBefore(always.getThenBlock()->getTerminator());
  OpBuilder nb(never.getThenBlock()->getTerminator());
  Value bad = nb.create<arith::ConstantOp>(nb.getUnknownLoc(), nb.getFloatAttr(nb.getF32Type(), 99.0)).getResult();
  nb.create<AffineStoreOp>(nb.getUnknownLoc(), bad, c.fn.front().back().getOperand(0),
                           ValueRange({c.loops[0].getInductionVar(), inner.getInductionVar()}));
  (void)maybe;
  auto m = c.f.module();
  auto countIfs = [&]() { int n = 0; c.fn->walk([&](Operation* o) { if (isa<AffineIfOp>(o)) ++n; }); return n; };
  CHECK(countIfs() == 3 && c.diff() == 0.0);
  Rewriter::take_off_true_if(m);
  CHECK(countIfs() == 2);
  Rewriter::delete_false_if(m);
  CHECK(countIfs() == 1);
  CHECK(c.f.verifies() && c.diff() == 0.0);
  // unroll the 4-trip outer loop completely, tag the inner one
  Rewriter::unroll(m, [&](AffineForOp l) { return l == c.loops[0]; });
  auto loops = Analyzer::collectFuncLoops(c.fn);
  CHECK(loops.size() == 4);
  Rewriter::unrollAttribute(m, [&](AffineForOp l) { return l.getConstantUpperBound() == 8; });
  for (auto l : loops) CHECK(l->getAttr("affine.loop").s == "unroll");
  CHECK(c.f.verifies() && c.diff() == 0.0);
}

static void testPipelineOnMatmul() {
  // the whole Matmul schedule exercises pipeline / detach_last_loop / schedule /
  // extract_loop / change_double_buffer; compare with the reference's dump (doc/pass.md:3-132)
  Fixture f;
  auto A = f.graph->create<PlaceHolder>(std::vector<int64_t>{256, 64}, std::string{"float32"});
  auto B = f.graph->create<PlaceHolder>(std::vector<int64_t>{64, 128}, std::string{"float32"});
  f.graph->create<Matmul>(A, B);
  std::vector<HostTensor> in{randomTensor({256, 64}, f.builder), randomTensor({64, 128}, f.builder)};
  auto ref = f.run(in);
  MatmulOptimizer opt;
  MatmulOptimizer::matmulConfig = {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 8}, {"GROUP_SIZE_M", 8},
                                   {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8}, {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 32}};
  auto m = f.module();
  CHECK(opt.applicable(m));
  opt.applyOptimzer(m, f.builder);
  CHECK(f.verifies());
  Interpreter I(m);
  std::vector<HostTensor> in2 = in;
  auto out = I.runGraph(in2);
  CHECK(maxDiff(ref[0], out[0]) == 0.0);           // same products in the same k order: bit-exact
  CHECK(I.barriersExecuted > 0);
  CHECK(I.sharedHazards == 0);                     // every shared element is separated by a barrier between threads
  std::ostringstream os;
  m->print(os);
  const std::string t = os.str();
  // buffers of the reference dump: smem 2x8x128 (twice), frags 2x8 (twice), tile 8x8, ldg regs 4 (twice)
  auto count = [&](const std::string& s) { size_t n = 0, p = 0; while ((p = t.find(s, p)) != std::string::npos) { ++n; p += s.size(); } return n; };
  CHECK(count("memref.alloc() : memref<2x8x128xf32, 2>") == 2);
  CHECK(count("memref.alloc() : memref<2x8xf32, 3>") == 2);
  CHECK(count("memref.alloc() : memref<8x8xf32, 3>") == 1);
  CHECK(count("memref.alloc() : memref<4xf32, 3>") == 2);
  CHECK(count("affine.parallel (%arg2, %arg3) = (0, 0) to (2, 1)") == 1);    // 256/128 x 128/128 workgroups
  CHECK(count("= (0, 0) to (16, 16)") == 1);                                 // 16 x 16 threads
  CHECK(count("affine_set<(d0) : (-d0 + 48 >= 0)>") == 2);                   // K - 2*BK = 64 - 16
  CHECK(count("step 8") == 1 && count("0 to 7 {") == 1);                     // k outer loop, peeled k inner loop
  CHECK(count("gpu.barrier") == 2);
  CHECK(count("func.state = \"gpu\"") == 1);
  // Lock-step execution hides a missing barrier (the values stay right); the audit does not.
  std::vector<Operation*> barriers;
  m->walk([&](Operation* o) { if (o->getKind() == OpKind::Barrier) barriers.push_back(o); });
  CHECK(barriers.size() == 2);
  for (Operation* b : barriers) b->erase();
  CHECK(f.verifies());
  Interpreter J(m);
  std::vector<HostTensor> in3 = in;
  auto out3 = J.runGraph(in3);
  CHECK(maxDiff(ref[0], out3[0]) == 0.0);
  CHECK(J.barriersExecuted == 0 && J.sharedHazards > 0);
  CHECK(J.firstHazard.find("without a barrier") != std::string::npos);
}

static void testHandScriptedScheduleGetsAKernel() {
  // A schedule written with the Rewriter alone, no optimizer and so no operator tag: rows split over workgroups and
  // threads, each thread's row segment staged through registers with 16-byte accesses.  The backend prints it
  // statement by statement (the reference's backend does nothing else, src/Backend/CUDA.cc:61-1184).
  EwCase c({64, 32});
  auto rows = Rewriter::split(c.loops[0], 2, {8});                 // 8 workgroups of 8 rows, one row per thread
  auto grid = Rewriter::parallel({rows[0]});
  auto block = Rewriter::parallel({rows[1]});
  auto indexOf = [](AffineParallelOp p) {                          // the level's index after normalisation
    Operation& first = p.getBody()->front();
    return isa<AffineApplyOp>(&first) ? first.getResult(0) : p.getIVs()[0];
  };
  Value gridRow = indexOf(grid), blockRow = indexOf(block);
  auto inner = Analyzer::collectFuncLoops(c.fn).back();            // the loop along the row
  Value X = c.fn.getArgument(0);
  Value Y = c.fn.front().back().getOperand(0);
  Type f32 = c.f.builder.getF32Type();
  Value regIn = Rewriter::alloc_buffer(inner, Position::before, MemorySpace::local, {32}, f32);
  Value regOut = Rewriter::alloc_buffer(inner, Position::before, MemorySpace::local, {32}, f32);
  AffineExpr d0 = getAffineDimExpr(0), d1 = getAffineDimExpr(1), d2 = getAffineDimExpr(2);
  AffineMap rowVec = AffineMap::get(3, 0, ArrayRef<AffineExpr>({d0 + d1, d2 * 4}));
  Rewriter::read(X, regIn, rowVec, {gridRow, blockRow}, 4, inner, Position::before);
  Rewriter::write(regOut, Y, rowVec, {gridRow, blockRow}, 4, inner, Position::after);
  AffineMap point = AffineMap::get(1, 0, d0);
  Rewriter::cache_read(inner, X, regIn, point, {inner.getInductionVar()});
  Rewriter::cache_write(inner, Y, regOut, point, {inner.getInductionVar()});
  CHECK(c.f.verifies() && c.diff() == 0.0);
  CHECK(!c.fn->hasAttr("kcg.op"));
  auto m = c.f.module();
  std::vector<KernelLaunchInfo> infos;
  std::string error;
  // not marked as scheduled yet: no kernel, and no error either
  CHECK(HIPGen(m, infos, &error).find("__global__ void __launch_bounds__") == std::string::npos && infos.empty() && error.empty());
  c.fn->setAttr("func.state", c.f.builder.getStringAttr("gpu"));
  const std::string src = HIPGen(m, infos, &error);
  if (!error.empty()) printf("  HIPGen: %s\n", error.c_str());
  CHECK(error.empty() && infos.size() == 1);
  if (infos.size() == 1) {
    CHECK(infos[0].name == "kernel0" && infos[0].grid[0] == 8 && infos[0].block[0] == 8 && infos[0].numArgs == 2);
    CHECK(infos[0].argBytes == std::vector<int64_t>({64 * 32 * 4, 64 * 32 * 4}));
  }
  CHECK(src.find("extern \"C\" __global__ void __launch_bounds__(8) kernel0(float* __restrict__ arg0, float* __restrict__ out0)") != std::string::npos);
  CHECK(src.find("(int)blockIdx.x") != std::string::npos && src.find("(int)threadIdx.x") != std::string::npos);
  CHECK(src.find("*(const kcg_v4_float*)(arg0 + ") != std::string::npos && src.find("tanhf(") != std::string::npos);
  // what has no lowering is refused with the reason, not printed wrongly: a third parallel level
  EwCase d({64, 32});
  auto r2 = Rewriter::split(d.loops[0], 2, {8});
  Rewriter::parallel({r2[0]});
  Rewriter::parallel({r2[1]});
  Rewriter::parallel({Analyzer::collectFuncLoops(d.fn).back()});
  d.fn->setAttr("func.state", d.f.builder.getStringAttr("gpu"));
  auto m2 = d.f.module();
  CHECK(HIPGen(m2, infos, &error).empty() && infos.empty());
  CHECK(error.find("nested deeper than grid and workgroup") != std::string::npos);
}

static void testSwapLoopsConstantLoopAndGridToBlock() {
  // swapLoops: pairs of (outer, inner) loops are interchanged
  {
    EwCase c({6, 8});
    Rewriter::swapLoops({{c.loops[0], c.loops[1]}});
    auto loops = Analyzer::collectFuncLoops(c.fn);
    CHECK(loops.size() == 2 && loops[0].getConstantUpperBound() == 8 && loops[1].getConstantUpperBound() == 6);
    CHECK(c.f.verifies() && c.diff() == 0.0);
  }
  // create_constant_loop: an empty loop with the given constant bounds and step where the builder stands
  {
    EwCase c({6, 8});
    OpBuilder b(c.loops[0].getOperation());
    auto loop = Rewriter::create_constant_loop(b, 2, 11, 3);
    CHECK(loop.getConstantLowerBound() == 2 && loop.getConstantUpperBound() == 11 && loop.getStep() == 3);
    CHECK(loop->getNextNode() == c.loops[0].getOperation());
    CHECK(loop.getBody()->getTerminator() && loop.getBody()->getTerminator()->getKind() == OpKind::AffineYield);
    CHECK(&loop.getBody()->front() == loop.getBody()->getTerminator());
    CHECK(c.f.verifies() && c.diff() == 0.0);
  }
  // scheduleOpGridToBlock: constants that stand at the grid level move into the workgroup level (behind its leading
  // affine.apply when it has one), where the backend expects a thread's values
  {
    EwCase c({16, 8});
    auto rows = Rewriter::split(c.loops[0], 2, {4});
    auto grid = Rewriter::parallel({rows[0]});
    auto block = Rewriter::parallel({rows[1]});
    OpBuilder gb = OpBuilder::atBlockBegin(grid.getBody());
    auto k1 = gb.create<arith::ConstantIndexOp>(gb.getUnknownLoc(), 7);
    auto k2 = gb.create<arith::ConstantOp>(gb.getUnknownLoc(), gb.getFloatAttr(gb.getF32Type(), 2.5));
    CHECK(k1->getParentOp() == grid.getOperation() && k2->getParentOp() == grid.getOperation());
    Rewriter::scheduleOpGridToBlock(grid, block);
    CHECK(k1->getParentOp() == block.getOperation() && k2->getParentOp() == block.getOperation());
    int atGrid = 0;
    for (auto& op : grid.getBody()->getOperations()) atGrid += op.getKind() == OpKind::Constant;
    CHECK(atGrid == 0);
    CHECK(c.f.verifies() && c.diff() == 0.0);
  }
}

static void testCollapseAndHelpers() {
  {
    EwCase c({4, 6, 10});
    auto two = Rewriter::combineToTowDim(c.loops);
    CHECK(two.size() == 2 && two[0].getConstantUpperBound() * two[1].getConstantUpperBound() == 240);
    CHECK(two[1].getConstantUpperBound() == 15 && two[0].getConstantUpperBound() == 16);   // largest divisor <= sqrt(240)
    CHECK(c.f.verifies() && c.diff() == 0.0);
    auto one = Rewriter::combineToOneDim(two);
    CHECK(one.getConstantUpperBound() == 240);
    CHECK(c.f.verifies() && c.diff() == 0.0);
    auto parts = Rewriter::split(one, 2, {8});
    auto unit = Rewriter::modifyLoopStepToOne(parts[0]);
    CHECK(unit.getStep() == 1 && unit.getConstantUpperBound() == 30);
    CHECK(c.f.verifies() && c.diff() == 0.0);
  }
  {
    // collapse of nests that thread a loop-carried value (the LayerNorm reductions)
    Fixture f;
    auto X = f.graph->create<PlaceHolder>(std::vector<int64_t>{3, 4, 8}, std::string{"float32"});
    auto S = f.graph->create<PlaceHolder>(std::vector<int64_t>{4, 8}, std::string{"float32"});
    auto Bv = f.graph->create<PlaceHolder>(std::vector<int64_t>{4, 8}, std::string{"float32"});
    f.graph->create<LayerNorm>(X, S, Bv, (int64_t)1, 1e-5f);
    std::vector<HostTensor> in{randomTensor({3, 4, 8}, f.builder), randomTensor({4, 8}, f.builder), randomTensor({4, 8}, f.builder)};
    auto ref = f.run(in);
    auto m = f.module();
    auto fn = Analyzer::collectFunctions(m, "LayerNorm")[0];
    auto loops = Analyzer::collectFuncLoops(fn);   // outer, (sum: 2), (var: 2), (norm: 2)
    CHECK(loops.size() == 7);
    auto sum = Rewriter::combineToOneDim({loops[1], loops[2]});
    CHECK(sum.getConstantUpperBound() == 32 && sum.getNumIterOperands() == 1);
    CHECK(f.verifies() && maxDiff(ref[0], f.run(in)[0]) == 0.0);
    Value cell = Rewriter::bufferizeLoopCarryVar(sum, &fn.front());
    CHECK(cell.getType().cast<MemRefType>().getMemorySpaceAsInt() == (unsigned)MemorySpace::shared);
    CHECK(sum.getNumIterOperands() == 0);
    CHECK(f.verifies() && maxDiff(ref[0], f.run(in)[0]) == 0.0);
    // bufferizeOpResult on the sqrt
    Operation* sq = nullptr;
    fn->walk([&](Operation* o) { if (o->getKind() == OpKind::Sqrt) sq = o; });
    CHECK(sq != nullptr);
    Value buf = Rewriter::alloc_buffer(AffineForOp(loops[0]), Position::before, MemorySpace::shared, {1}, f.builder.getF32Type());
    Rewriter::bufferizeOpResult(sq, buf);
    CHECK(f.verifies() && maxDiff(ref[0], f.run(in)[0]) == 0.0);
  }
  {
    // builders: set_buffer, create_constant_loop, outer_product
    Fixture f;
    auto m = f.module();
    OpBuilder b = f.builder;
    b.setInsertionPointToStart(m.getBody());
    auto fn = buildFuction(m, b, "scratch", {MemRefType::get({3, 5}, b.getF32Type(), {}, 1), MemRefType::get({3}, b.getF32Type(), {}, 1),
                                             MemRefType::get({5}, b.getF32Type(), {}, 1)},
                           {MemRefType::get({3, 5}, b.getF32Type(), {}, 1)});
    b.setInsertionPointToStart(&fn.front());
    Value one = b.create<arith::ConstantOp>(b.getUnknownLoc(), b.getFloatAttr(b.getF32Type(), 1.0)).getResult();
    Rewriter::set_buffer(b, fn.getArgument(0), one);
    auto outer = Rewriter::outer_product(b, fn.getArgument(0), fn.getArgument(1), fn.getArgument(2), 3, 5);
    CHECK(outer.getConstantUpperBound() == 3);
    b.setInsertionPointToEnd(&fn.front());
    b.create<func::ReturnOp>(b.getUnknownLoc(), ValueRange({fn.getArgument(0)}));
    CHECK(f.verifies());
    std::vector<HostTensor> args{randomTensor({3, 5}, b), randomTensor({3}, b), randomTensor({5}, b)};
    Interpreter I(m);
    auto out = I.run(fn, args);
    for (int i = 0; i < 3; ++i)
      for (int j = 0; j < 5; ++j) CHECK(out[0].data[i * 5 + j] == (double)(float)((float)(args[1].data[i] * args[2].data[j]) + 1.0f));
  }
}

static void testIrregularMatAndBlockHelpers() {
  // 10 x 7 elementwise map tiled 4 x 4 by hand: ragged in both directions
  EwCase c({10, 7});
  const int rows = 10, cols = 7, tr = 4, tc = 4;
  // outer tile loops (ceil) with inner 4 x 4 loops, then irregularMat guards the inner nest
  OpBuilder b(c.loops[0].getOperation());
  Location loc = b.getUnknownLoc();
  auto ty = b.create<AffineForOp>(loc, 0, (rows + tr - 1) / tr * tr, tr);
  b.setInsertionPointToStart(ty.getBody());
  auto tx = b.create<AffineForOp>(loc, 0, (cols + tc - 1) / tc * tc, tc);
  b.setInsertionPointToStart(tx.getBody());
  Value zero = b.create<arith::ConstantIndexOp>(loc, 0).getResult();
  auto iy = b.create<AffineForOp>(loc, 0, tr, 1);
  b.setInsertionPointToStart(iy.getBody());
  auto ix = b.create<AffineForOp>(loc, 0, tc, 1);
  // move the body of the old nest, re-indexed by tile + inner index
  Operation* op = &c.loops[1].getBody()->front();
  while (op && op->getKind() != OpKind::AffineYield) { Operation* n = op->getNextNode(); op->moveBefore(ix.getBody()->getTerminator()); op = n; }
  AffineExpr d0 = getAffineDimExpr(0), d1 = getAffineDimExpr(1), d2 = getAffineDimExpr(2), d3 = getAffineDimExpr(3);
  AffineMap idx = AffineMap::get(4, 0, ArrayRef<AffineExpr>({d0 + d1, d2 + d3}));
  ix->getParentOp();
  std::vector<Operation*> accesses;
  ix->walk([&](Operation* o) { if (o->getKind() == OpKind::AffineLoad || o->getKind() == OpKind::AffineStore) accesses.push_back(o); });
  for (auto* o : accesses) {
    ValueRange ops({ty.getInductionVar(), iy.getInductionVar(), tx.getInductionVar(), ix.getInductionVar()});
    if (o->getKind() == OpKind::AffineLoad) AffineLoadOp(o).setAccess(AffineLoadOp(o).getMemRef(), idx, ops);
    else AffineStoreOp(o).setAccess(AffineStoreOp(o).getMemRef(), idx, ops);
  }
  c.loops[0].erase();
  // operands: (tile row start, tile column start, 0, 0)
  auto first = Rewriter::irregularMat(iy, {rows, cols, tr, tc}, {ty.getInductionVar(), tx.getInductionVar(), zero, zero});
  CHECK(first);
  CHECK(c.f.verifies());
  CHECK(c.diff() == 0.0);   // every element written exactly once, nothing out of bounds (the interpreter checks bounds)
  // one-dimensional thread index -> (y, x)
  Fixture f;
  auto X = f.graph->create<PlaceHolder>(std::vector<int64_t>{8, 8}, std::string{"float32"});
  f.graph->create<ElementWise>(X, "Relu", MemorySpace::global);
  auto m = f.module();
  auto loops = Analyzer::collectFuncLoops(Analyzer::collectFunctions(m, "Elementwise")[0]);
  auto one = Rewriter::combineToOneDim(loops);
  auto par = Rewriter::parallel({one});
  auto yx = Rewriter::blockLevelOneToTwo(par, 8);
  CHECK(yx.size() == 2 && yx[0].getDefiningOp<AffineApplyOp>().getAffineMap().getResult(0).evaluate({19}) == 2);
  CHECK(yx[1].getDefiningOp<AffineApplyOp>().getAffineMap().getResult(0).evaluate({19}) == 3);
  // constant de-duplication
  OpBuilder pb = OpBuilder::atBlockBegin(par.getBody());
  for (int i = 0; i < 3; ++i) pb.create<arith::ConstantIndexOp>(pb.getUnknownLoc(), 5);
  Rewriter::deleteExtraCstOp(par);
  int fives = 0;
  par->walk([&](Operation* o) { if (auto cst = dyn_cast<arith::ConstantIndexOp>(o)) if (cst.value() == 5) ++fives; });
  CHECK(fives == 1);
  CHECK(f.verifies());
}

static void testUsageContract() {
  // the shape of the reference's test driver (test/test.cc:8-49): Cast on {2,768,768}
  KernelCodeGenerator generator("ROCm");
  auto graph = generator.createGraph("demo");
  generator.setLogMode(Log::Release);
  generator.opts.push_back(std::move(std::make_unique<ElementWiseOptimizer>()));
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{2, 768, 768}, std::string{"float32"});
  auto cast = graph.create<ElementWise>(A, "Cast", MemorySpace::global, "int32");
  CHECK(cast);
  graph.dump();
  auto module = generator.optimize(graph);
  generator.dump(module);
  auto&& sourceCode = generator.codegen(module);
  CHECK(!sourceCode.empty() && generator.launchInfos().size() == 1);
  CHECK(sourceCode.find("extern \"C\" __global__") != std::string::npos);
  CHECK(sourceCode.find("// grid dims:(") != std::string::npos && sourceCode.find("kernel0") != std::string::npos);
  CHECK(sourceCode.find("cuda") == std::string::npos && sourceCode.find("__shfl_down_sync") == std::string::npos);
  CHECK(generator.launchInfos()[0].numArgs == 2);   // (X, Z)
  // numbering restarts at every codegen call
  auto again = generator.codegen(module);
  CHECK(again == sourceCode);
}


// ---------------------------------------------------------------------------
// The helper members of the per-operator optimizers (reference: include/Optimizer/Optimizer.h:89-108,
// 159-164, 191-192, 221-224, 267): index maps by evaluation, shape classification, and every loop rewrite by
// running the function on the interpreter before and after.
struct Scratch {
  Fixture f;
  OpBuilder b;
  func::FuncOp fn;
  Type f32;
  Scratch(const char* name, std::vector<std::vector<int64_t>> args, std::vector<int64_t> result) : b(f.builder) {
    auto m = f.module();
    f32 = b.getF32Type();
    b.setInsertionPointToStart(m.getBody());
    std::vector<Type> types;
    for (auto& shape : args) types.push_back(MemRefType::get(shape, f32, {}, 1));
    fn = buildFuction(m, b, name, types, {MemRefType::get(result, f32, {}, 1)});
    b.setInsertionPointToStart(&fn.front());
  }
  Value alloc(std::vector<int64_t> shape, MemorySpace ms) {
    return b.create<memref::AllocOp>(b.getUnknownLoc(), MemRefType::get(shape, f32, {}, (int)ms)).getResult();
  }
  Value constant(double v) { return b.create<arith::ConstantOp>(b.getUnknownLoc(), b.getFloatAttr(f32, v)).getResult(); }
  AffineForOp loop(int64_t ub, const std::function<void(OpBuilder&, Value)>& body) {
    return b.create<AffineForOp>(b.getUnknownLoc(), 0, ub, 1, ValueRange({}), [&](OpBuilder& lb, Location loc, Value iv, ValueRange) {
      body(lb, iv);
      lb.create<AffineYieldOp>(loc, ValueRange({}));
    });
  }
  // a grid of one workgroup, then thread levels inside it (the interpreter runs the threads of a level that is
  // nested in a grid level in lock-step)
  void enterGrid() {
    auto grid = b.create<AffineParallelOp>(b.getUnknownLoc(), std::vector<int64_t>{0}, std::vector<int64_t>{1});
    b.setInsertionPointToStart(grid.getBody());
  }
  AffineParallelOp threads(int64_t count) {
    return b.create<AffineParallelOp>(b.getUnknownLoc(), std::vector<int64_t>{0}, std::vector<int64_t>{count});
  }
  void finish(Value result) {
    b.setInsertionPointToEnd(&fn.front());
    b.create<func::ReturnOp>(b.getUnknownLoc(), ValueRange({result}));
  }
  HostTensor run(std::vector<HostTensor> args) {
    Interpreter I(f.module());
    return I.run(fn, args)[0];
  }
};

static void testOptimizerHelperMembers() {
  Location loc;
  // ---- index maps -----------------------------------------------------------------------------------
  {
    Fixture f;
    OpBuilder& b = f.builder;
    BinaryOptimizer bin;
    // tensor (2, 20, 256) refolded to y * 80 + x: extras = {rank, stride 0, stride 1, last extent, X}
    std::vector<int64_t> extras{3, 5120, 256, 256, 80};
    auto full = bin.getAffineMap("MaxLoadOrStore", b, extras);
    CHECK(full.getNumDims() == 6 && full.getNumResults() == 3);
    for (int64_t by : {0, 64}) for (int64_t ty : {0, 12}) for (int64_t iy : {0, 3}) for (int64_t tx : {0, 16}) for (int64_t ix : {0, 3}) {
      const int64_t flat = (by + ty + iy) * 80 + (0 + tx + ix * 4);
      auto r = full.evaluate({by, ty, iy, 0, tx, ix});
      CHECK(r[0] == flat / 5120 && r[1] == (flat % 5120) / 256 && r[2] == flat % 256);
    }
    auto two = bin.getAffineMap("MaxLoadOrStore", b, {2, 80});
    CHECK(two.evaluate({8, 2, 1, 64, 4, 2}) == (std::vector<int64_t>{11, 76}));
    // the broadcast operand (20, 256) of that tensor: its last two coordinates
    auto small = bin.getAffineMap("MinVectorLoad", b, extras, 2, 0);
    CHECK(small.getNumResults() == 2 && small.evaluate({64, 12, 3, 0, 16, 3}) == (std::vector<int64_t>{((79 * 80 + 28) % 5120) / 256, (79 * 80 + 28) % 256}));
    // (1, 20, 256): one broadcast coordinate fed by the extra leading input
    auto lead = bin.getAffineMap("MinVectorLoad", b, extras, 2, 1);
    CHECK(lead.getNumDims() == 7 && lead.getNumResults() == 3 && lead.evaluate({0, 64, 12, 3, 0, 16, 3})[0] == 0);
    CHECK(bin.getAffineMap("CacheLoadOrStore", b).evaluate({5}) == (std::vector<int64_t>{5}));
    GatherOptimizer ga;
    CHECK(ga.getAffineMap("VectorLoadOrStore", b, extras).evaluate({64, 12, 3, 0, 16, 3}) == full.evaluate({64, 12, 3, 0, 16, 3}));
    CHECK(ga.getAffineMap("PointLoadOrStore", b).evaluate({9}) == (std::vector<int64_t>{9}));
    FMHAOptimizer fa;
    FMHAOptimizer::fmhaConfig = {{"BLOCK_SIZE", 256}};
    CHECK(fa.getAffineMap("loadTileQ", b).evaluate({1, 2, 3, 17, 0}) == (std::vector<int64_t>{1, 2, 3 * 256 + 17, 0}));
    CHECK(fa.getAffineMap("loadTileK", b).evaluate({1, 2, 99}) == (std::vector<int64_t>{1, 2, 99, 0}));
    // operand shapes -> broadcast class
    auto shape = [&](std::vector<int64_t> s) { return f.graph->create<PlaceHolder>(s, std::string{"float32"}); };
    Value big = shape({2, 20, 256});
    auto classify = [&](Value small_) { BinaryOptimizer::BinaryOpData d; bin.getBinaryOpData(big, small_, d); return d; };
    using T = BinaryOptimizer::BinaryType;
    CHECK(classify(nullptr).type == T::constant);
    CHECK(classify(shape({1, 1})).type == T::allOne);
    CHECK(classify(shape({2, 20, 256})).type == T::allEqual);
    auto d1 = classify(shape({1, 20, 256}));
    CHECK(d1.type == T::hasOneOrder && d1.oneDimNums == 1 && d1.needDimNums == 2);
    auto d2 = classify(shape({1, 256}));
    CHECK(d2.type == T::hasOneOrder && d2.oneDimNums == 1 && d2.needDimNums == 1);
    auto d3 = classify(shape({20, 256}));
    CHECK(d3.type == T::noOneOrder && d3.needDimNums == 2);
    CHECK(classify(shape({20, 1})).type == T::hasOneUnorder && classify(shape({1, 20, 1})).type == T::hasOneUnorder);
    llvm::SmallVector<Value> six{big, big, big, shape({3}), shape({4}), big};
    CHECK(bin.getMinLoadOperands(2, six).size() == 2 && bin.getMinLoadOperands(2, six, big).size() == 3 && bin.getMinLoadOperands(3, six, big).size() == 7);
  }
  LayerNormOptimizer ln;
  LayerNormOptimizer::layerNormConfig = {{"VECTORIZE_WIDTH", 4}};
  // ---- read: loads staged through a cache by a vectorised copy loop -------------------------------------
  {
    Scratch s("staged", {{16}, {16}}, {16});
    Value src = s.fn.getArgument(0), out = s.fn.getArgument(1);
    Value cache = s.alloc({16}, MemorySpace::local);
    Value two = s.constant(2.0);
    auto loop = s.loop(16, [&](OpBuilder& lb, Value i) {
      Value v = lb.create<AffineLoadOp>(loc, src, ValueRange({i})).getResult();
      lb.create<AffineStoreOp>(loc, lb.create<arith::MulFOp>(loc, v, two).getResult(), out, ValueRange({i}));
    });
    s.finish(out);
    std::vector<HostTensor> in{randomTensor({16}, s.b), randomTensor({16}, s.b)};
    auto ref = s.run(in);
    auto loops = ln.read(loop, {cache, src});
    CHECK(loops.size() == 2 && loops[0].getStep() == 4 && loops[1] == loop);
    CHECK(s.f.verifies() && maxDiff(ref, s.run(in)) == 0.0);
    int fromSrc = 0;
    loop->walk([&](Operation* o) { if (auto l = dyn_cast<AffineLoadOp>(o)) fromSrc += l.getMemRef() == src; }, WalkOrder::PreOrder);
    CHECK(fromSrc == 0);
  }
  // ---- extractOpsFromLoop / write: loop fission ------------------------------------------------------------
  {
    Scratch s("fission", {{16}, {16}, {16}}, {16});
    Value a = s.fn.getArgument(0), m = s.fn.getArgument(1), out = s.fn.getArgument(2);
    auto loop = s.loop(16, [&](OpBuilder& lb, Value i) {
      Value x = lb.create<AffineLoadOp>(loc, a, ValueRange({i})).getResult();
      Value y = lb.create<AffineLoadOp>(loc, m, ValueRange({i})).getResult();
      Value d = lb.create<arith::SubFOp>(loc, x, y).getResult();
      Value q = lb.create<arith::MulFOp>(loc, d, d).getResult();
      lb.create<AffineStoreOp>(loc, q, out, ValueRange({i}));
    });
    s.finish(out);
    std::vector<HostTensor> in{randomTensor({16}, s.b), randomTensor({16}, s.b), randomTensor({16}, s.b)};
    auto ref = s.run(in);
    auto front = ln.extractOpsFromLoop(loop, {a, m});
    CHECK(front != loop && front->getNextNode() == loop.getOperation());
    int arithLeft = 0;
    for (auto& op : *loop.getBody()) arithLeft += op.getKind() == OpKind::SubF || op.getKind() == OpKind::MulF;
    CHECK(arithLeft == 0);
    CHECK(s.f.verifies() && maxDiff(ref, s.run(in)) == 0.0);
    // now the loop reads a[i] (the staged value) and stores it to out[i]: split the store off
    auto storeLoop = ln.write(loop, {a, out});
    CHECK(storeLoop != loop);
    int stores = 0;
    for (auto& op : *loop.getBody()) stores += isa<AffineStoreOp>(op);
    CHECK(stores == 0);
    CHECK(s.f.verifies() && maxDiff(ref, s.run(in)) == 0.0);
  }
  // ---- reduceUnrollOptimize: strided per-thread sums, halving steps, wavefront shuffles ----------------------
  {
    const int64_t T = 256, P = 4;
    Scratch s("tree", {{T * P}}, {1});
    Value x = s.fn.getArgument(0);
    Value cell = s.alloc({1}, MemorySpace::global);
    Value zeroIdx = s.b.create<arith::ConstantIndexOp>(loc, 0).getResult();
    s.b.create<AffineStoreOp>(loc, s.constant(0.0), cell, ValueRange({zeroIdx}));
    s.enterGrid();
    auto pal = s.threads(T);
    Value tid = pal.getIVs()[0];
    s.b.setInsertionPointToStart(pal.getBody());
    auto loop = s.loop(P, [&](OpBuilder& lb, Value i) {
      Value v = lb.create<AffineLoadOp>(loc, x, AffineMap::get(2, 0, getAffineDimExpr(0) + getAffineDimExpr(1) * T), ValueRange({tid, i})).getResult();
      Value c = lb.create<AffineLoadOp>(loc, cell, ValueRange({zeroIdx})).getResult();
      lb.create<AffineStoreOp>(loc, lb.create<arith::AddFOp>(loc, c, v).getResult(), cell, ValueRange({zeroIdx}));
    });
    s.finish(cell);
    auto created = ln.reduceUnrollOptimize(loop, pal);
    CHECK(created.size() >= 5 && s.f.verifies());
    int shuffles = 0, ifs = 0;
    pal->walk([&](Operation* o) { shuffles += o->getKind() == OpKind::Shuffle; ifs += o->getKind() == OpKind::AffineIf; }, WalkOrder::PreOrder);
    CHECK(shuffles == 6 && ifs == 2 /* 128, 64 */ + 2 /* wavefront, thread 0 */);
    std::vector<HostTensor> in{randomTensor({T * P}, s.b)};
    double want = 0;
    for (double v : in[0].data) want += v;
    CHECK(std::fabs(s.run(in).data[0] - want) < 1e-4);
  }
  // ---- elementWiseUnrollOptimize: iteration i of thread t works on element t + i * T --------------------------
  {
    const int64_t T = 64, P = 4;
    Scratch s("strided", {{T * P}, {T * P}}, {T * P});
    Value x = s.fn.getArgument(0), y = s.fn.getArgument(1);
    Value three = s.constant(3.0);
    s.enterGrid();
    auto pal = s.threads(T);
    s.b.setInsertionPointToStart(pal.getBody());
    auto loop = s.loop(P, [&](OpBuilder& lb, Value i) {
      Value v = lb.create<AffineLoadOp>(loc, x, ValueRange({i})).getResult();
      lb.create<AffineStoreOp>(loc, lb.create<arith::MulFOp>(loc, v, three).getResult(), y, ValueRange({i}));
    });
    s.finish(y);
    ln.elementWiseUnrollOptimize(loop, pal);
    CHECK(s.f.verifies());
    int loopsLeft = 0, stores = 0;
    pal->walk([&](Operation* o) { loopsLeft += o->getKind() == OpKind::AffineFor; stores += o->getKind() == OpKind::AffineStore; }, WalkOrder::PreOrder);
    CHECK(loopsLeft == 0 && stores == P);
    std::vector<HostTensor> in{randomTensor({T * P}, s.b), randomTensor({T * P}, s.b)};
    auto out = s.run(in);
    for (int64_t i = 0; i < T * P; ++i) CHECK(out.data[i] == (double)(float)(in[0].data[i] * 3.0));
  }
  // ---- combineParallel: two thread levels and the scalar work between them become one level ---------------------
  {
    const int64_t T = 64;
    Scratch s("merged", {{T}, {T}}, {T});
    Value x = s.fn.getArgument(0), y = s.fn.getArgument(1);
    Value stage = s.alloc({T}, MemorySpace::shared), cell = s.alloc({1}, MemorySpace::shared);
    Value two = s.constant(2.0);
    Value zeroIdx = s.b.create<arith::ConstantIndexOp>(loc, 0).getResult();
    s.enterGrid();
    auto first = s.threads(T);
    {
      OpBuilder pb = OpBuilder::atBlockBegin(first.getBody());
      Value t = first.getIVs()[0];
      Value v = pb.create<AffineLoadOp>(loc, x, ValueRange({t})).getResult();
      pb.create<AffineStoreOp>(loc, pb.create<arith::MulFOp>(loc, v, two).getResult(), stage, ValueRange({t}));
    }
    s.b.setInsertionPointAfter(first.getOperation());
    Value head = s.b.create<AffineLoadOp>(loc, stage, ValueRange({zeroIdx})).getResult();
    s.b.create<AffineStoreOp>(loc, head, cell, ValueRange({zeroIdx}));
    auto second = s.threads(T);
    {
      OpBuilder pb = OpBuilder::atBlockBegin(second.getBody());
      Value t = second.getIVs()[0];
      Value v = pb.create<AffineLoadOp>(loc, stage, ValueRange({t})).getResult();
      Value c = pb.create<AffineLoadOp>(loc, cell, ValueRange({zeroIdx})).getResult();
      pb.create<AffineStoreOp>(loc, pb.create<arith::AddFOp>(loc, v, c).getResult(), y, ValueRange({t}));
    }
    s.finish(y);
    std::vector<HostTensor> in{randomTensor({T}, s.b), randomTensor({T}, s.b)};
    auto ref = s.run(in);
    auto merged = ln.combineParallel({first, second});
    CHECK(merged == first && s.f.verifies());
    int levels = 0, barriers = 0;
    s.fn->walk([&](Operation* o) { levels += o->getKind() == OpKind::AffineParallel; barriers += o->getKind() == OpKind::Barrier; }, WalkOrder::PreOrder);
    CHECK(levels == 2 && barriers == 2);   // the grid level and the merged thread level
    CHECK(maxDiff(ref, s.run(in)) == 0.0);
  }
  // ---- Gather::oneIndexLoad, BatchMatmul::threadLevelOneToTwo, FMHA::softmaxIR ------------------------------------
  {
    Scratch s("hoist", {{8}, {8}}, {8});
    Value idx = s.fn.getArgument(0), out = s.fn.getArgument(1);
    s.enterGrid();
    auto pal = s.threads(1);
    s.b.setInsertionPointToStart(pal.getBody());
    auto loop = s.loop(8, [&](OpBuilder& lb, Value i) {
      Value zero = lb.create<arith::ConstantIndexOp>(loc, 0).getResult();
      Value v = lb.create<AffineLoadOp>(loc, idx, ValueRange({zero})).getResult();
      lb.create<AffineStoreOp>(loc, v, out, ValueRange({i}));
    });
    s.finish(out);
    std::vector<HostTensor> in{randomTensor({8}, s.b), randomTensor({8}, s.b)};
    auto ref = s.run(in);
    GatherOptimizer().oneIndexLoad(loop, pal);
    int loadsInLoop = 0;
    for (auto& op : *loop.getBody()) loadsInLoop += isa<AffineLoadOp>(op);
    CHECK(loadsInLoop == 0 && s.f.verifies() && maxDiff(ref, s.run(in)) == 0.0);
  }
  {
    Scratch s("two_d", {{256}}, {256});
    s.enterGrid();
    auto pal = s.threads(256);
    s.finish(s.fn.getArgument(0));
    BatchMatmulOptimizer::batchMatmulConfig = {{"BLOCK_SIZE_N", 128}, {"THREAD_SIZE_N", 8}, {"BLOCK_SIZE_M", 128}, {"THREAD_SIZE_M", 8}};
    auto yx = BatchMatmulOptimizer().threadLevelOneToTwo(pal);
    CHECK(yx.size() == 2);
    auto ay = yx[0].getDefiningOp<AffineApplyOp>(), ax = yx[1].getDefiningOp<AffineApplyOp>();
    CHECK(ay && ax && ay.getAffineMap().evaluate({37})[0] == 37 / 16 && ax.getAffineMap().evaluate({37})[0] == 37 % 16);
  }
  {
    // two tiles of scores go through softmaxIR one after the other; the running statistics must be those of
    // the concatenated rows, and the factor the ratio of the two running maxima's exponentials
    const int64_t Br = 4, Bc = 8;
    FMHAOptimizer::fmhaConfig = {{"BrTileS", (int)Br}, {"BcTileS", (int)Bc}};
    Scratch s("online", {{Bc, Br}, {Bc, Br}}, {3, Br});
    Value t0 = s.fn.getArgument(0), t1 = s.fn.getArgument(1);
    Value rowMax = s.alloc({Br}, MemorySpace::local), rowSum = s.alloc({Br}, MemorySpace::local);
    Value smMax = s.alloc({Br}, MemorySpace::local), smSum = s.alloc({Br}, MemorySpace::local), smFac = s.alloc({Br}, MemorySpace::local);
    Value stats = s.alloc({3, Br}, MemorySpace::global);
    Value zero = s.constant(0.0), lowest = s.constant(-3.0e38);
    Rewriter::set_buffer(s.b, smMax, lowest);
    Rewriter::set_buffer(s.b, smSum, zero);
    Value tid = s.b.create<arith::ConstantIndexOp>(loc, 0).getResult();
    FMHAOptimizer fa;
    fa.softmaxIR(s.b, t0, rowMax, smMax, rowSum, smSum, smFac, zero, lowest, tid);
    fa.softmaxIR(s.b, t1, rowMax, smMax, rowSum, smSum, smFac, zero, lowest, tid);
    Value i0 = s.b.create<arith::ConstantIndexOp>(loc, 0).getResult(), i1 = s.b.create<arith::ConstantIndexOp>(loc, 1).getResult(),
          i2 = s.b.create<arith::ConstantIndexOp>(loc, 2).getResult();
    s.loop(Br, [&](OpBuilder& lb, Value r) {
      lb.create<AffineStoreOp>(loc, lb.create<AffineLoadOp>(loc, smMax, ValueRange({r})).getResult(), stats, ValueRange({i0, r}));
      lb.create<AffineStoreOp>(loc, lb.create<AffineLoadOp>(loc, smSum, ValueRange({r})).getResult(), stats, ValueRange({i1, r}));
      lb.create<AffineStoreOp>(loc, lb.create<AffineLoadOp>(loc, smFac, ValueRange({r})).getResult(), stats, ValueRange({i2, r}));
    });
    s.finish(stats);
    CHECK(s.f.verifies());
    std::vector<HostTensor> in{randomTensor({Bc, Br}, s.b), randomTensor({Bc, Br}, s.b)};
    for (auto& v : in[1].data) v = (double)(float)(v * 3.0);
    auto out = s.run(in);
    for (int64_t r = 0; r < Br; ++r) {
      double m0 = -1e30, m = -1e30, sum = 0;
      for (int64_t c = 0; c < Bc; ++c) m0 = std::max(m0, in[0].data[c * Br + r]);
      m = m0;
      for (int64_t c = 0; c < Bc; ++c) m = std::max(m, in[1].data[c * Br + r]);
      for (int t = 0; t < 2; ++t)
        for (int64_t c = 0; c < Bc; ++c) sum += std::exp(in[t].data[c * Br + r] - m);
      CHECK(out.data[0 * Br + r] == m);
      CHECK(std::fabs(out.data[1 * Br + r] - sum) < 1e-5 * sum);
      CHECK(std::fabs(out.data[2 * Br + r] - std::exp(m0 - m)) < 1e-6);
    }
  }
}

static void testFmhaTiledMaps() {
  // The 18 index maps of the tiled attention schedule (reference: src/Optimizer/Optimizer.cc:2201-2437), enumerated
  // over every thread and loop index: each copy covers its tile exactly once, what is loaded from (row, col) lands at
  // the transposed place, and the maps that must name the same element (fragment loads, statistics rows, the
  // probability tile's store and reload, the result store) agree.  The reference's layout (32-lane warps, Hd 64), the
  // same with 64-wide wavefronts, and Hd 128 (Br 64, Bc 128).
  OpBuilder b;
  struct Case { int warp, hd; };
  for (Case c : {Case{32, 64}, Case{64, 64}, Case{64, 128}, Case{32, 128}}) {
    FMHAOptimizer::fmhaConfig = {{"BLOCK_SIZE", 128}, {"HdxBr", 8192}, {"BrxBc", 8192}, {"WarpX_O", 2}, {"Slice", 8}, {"BrTileS", 8},
                                 {"BcTileS", 8}, {"BrTileO", 8}, {"HdTileO", 8}, {"Width", 4}, {"WARP_SIZE", c.warp}};
    int64_t Br = 0, Bc = 0;
    std::string why;
    CHECK(FMHAOptimizer::tiledLayout(2048, c.hd, Br, Bc, &why));
    CHECK(Br == 8192 / c.hd && Bc == 8192 / Br);
    FMHAOptimizer::fmhaConfig["Hd"] = c.hd;
    FMHAOptimizer::fmhaConfig["Br"] = (int)Br;
    FMHAOptimizer::fmhaConfig["Bc"] = (int)Bc;
    FMHAOptimizer fa;
    const int64_t T = 128, W = 4, Slice = 8, Hd = c.hd;
    auto M = [&](const char* name) { return fa.getAffineMap(name, b); };
    // global -> registers -> shared, Q and K slices (stored transposed), V slice (stored as it lies)
    struct Copy { const char *load, *store; int64_t rows, cols; bool transposed; };
    for (Copy cp : {Copy{"loadTileQ", "storeTileQ", Br, Slice, true}, Copy{"loadTileK", "storeTileK", Bc, Slice, true},
                    Copy{"loadTileV", "storeTileV", Slice, Hd, false}}) {
      std::vector<int> seen(cp.rows * cp.cols, 0), stored(cp.rows * cp.cols, 0);
      const int64_t iters = cp.rows * cp.cols / T / W;
      CHECK(iters >= 1);
      for (int64_t tid = 0; tid < T; ++tid)
        for (int64_t iv = 0; iv < iters; ++iv) {
          std::vector<int64_t> g;
          if (std::string(cp.load) == "loadTileQ") g = M(cp.load).evaluate({3, 5, 7, tid, 16, iv});          // (b, h, bx, tid, hd_outer, iv)
          else if (std::string(cp.load) == "loadTileK") g = M(cp.load).evaluate({3, 5, tid, 640, 16, iv});   // (b, h, tid, kv, hd_outer, iv)
          else g = M(cp.load).evaluate({3, 5, tid, 640, 24, iv});                                           // (b, h, tid, kv, bc_outer, iv)
          CHECK(g.size() == 4 && g[0] == 3 && g[1] == 5);
          int64_t row, col;
          if (std::string(cp.load) == "loadTileQ") { row = g[2] - 7 * Br; col = g[3] - 16; }
          else if (std::string(cp.load) == "loadTileK") { row = g[2] - 640; col = g[3] - 16; }
          else { row = g[2] - 640 - 24; col = g[3]; }
          CHECK(row >= 0 && row < cp.rows && col >= 0 && col + W <= cp.cols && col % W == 0);
          for (int64_t e = 0; e < W; ++e) {
            ++seen[row * cp.cols + col + e];
            std::vector<int64_t> sm = cp.transposed ? M(cp.store).evaluate({tid, iv, e}) : M(cp.store).evaluate({tid, iv});
            CHECK(sm.size() == 2);
            if (cp.transposed) CHECK(sm[0] == col + e && sm[1] == row);
            else CHECK(sm[0] == row && sm[1] == col);
            ++stored[row * cp.cols + col + e];
          }
        }
      for (int v : seen) CHECK(v == 1);
      for (int v : stored) CHECK(v == 1);
    }
    // the score tile [Bc][Br]: thread tid holds (bc, br), bc, br < 8
    {
      std::vector<int> seen(Bc * Br, 0);
      for (int64_t tid = 0; tid < T; ++tid)
        for (int64_t bc = 0; bc < 8; ++bc)
          for (int64_t br = 0; br < 8; ++br) {
            const int64_t key = M("bcIdxS").evaluate({tid, bc})[0], query = M("brIdxS").evaluate({tid, br})[0];
            CHECK(key >= 0 && key < Bc && query >= 0 && query < Br);
            ++seen[key * Br + query];
            // the fragments that feed tileS[bc][br] are K[key] and Q[query]
            CHECK(M("loadFragK").evaluate({tid, 5, bc / W}) == (std::vector<int64_t>{5, key - bc % W}));
            CHECK(M("loadFragQ").evaluate({tid, 5, br / W}) == (std::vector<int64_t>{5, query - br % W}));
            // and the probability goes to smP[key][query] (a Width-vector along the queries from br - br % W)
            CHECK(M("storeTileP").evaluate({tid, bc, br - br % W}) == (std::vector<int64_t>{key, query - br % W}));
            CHECK(M("readTileS").evaluate({bc, br}) == (std::vector<int64_t>{bc, br}));
          }
      for (int v : seen) CHECK(v == 1);
      // the threads that share a query differ in tid mod (Bc / 8) only: what the shuffles of softmaxIR assume
      const int64_t lanes = Bc / 8;
      for (int64_t tid = 0; tid < T; ++tid)
        for (int64_t br = 0; br < 8; ++br)
          CHECK(M("brIdxS").evaluate({tid, br}) == M("brIdxS").evaluate({tid - tid % lanes, br}));
    }
    // the output tile [Br][Hd]: thread tid holds (br, hd), br, hd < 8
    {
      std::vector<int> seen(Br * Hd, 0);
      for (int64_t tid = 0; tid < T; ++tid)
        for (int64_t br = 0; br < 8; ++br)
          for (int64_t hd = 0; hd < 8; ++hd) {
            auto o = M("storeTileO").evaluate({3, 5, 7, tid, br, hd - hd % W});       // (b, h, bx, tid, br, hd)
            CHECK(o.size() == 4 && o[0] == 3 && o[1] == 5);
            const int64_t query = o[2] - 7 * Br, d = o[3] + hd % W;
            CHECK(query >= 0 && query < Br && d >= 0 && d < Hd);
            ++seen[query * Hd + d];
            CHECK(M("brIdxO").evaluate({tid, br / W})[0] + br % W == query);
            CHECK(M("loadFactor").evaluate({tid, br / W})[0] + br % W == query);
            CHECK(M("loadFragP").evaluate({tid, 24, 3, br / W}) == (std::vector<int64_t>{27, query - br % W}));
            CHECK(M("loadFragV").evaluate({tid, 3, hd / W}) == (std::vector<int64_t>{3, d - hd % W}));
          }
      for (int v : seen) CHECK(v == 1);
    }
  }
  // shapes and configs that the layout rules turn down, each with its reason
  {
    FMHAOptimizer::fmhaConfig = {{"BLOCK_SIZE", 128}, {"HdxBr", 8192}, {"BrxBc", 8192}, {"WarpX_O", 2}, {"Slice", 8}, {"BrTileS", 8},
                                 {"BcTileS", 8}, {"BrTileO", 8}, {"HdTileO", 8}, {"Width", 4}, {"WARP_SIZE", 64}};
    int64_t Br, Bc;
    std::string why;
    CHECK(!FMHAOptimizer::tiledLayout(2000, 64, Br, Bc, &why) && !why.empty());     // no multiple of Br
    CHECK(!FMHAOptimizer::tiledLayout(2048, 96, Br, Bc, &why));                     // 8192 / 96
    CHECK(!FMHAOptimizer::tiledLayout(2048, 32, Br, Bc, &why));                     // Br 256, Bc 32: 4 lanes along the keys, 16 along ... rows do not add up
    FMHAOptimizer::fmhaConfig.erase("Slice");
    CHECK(!FMHAOptimizer::tiledLayout(2048, 64, Br, Bc, &why));
  }
  FMHAOptimizer::fmhaConfig.clear();
}

static void testEveryOperatorThroughBothLowerings() {
  // One graph per operator through optimize() and codegen(), once with the kernel families and once with the schedules
  // printed statement by statement; shapes that no tile divides among them (a ragged product, attention over 77
  // queries).  Judged by what must hold whatever the operator: the module verifies, every scheduled function gets a
  // kernel, the two lowerings agree on the kernel's arguments.  (Under the sanitizers this walks the optimizers, the
  // family emitters and the schedule emitter.)
  struct Case {
    const char* name;
    std::function<void(ComputeDAG&)> build;
    std::function<void(KernelCodeGenerator&)> prepare;
  };
  auto f32 = std::string{"float32"};
  std::vector<Case> cases = {
      {"matmul_ragged", [&](ComputeDAG& g) {
         auto A = g.create<PlaceHolder>(std::vector<int64_t>{100, 33}, f32);
         auto B = g.create<PlaceHolder>(std::vector<int64_t>{33, 77}, f32);
         g.create<Matmul>(A, B);
       }, [](KernelCodeGenerator& gen) { gen.opts.push_back(std::make_unique<MatmulOptimizer>()); }},
      {"layernorm_gelu", [&](ComputeDAG& g) {
         auto X = g.create<PlaceHolder>(std::vector<int64_t>{8, 1024}, f32);
         auto S = g.create<PlaceHolder>(std::vector<int64_t>{1024}, f32);
         auto B = g.create<PlaceHolder>(std::vector<int64_t>{1024}, f32);
         auto Y = g.create<LayerNorm>(X, S, B, 1, 1e-5f);
         g.create<ElementWise>(Y, "Gelu", MemorySpace::inplace);
       }, [](KernelCodeGenerator& gen) { gen.opts.push_back(std::make_unique<LayerNormOptimizer>()); }},
      {"softmax", [&](ComputeDAG& g) {
         auto X = g.create<PlaceHolder>(std::vector<int64_t>{16, 512}, f32);
         g.create<Softmax>(X, -1, MemorySpace::inplace);
       }, [](KernelCodeGenerator& gen) { gen.opts.push_back(std::make_unique<SoftmaxOptimizer>()); }},
      {"attention_77_queries", [&](ComputeDAG& g) {
         std::vector<int64_t> shp{2, 2, 77, 32};
         auto Q = g.create<PlaceHolder>(shp, f32), K = g.create<PlaceHolder>(shp, f32), V = g.create<PlaceHolder>(shp, f32);
         auto S = g.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
         auto P = g.create<Softmax>(S, -1, MemorySpace::inplace);
         g.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
       }, [](KernelCodeGenerator& gen) {
         gen.setConfigs("FMHA", {{{"BLOCK_SIZE", 32}, {"CAUSAL", 1}, {"SCALE_RSQRT_D", 1}}});
         gen.opts.push_back(std::make_unique<FMHAOptimizer>());
       }},
  };
  for (auto& c : cases) {
    std::vector<int> args;
    for (const char* lowering : {"families", "schedule"}) {
      KernelCodeGenerator gen("ROCm");
      gen.setLogMode(Log::Release);
      c.prepare(gen);
      auto graph = gen.createGraph(c.name);
      c.build(graph);
      auto module = gen.optimize(graph);
      CHECK(gen.setLowering(lowering));
      const std::string src = gen.codegen(module);
      if (gen.launchInfos().size() != 1) printf("  %s / %s: %zu kernels\n", c.name, lowering, gen.launchInfos().size());
      CHECK(gen.launchInfos().size() == 1 && gen.skippedFunctions().empty());
      const auto& info = gen.launchInfos()[0];
      CHECK(src.find("extern \"C\" __global__") != std::string::npos && info.numArgs >= 1);
      CHECK(std::string(lowering) != "schedule" || info.lowering.rfind("schedule", 0) == 0);
      args.push_back(info.numArgs);
    }
    CHECK(args[0] == args[1]);
  }
}

int main() {
  run("every_operator_both_lowerings", testEveryOperatorThroughBothLowerings);
  run("affine_algebra", testAffineAlgebra);
  run("ir_basics_and_analyzer", testIRBasics);
  run("identify_batch_matmul", testIdentifyBatchMatmul);
  run("split", testSplit);
  run("reorder_and_bufferize", testReorderPerfectAndImperfect);
  run("parallel", testParallelAndNormalise);
  run("read_write_vectorize_cache", testReadWriteVectorizeCache);
  run("if_simplification_and_unroll", testIfSimplificationAndUnroll);
  run("matmul_schedule_pipeline", testPipelineOnMatmul);
  run("hand_scripted_schedule_lowering", testHandScriptedScheduleGetsAKernel);
  run("swap_constant_loop_grid_to_block", testSwapLoopsConstantLoopAndGridToBlock);
  run("collapse_and_helpers", testCollapseAndHelpers);
  run("irregular_and_block_helpers", testIrregularMatAndBlockHelpers);
  run("usage_contract", testUsageContract);
  run("optimizer_helper_members", testOptimizerHelperMembers);
  run("fmha_tiled_maps", testFmhaTiledMaps);
  printf(failures ? "FAILED %d\n" : "ALL OK\n", failures);
  return failures ? 1 : 0;
}
