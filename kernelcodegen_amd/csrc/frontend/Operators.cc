// Frontend operator builders: each emits the operator's naive affine loop nest
// into a func.func tagged func.state = "cpu" and a func.call in the graph.
// Function names and nest semantics follow the reference
// (src/Frontend/Operators.cc); the code is organised around three helpers
// (describe the operand, open the function, close it with a call).
#include "Frontend/Operators.h"

#include <algorithm>
#include <numeric>

namespace KernelCodeGen {

using namespace mlir;

// --------------------------------------------------------------------------
// dtype names (reference: Operators.cc:5-29; bfloat16 / float8_e4m3 are new)
// --------------------------------------------------------------------------
Type getDType(OpBuilder& builder, const std::string& dtype) {
  if (dtype == "float32") return builder.getF32Type();
  if (dtype == "float64") return builder.getF64Type();
  if (dtype == "float16") return builder.getF16Type();
  if (dtype == "bfloat16") return builder.getBF16Type();
  if (dtype == "float8_e4m3") return builder.getF8E4M3FNType();
  if (dtype == "int64") return builder.getIntegerType(64);
  if (dtype == "int32") return builder.getIntegerType(32);
  if (dtype == "int16") return builder.getIntegerType(16);
  if (dtype == "index") return builder.getIndexType();
  if (dtype == "bool") return builder.getIntegerType(1);
  return nullptr;
}

std::string toStr(Type type) {
  if (!type) return "";
  if (type.isF16()) return "float16";
  if (type.isBF16()) return "bfloat16";
  if (type.isF32()) return "float32";
  if (type.isF64()) return "float64";
  if (type.isa<Float8E4M3FNType>()) return "float8_e4m3";
  if (type.isIndex()) return "index";
  if (auto it = type.dyn_cast<IntegerType>()) {
    switch (it.getWidth()) {
      case 1: return "bool";
      case 16: return "int16";
      case 32: return "int32";
      case 64: return "int64";
      default: return "";
    }
  }
  return "";
}

// --------------------------------------------------------------------------
// helpers
// --------------------------------------------------------------------------
namespace {

struct Operand {
  MemRefType type;
  std::vector<int64_t> shape;
  Type element;
  bool ok = false;
};

Operand describe(Value v, const char* opName, const char* role) {
  Operand d;
  if (!v) {
    llvm::errs() << opName << ": " << role << " is null.\n";
    return d;
  }
  d.type = v.getType().dyn_cast<MemRefType>();
  if (!d.type) {
    llvm::errs() << "Type of " << role << " of " << opName << " is not Memref.\n";
    return d;
  }
  d.shape = d.type.getShape().vec();
  d.element = d.type.getElementType();
  d.ok = true;
  return d;
}

std::string shapeSuffix(const std::vector<int64_t>& shape, size_t count) {
  std::string s;
  for (size_t i = 0; i < count; ++i) s += "_" + std::to_string(shape[i]);
  return s;
}

MemRefType globalMemref(const std::vector<int64_t>& shape, Type element, MemorySpace ms = MemorySpace::global) {
  return MemRefType::get(shape, element, {}, static_cast<int>(ms));
}

// Emits the call at `ip`, tags the function, returns the call's first result.
Value finishWithCall(OpBuilder& builder, OpBuilder::InsertPoint ip, func::FuncOp funcOp, ValueRange args) {
  builder.restoreInsertionPoint(ip);
  auto call = builder.create<func::CallOp>(builder.getUnknownLoc(), funcOp, args);
  funcOp->setAttr("func.state", builder.getStringAttr("cpu"));
  return call.getResult(0);
}

// A float operand narrower than the accumulate type is extended; equal types pass through.
Value widen(OpBuilder& b, Value v, Type to) {
  if (v.getType() == to) return v;
  return b.create<arith::ExtFOp>(b.getUnknownLoc(), to, v);
}

std::vector<int64_t> zeros(size_t n) { return std::vector<int64_t>(n, 0); }
std::vector<int64_t> ones(size_t n) { return std::vector<int64_t>(n, 1); }

// Nest of loops that thread ONE loop-carried value through every level; the
// innermost body returns the next value (reference: buildAffineLoopNest_,
// Operators.cc:31-67).  Returns the outermost loop.
AffineForOp buildReductionNest(OpBuilder& builder, Location loc, const std::vector<int64_t>& ubs, Value init,
                               const loopfunc& body) {
  OpBuilder::InsertionGuard guard(builder);
  std::vector<Value> ivs;
  AffineForOp outermost;
  std::function<Value(size_t, Value)> emitLevel = [&](size_t level, Value carried) -> Value {
    AffineForOp loop = builder.create<AffineForOp>(
        loc, 0, ubs[level], 1, ValueRange({carried}),
        [&](OpBuilder& nested, Location nestedLoc, Value iv, ValueRange iterArgs) {
          ivs.push_back(iv);
          Value next;
          if (level + 1 == ubs.size()) next = body(nested, nestedLoc, ValueRange(ivs), iterArgs);
          else next = emitLevel(level + 1, iterArgs[0]);
          nested.create<AffineYieldOp>(nestedLoc, ValueRange({next}));
          ivs.pop_back();
        });
    if (level == 0) outermost = loop;
    return loop.getResult(0);
  };
  emitLevel(0, init);
  return outermost;
}

// Indices of a tensor broadcast against `ivs` by trailing-dimension match:
// a size-1 (or mismatching) dimension reads index `zero`.
std::vector<Value> broadcastIndices(const std::vector<int64_t>& shape, const std::vector<int64_t>& full,
                                    ValueRange ivs, Value zero) {
  std::vector<Value> idx(shape.size());
  for (size_t i = 0; i < shape.size(); ++i) {
    const size_t s = shape.size() - 1 - i, f = full.size() - 1 - i;
    idx[s] = (shape[s] == full[f]) ? ivs[f] : zero;
  }
  return idx;
}

}  // namespace

// --------------------------------------------------------------------------
// buildFuction [sic] (reference: Operators.cc:69-110)
// --------------------------------------------------------------------------
func::FuncOp buildFuction(ModuleOp module, OpBuilder& builder, const std::string& funcName,
                          const std::vector<Type>& inputsTypes, const std::vector<Type>& outputsTypes) {
  func::FuncOp found;
  module.walk<WalkOrder::PreOrder>([&](func::FuncOp f) {
    if (!found && f.getSymName() == funcName) found = f;
  });
  if (found) return found;

  builder.setInsertionPointToStart(module.getBody());
  auto type = builder.getFunctionType(TypeRange(inputsTypes), TypeRange(outputsTypes));
  auto funcOp = builder.create<func::FuncOp>(builder.getUnknownLoc(), StringRef(funcName), type);
  Block& entry = funcOp.getBody().emplaceBlock();
  for (Type t : inputsTypes) entry.addArgument(t, builder.getUnknownLoc());
  return funcOp;
}

// --------------------------------------------------------------------------
// PlaceHolder (reference: Operators.cc:112-118)
// --------------------------------------------------------------------------
Value PlaceHolder::build(ComputeDAG* graph, const std::vector<int64_t>& shapes, const std::string& dtype) {
  OpBuilder& builder = graph->builder;
  Type element = getDType(builder, dtype);
  if (!element) {
    llvm::errs() << "PlaceHolder: unknown dtype \"" << dtype << "\".\n";
    return nullptr;
  }
  for (auto d : shapes)
    if (d <= 0) {
      llvm::errs() << "PlaceHolder: dimensions must be positive.\n";
      return nullptr;
    }
  return builder.create<memref::AllocOp>(builder.getUnknownLoc(), globalMemref(shapes, element)).getResult();
}

// --------------------------------------------------------------------------
// Matmul (reference: Operators.cc:120-220): C[i,j] = sum_k A[i,k] * B[k,j],
// accumulator starts at 0, mulf then addf, C allocated inside the function.
// --------------------------------------------------------------------------
namespace {
// A per-tensor scale of a quantised product: a placeholder of one fp32 value.
bool isScale(Value v, const char* op) {
  auto type = v ? v.getType().dyn_cast<MemRefType>() : MemRefType();
  if (!type || type.getNumElements() != 1 || !type.getElementType().isF32()) {
    llvm::errs() << op << ": a scale is a float32 placeholder of one element.\n";
    return false;
  }
  return true;
}
// sum * (scaleA[0] * scaleB[0]), the scales read at index 0 of every dimension
Value applyScales(OpBuilder& nb, Location loc, Value sum, Value scaleA, Value scaleB) {
  auto at0 = [&](Value memref) {
    const int64_t rank = memref.getType().cast<MemRefType>().getRank();
    std::vector<AffineExpr> zeros(rank, getAffineConstantExpr(0));
    return nb.create<AffineLoadOp>(loc, memref, AffineMap::get(0, 0, ArrayRef<AffineExpr>(zeros)), ValueRange({})).getResult();
  };
  Value sa = at0(scaleA), sb = at0(scaleB);
  if (sum.getType() != sa.getType()) {
    // the scales are fp32; a product in another type takes them in its own
    sa = sum.getType().getIntOrFloatBitWidth() < 32 ? nb.create<arith::TruncFOp>(loc, sum.getType(), sa).getResult()
                                                    : nb.create<arith::ExtFOp>(loc, sum.getType(), sa).getResult();
    sb = sum.getType().getIntOrFloatBitWidth() < 32 ? nb.create<arith::TruncFOp>(loc, sum.getType(), sb).getResult()
                                                    : nb.create<arith::ExtFOp>(loc, sum.getType(), sb).getResult();
  }
  Value both = nb.create<arith::MulFOp>(loc, sa, sb).getResult();
  return nb.create<arith::MulFOp>(loc, sum, both).getResult();
}
Value buildMatmul(ComputeDAG* graph, Value A, Value B, Value scaleA, Value scaleB, const std::string& dtype_);
Value buildBatchedMatmul(ComputeDAG* graph, Value A, Layout layoutA, Value B, Layout layoutB, Value scaleA, Value scaleB,
                         const std::string& dtype_);
}  // namespace

Value Matmul::build(ComputeDAG* graph, Value A, Value B, const std::string& dtype_) {
  return buildMatmul(graph, A, B, nullptr, nullptr, dtype_);
}
Value Matmul::build(ComputeDAG* graph, Value A, Value B, Value scaleA, Value scaleB, const std::string& dtype_) {
  if (!isScale(scaleA, "Matmul") || !isScale(scaleB, "Matmul")) return nullptr;
  return buildMatmul(graph, A, B, scaleA, scaleB, dtype_);
}

namespace {
Value buildMatmul(ComputeDAG* graph, Value A, Value B, Value scaleA, Value scaleB, const std::string& dtype_) {
  const bool scaled = (bool)scaleA;
  OpBuilder& builder = graph->builder;
  Operand a = describe(A, "Matmul", "left operand"), b = describe(B, "Matmul", "right operand");
  if (!a.ok || !b.ok) return nullptr;
  if (a.shape.size() != 2 || b.shape.size() != 2) {
    llvm::errs() << "Matmul needs two 2-d operands.\n";
    return nullptr;
  }
  const int64_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
  if (k != b.shape[0]) {
    llvm::errs() << "Can't apply Matmul Operation due to imcompatible K-dim.\n";
    return nullptr;
  }
  const std::string dtype = dtype_.empty() ? toStr(a.element) : dtype_;
  Type acc = getDType(builder, dtype);
  if (!acc || !acc.isFloat()) {
    llvm::errs() << "Matmul: unsupported dtype \"" << dtype << "\".\n";
    return nullptr;
  }
  const std::string funcName = "Matmul_m" + std::to_string(m) + "n" + std::to_string(n) + "k" + std::to_string(k) + (scaled ? "_scaled" : "");
  MemRefType typeC = globalMemref({m, n}, acc);

  auto ip = builder.saveInsertionPoint();
  std::vector<Type> argTypes{a.type, b.type};
  std::vector<Value> callArgs{A, B};
  if (scaled) {
    argTypes.push_back(scaleA.getType()); argTypes.push_back(scaleB.getType());
    callArgs.push_back(scaleA); callArgs.push_back(scaleB);
  }
  auto funcOp = buildFuction(graph->module, builder, funcName, argTypes, {typeC});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, callArgs);  // already built for this shape
  if (scaled) funcOp->setAttr("kcg.scales", builder.getI64IntegerAttr(2));   // position of the first scale argument

  builder.setInsertionPointToStart(&body);
  Value argA = body.getArgument(0), argB = body.getArgument(1);
  Value C = builder.create<memref::AllocOp>(builder.getUnknownLoc(), typeC).getResult();
  buildAffineLoopNest(builder, builder.getUnknownLoc(), {0, 0}, {m, n}, {1, 1},
    [&](OpBuilder& nb, Location loc, ValueRange ivs) {
      Value i = ivs[0], j = ivs[1];
      Value zero = nb.create<arith::ConstantOp>(loc, nb.getFloatAttr(acc, 0));
      auto kLoop = nb.create<AffineForOp>(loc, 0, k, 1, ValueRange({zero}),
        [&](OpBuilder& kb, Location kloc, Value kk, ValueRange iterArgs) {
          Value va = widen(kb, kb.create<AffineLoadOp>(kloc, argA, ValueRange({i, kk})), acc);
          Value vb = widen(kb, kb.create<AffineLoadOp>(kloc, argB, ValueRange({kk, j})), acc);
          Value mul = kb.create<arith::MulFOp>(kloc, va, vb);
          Value add = kb.create<arith::AddFOp>(kloc, mul, iterArgs[0]);
          kb.create<AffineYieldOp>(kloc, ValueRange({add}));
        });
      Value result = kLoop.getResult(0);
      if (scaled) result = applyScales(nb, loc, result, body.getArgument(2), body.getArgument(3));
      nb.create<AffineStoreOp>(loc, result, C, ValueRange({i, j}));
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({C}));
  return finishWithCall(builder, ip, funcOp, callArgs);
}
}  // namespace

// --------------------------------------------------------------------------
// Relu (reference: Operators.cc:222-289)
// --------------------------------------------------------------------------
Value Relu::build(ComputeDAG* graph, Value input, MemorySpace ms, const std::string& dtype_) {
  OpBuilder& builder = graph->builder;
  Operand in = describe(input, "Relu", "input");
  if (!in.ok) return nullptr;
  const std::string dtype = dtype_.empty() ? toStr(in.element) : dtype_;
  Type element = getDType(builder, dtype);
  if (!element || element != in.element || !element.isFloat()) {
    llvm::errs() << "Relu: dtype must be the input's float element type.\n";
    return nullptr;
  }
  const std::string funcName = "Relu_Elementwise" + shapeSuffix(in.shape, in.shape.size());
  auto ip = builder.saveInsertionPoint();
  MemRefType outType = ms == MemorySpace::inplace ? in.type : globalMemref(in.shape, element, ms);
  auto funcOp = buildFuction(graph->module, builder, funcName, {in.type}, {outType});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, {input});

  builder.setInsertionPointToStart(&body);
  Value arg = body.getArgument(0);
  Value out = ms == MemorySpace::inplace ? arg : builder.create<memref::AllocOp>(builder.getUnknownLoc(), outType).getResult();
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(in.shape.size()), in.shape, ones(in.shape.size()),
    [&](OpBuilder& nb, Location loc, ValueRange ivs) {
      Value zero = nb.create<arith::ConstantOp>(loc, nb.getFloatAttr(element, 0));
      Value x = nb.create<AffineLoadOp>(loc, arg, ivs);
      Value y = nb.create<arith::MaxFOp>(loc, zero, x);
      nb.create<AffineStoreOp>(loc, y, out, ivs);
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({out}));
  return finishWithCall(builder, ip, funcOp, {input});
}

// --------------------------------------------------------------------------
// BatchedMatmul (reference: Operators.cc:291-457).  C is a PlaceHolder created
// next to B and passed as the third function argument.  A column-major A reads
// A[.., k, i]; the reference's nest reads A[.., k, j] there (Operators.cc:427-429),
// an indexing slip that is not reproduced.
// --------------------------------------------------------------------------
Value BatchedMatmul::build(ComputeDAG* graph, Value A, Layout layoutA, Value B, Layout layoutB, const std::string& dtype_) {
  return buildBatchedMatmul(graph, A, layoutA, B, layoutB, nullptr, nullptr, dtype_);
}
Value BatchedMatmul::build(ComputeDAG* graph, Value A, Layout layoutA, Value B, Layout layoutB, Value scaleA, Value scaleB,
                           const std::string& dtype_) {
  if (!isScale(scaleA, "BatchedMatmul") || !isScale(scaleB, "BatchedMatmul")) return nullptr;
  return buildBatchedMatmul(graph, A, layoutA, B, layoutB, scaleA, scaleB, dtype_);
}

namespace {
Value buildBatchedMatmul(ComputeDAG* graph, Value A, Layout layoutA, Value B, Layout layoutB, Value scaleA, Value scaleB,
                         const std::string& dtype_) {
  const bool scaled = (bool)scaleA;
  OpBuilder& builder = graph->builder;
  Operand a = describe(A, "BatchedMatmul", "left operand"), b = describe(B, "BatchedMatmul", "right operand");
  if (!a.ok || !b.ok) return nullptr;
  const size_t rank = a.shape.size();
  if (rank < 2) {
    llvm::errs() << "BatchedMatmul needs at least 2 dim but got " << rank << "\n";
    return nullptr;
  }
  if (b.shape.size() != rank) {
    llvm::errs() << "BatchedMatmul: A, B dim not matched.\n";
    return nullptr;
  }
  for (size_t i = 0; i + 2 < rank; ++i)
    if (a.shape[i] != b.shape[i]) {
      llvm::errs() << "BatchedMatmul: batch dims differ.\n";
      return nullptr;
    }
  const bool tA = layoutA == Layout::colMajor, tB = layoutB == Layout::colMajor;
  const int64_t m = tA ? a.shape[rank - 1] : a.shape[rank - 2];
  const int64_t k = tA ? a.shape[rank - 2] : a.shape[rank - 1];
  const int64_t n = tB ? b.shape[rank - 2] : b.shape[rank - 1];
  const int64_t k2 = tB ? b.shape[rank - 1] : b.shape[rank - 2];
  if (k != k2) {
    llvm::errs() << "Can't apply BatchedMatmul Operation due to imcompatible K-dim.\n";
    return nullptr;
  }
  const std::string dtype = dtype_.empty() ? toStr(a.element) : dtype_;
  Type acc = getDType(builder, dtype);
  if (!acc || !acc.isFloat()) {
    llvm::errs() << "BatchedMatmul: unsupported dtype \"" << dtype << "\".\n";
    return nullptr;
  }
  std::vector<int64_t> shapeC(a.shape.begin(), a.shape.end() - 2);
  shapeC.push_back(m);
  shapeC.push_back(n);

  Value C = graph->create<PlaceHolder>(shapeC, dtype);
  // an output buffer, not a graph input: hosts that bind inputs by position skip it
  C.getDefiningOp()->setAttr("kcg.result", builder.getUnitAttr());
  if (Operation* defB = B.getDefiningOp())
    if (defB->getBlock() == C.getDefiningOp()->getBlock()) C.getDefiningOp()->moveAfter(defB);

  std::string funcName = "BatchMatmul" + shapeSuffix(shapeC, rank - 2);
  funcName += "_m" + std::to_string(m) + "_n" + std::to_string(n) + "_k" + std::to_string(k) + "_";
  funcName += tA ? 'T' : 'N';
  funcName += tB ? 'T' : 'N';
  if (scaled) funcName += "_scaled";          // identifyBatchMatmul reads past this part

  MemRefType typeC = C.getType().cast<MemRefType>();
  auto ip = builder.saveInsertionPoint();
  std::vector<Type> argTypes{a.type, b.type, typeC};
  std::vector<Value> callArgs{A, B, C};
  if (scaled) {
    argTypes.push_back(scaleA.getType()); argTypes.push_back(scaleB.getType());
    callArgs.push_back(scaleA); callArgs.push_back(scaleB);
  }
  auto funcOp = buildFuction(graph->module, builder, funcName, argTypes, {typeC});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, callArgs);
  if (scaled) funcOp->setAttr("kcg.scales", builder.getI64IntegerAttr(3));   // position of the first scale argument

  builder.setInsertionPointToStart(&body);
  Value argA = body.getArgument(0), argB = body.getArgument(1), argC = body.getArgument(2);
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(rank), shapeC, ones(rank),
    [&](OpBuilder& nb, Location loc, ValueRange ivs) {
      Value i = ivs[rank - 2], j = ivs[rank - 1];
      std::vector<Value> batch(ivs.begin(), ivs.end() - 2);
      Value zero = nb.create<arith::ConstantOp>(loc, nb.getFloatAttr(acc, 0));
      auto kLoop = nb.create<AffineForOp>(loc, 0, k, 1, ValueRange({zero}),
        [&](OpBuilder& kb, Location kloc, Value kk, ValueRange iterArgs) {
          std::vector<Value> idxA = batch, idxB = batch;
          if (tA) { idxA.push_back(kk); idxA.push_back(i); } else { idxA.push_back(i); idxA.push_back(kk); }
          if (tB) { idxB.push_back(j); idxB.push_back(kk); } else { idxB.push_back(kk); idxB.push_back(j); }
          Value va = widen(kb, kb.create<AffineLoadOp>(kloc, argA, ValueRange(idxA)), acc);
          Value vb = widen(kb, kb.create<AffineLoadOp>(kloc, argB, ValueRange(idxB)), acc);
          Value mul = kb.create<arith::MulFOp>(kloc, va, vb);
          Value add = kb.create<arith::AddFOp>(kloc, mul, iterArgs[0]);
          kb.create<AffineYieldOp>(kloc, ValueRange({add}));
        });
      Value result = kLoop.getResult(0);
      if (scaled) result = applyScales(nb, loc, result, body.getArgument(3), body.getArgument(4));
      nb.create<AffineStoreOp>(loc, result, argC, ivs);
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({argC}));
  return finishWithCall(builder, ip, funcOp, callArgs);
}
}  // namespace

// Declared by the reference with an empty body (Operators.cc:459-460).
Value Transpose::build(ComputeDAG*, Value) {
  llvm::errs() << "Transpose is not implemented.\n";
  return nullptr;
}

// --------------------------------------------------------------------------
// Softmax over the last axis, in place (reference: Operators.cc:462-578):
// sum = sum_k exp(x[k]) without max subtraction, then x[k] = exp(x[k]) / sum.
// --------------------------------------------------------------------------
Value Softmax::build(ComputeDAG* graph, Value input, int axis, MemorySpace, const std::string& dtype_) {
  OpBuilder& builder = graph->builder;
  Operand in = describe(input, "Softmax", "input");
  if (!in.ok) return nullptr;
  const int rank = (int)in.shape.size();
  const int reduceAxis = axis < 0 ? axis + rank : axis;
  if (reduceAxis != rank - 1) {
    llvm::errs() << "At present, only support reduction on the last dim.\n";
    return nullptr;
  }
  const std::string dtype = dtype_.empty() ? toStr(in.element) : dtype_;
  Type element = getDType(builder, dtype);
  if (!element || element != in.element || !element.isFloat()) {
    llvm::errs() << "Softmax: dtype must be the input's float element type.\n";
    return nullptr;
  }
  const std::string funcName = "Softmax" + shapeSuffix(in.shape, rank) + "_axis" + std::to_string(reduceAxis);
  auto ip = builder.saveInsertionPoint();
  auto funcOp = buildFuction(graph->module, builder, funcName, {in.type}, {in.type});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, {input});

  builder.setInsertionPointToStart(&body);
  Value arg = body.getArgument(0);
  const int64_t cols = in.shape.back();
  std::vector<int64_t> outer(in.shape.begin(), in.shape.end() - 1);
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(outer.size()), outer, ones(outer.size()),
    [&](OpBuilder& nb, Location loc, ValueRange ivs) {
      Value zero = nb.create<arith::ConstantOp>(loc, nb.getFloatAttr(element, 0));
      auto sumLoop = nb.create<AffineForOp>(loc, 0, cols, 1, ValueRange({zero}),
        [&](OpBuilder& kb, Location kloc, Value kk, ValueRange iterArgs) {
          std::vector<Value> idx(ivs.begin(), ivs.end());
          idx.push_back(kk);
          Value x = kb.create<AffineLoadOp>(kloc, arg, ValueRange(idx));
          Value e = kb.create<math::ExpOp>(kloc, x);
          Value s = kb.create<arith::AddFOp>(kloc, e, iterArgs[0]);
          kb.create<AffineYieldOp>(kloc, ValueRange({s}));
        });
      nb.create<AffineForOp>(loc, 0, cols, 1, ValueRange({}),
        [&](OpBuilder& eb, Location eloc, Value kk, ValueRange) {
          std::vector<Value> idx(ivs.begin(), ivs.end());
          idx.push_back(kk);
          Value x = eb.create<AffineLoadOp>(eloc, arg, ValueRange(idx));
          Value e = eb.create<math::ExpOp>(eloc, x);
          Value p = eb.create<arith::DivFOp>(eloc, e, sumLoop.getResult(0));
          eb.create<AffineStoreOp>(eloc, p, arg, ValueRange(idx));
          eb.create<AffineYieldOp>(eloc);
        });
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({arg}));
  return finishWithCall(builder, ip, funcOp, {input});
}

// --------------------------------------------------------------------------
// Binary with trailing-dimension broadcast (reference: Operators.cc:580-889)
// --------------------------------------------------------------------------
Value Binary::add(OpBuilder& b, Value x, Value y) { return b.create<arith::AddFOp>(b.getUnknownLoc(), x, y); }
Value Binary::mul(OpBuilder& b, Value x, Value y) { return b.create<arith::MulFOp>(b.getUnknownLoc(), x, y); }
Value Binary::div(OpBuilder& b, Value x, Value y) { return b.create<arith::DivFOp>(b.getUnknownLoc(), x, y); }
Value Binary::sub(OpBuilder& b, Value x, Value y) { return b.create<arith::SubFOp>(b.getUnknownLoc(), x, y); }
Value Binary::pow(OpBuilder& b, Value x, Value y) { return b.create<math::PowFOp>(b.getUnknownLoc(), x, y); }
Value Binary::equal(OpBuilder& b, Value x, Value y) {
  return b.create<arith::CmpFOp>(b.getUnknownLoc(), arith::CmpFPredicate::OEQ, x, y);
}
Value Binary::greater(OpBuilder& b, Value x, Value y) {
  return b.create<arith::CmpFOp>(b.getUnknownLoc(), arith::CmpFPredicate::OGT, x, y);
}
std::map<std::string, std::function<Value(OpBuilder&, Value, Value)>> Binary::operationMap = {
    {"Add", &Binary::add}, {"Mul", &Binary::mul}, {"Div", &Binary::div}, {"Sub", &Binary::sub},
    {"Pow", &Binary::pow}, {"Equal", &Binary::equal}, {"Greater", &Binary::greater}};

Value Binary::build(ComputeDAG* graph, Value A, Value B, std::string operation, MemorySpace ms, const std::string& dtype_) {
  OpBuilder& builder = graph->builder;
  Operand a = describe(A, operation.c_str(), "left operand"), b = describe(B, operation.c_str(), "right operand");
  if (!a.ok || !b.ok) return nullptr;
  auto opIt = operationMap.find(operation);
  if (opIt == operationMap.end()) {
    llvm::errs() << "Binary: unknown operation \"" << operation << "\".\n";
    return nullptr;
  }
  const std::string dtype = dtype_.empty() ? toStr(a.element) : dtype_;
  Type element = getDType(builder, dtype);
  if (!element) return nullptr;
  const size_t rank = std::max(a.shape.size(), b.shape.size());
  std::vector<int64_t> full(rank, 1);
  bool broadcast = false;
  for (size_t i = 0; i < rank; ++i) {
    const int64_t da = i < a.shape.size() ? a.shape[a.shape.size() - 1 - i] : 1;
    const int64_t db = i < b.shape.size() ? b.shape[b.shape.size() - 1 - i] : 1;
    if (da != db && da != 1 && db != 1) {
      llvm::errs() << "dim not equal\n";
      return nullptr;
    }
    if (da != db) broadcast = true;
    full[rank - 1 - i] = std::max(da, db);
  }
  if (operation == "Equal" || operation == "Greater") element = builder.getIntegerType(1);
  std::string funcName = operation + "_Binary" + shapeSuffix(a.shape, a.shape.size()) + "_" + operation +
                         shapeSuffix(b.shape, b.shape.size());
  MemRefType typeC = ms == MemorySpace::inplace ? a.type : globalMemref(full, element, ms);
  auto ip = builder.saveInsertionPoint();
  auto funcOp = buildFuction(graph->module, builder, funcName, {a.type, b.type}, {typeC});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, {A, B});

  builder.setInsertionPointToStart(&body);
  Value argA = body.getArgument(0), argB = body.getArgument(1);
  Value out = ms == MemorySpace::inplace ? argA : builder.create<memref::AllocOp>(builder.getUnknownLoc(), typeC).getResult();
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(rank), full, ones(rank),
    [&](OpBuilder& nb, Location loc, ValueRange ivs) {
      Value zero;
      if (broadcast || a.shape.size() != b.shape.size()) zero = nb.create<arith::ConstantIndexOp>(loc, 0);
      Value x = nb.create<AffineLoadOp>(loc, argA, ValueRange(broadcastIndices(a.shape, full, ivs, zero)));
      Value y = nb.create<AffineLoadOp>(loc, argB, ValueRange(broadcastIndices(b.shape, full, ivs, zero)));
      Value r = opIt->second(nb, x, y);
      nb.create<AffineStoreOp>(loc, r, out, ivs);
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({out}));
  return finishWithCall(builder, ip, funcOp, {A, B});
}

// --------------------------------------------------------------------------
// ElementWise (reference: Operators.cc:960-1074).  GELU is the tanh form with
// the constants 0.797884 and 0.044715, in the reference's operation order.
// --------------------------------------------------------------------------
Value ElementWise::tanh(OpBuilder& b, Value x, Type) { return b.create<math::TanhOp>(b.getUnknownLoc(), x); }
Value ElementWise::sqrt(OpBuilder& b, Value x, Type) { return b.create<math::SqrtOp>(b.getUnknownLoc(), x); }
Value ElementWise::log(OpBuilder& b, Value x, Type) { return b.create<math::LogOp>(b.getUnknownLoc(), x); }
Value ElementWise::relu(OpBuilder& b, Value x, Type type) {
  Value zero = b.create<arith::ConstantOp>(b.getUnknownLoc(), b.getFloatAttr(type, 0));
  return b.create<arith::MaxFOp>(b.getUnknownLoc(), zero, x);
}
Value ElementWise::cast(OpBuilder& b, Value x, Type type) { return b.create<arith::BitcastOp>(b.getUnknownLoc(), type, x); }
Value ElementWise::gelu(OpBuilder& b, Value x, Type type) {
  Location loc = b.getUnknownLoc();
  auto cst = [&](double v) -> Value { return b.create<arith::ConstantOp>(loc, b.getFloatAttr(type, v)); };
  Value one = cst(1.0), half = cst(0.5), c0 = cst(0.797884), c1 = cst(0.044715);
  Value t1 = b.create<arith::MulFOp>(loc, x, half);
  Value t2 = b.create<arith::MulFOp>(loc, x, x);
  Value t3 = b.create<arith::MulFOp>(loc, x, t2);
  Value t4 = b.create<arith::MulFOp>(loc, c1, t3);
  Value t5 = b.create<arith::AddFOp>(loc, t4, x);
  Value t6 = b.create<arith::MulFOp>(loc, c0, t5);
  Value t7 = b.create<math::TanhOp>(loc, t6);
  Value t8 = b.create<arith::AddFOp>(loc, t7, one);
  return b.create<arith::MulFOp>(loc, t1, t8);
}
std::map<std::string, std::function<Value(OpBuilder&, Value, Type)>> ElementWise::operationMap = {
    {"Tanh", &ElementWise::tanh}, {"Sqrt", &ElementWise::sqrt}, {"Log", &ElementWise::log},
    {"Relu", &ElementWise::relu}, {"Cast", &ElementWise::cast}, {"Gelu", &ElementWise::gelu}};

Value ElementWise::build(ComputeDAG* graph, Value input, std::string operation, MemorySpace ms, const std::string& dtype_) {
  OpBuilder& builder = graph->builder;
  Operand in = describe(input, operation.c_str(), "operand");
  if (!in.ok) return nullptr;
  auto opIt = operationMap.find(operation);
  if (opIt == operationMap.end()) {
    llvm::errs() << "ElementWise: unknown operation \"" << operation << "\".\n";
    return nullptr;
  }
  const std::string dtype = dtype_.empty() ? toStr(in.element) : dtype_;
  Type element = getDType(builder, dtype);
  if (!element) {
    llvm::errs() << "ElementWise: unknown dtype \"" << dtype << "\".\n";
    return nullptr;
  }
  if (operation != "Cast" && element != in.element) {
    llvm::errs() << "ElementWise: only Cast changes the element type.\n";
    return nullptr;
  }
  if (operation == "Cast" && ms == MemorySpace::inplace) {
    llvm::errs() << "ElementWise: Cast needs MemorySpace::global.\n";
    return nullptr;
  }
  const std::string funcName = operation + "_Elementwise" + shapeSuffix(in.shape, in.shape.size());
  MemRefType outType = ms == MemorySpace::inplace ? in.type : globalMemref(in.shape, element, ms);
  auto ip = builder.saveInsertionPoint();
  auto funcOp = buildFuction(graph->module, builder, funcName, {in.type}, {outType});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, {input});

  builder.setInsertionPointToStart(&body);
  Value arg = body.getArgument(0);
  Value out = ms == MemorySpace::inplace ? arg : builder.create<memref::AllocOp>(builder.getUnknownLoc(), outType).getResult();
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(in.shape.size()), in.shape, ones(in.shape.size()),
    [&](OpBuilder& nb, Location loc, ValueRange ivs) {
      Value x = nb.create<AffineLoadOp>(loc, arg, ivs);
      Value y = opIt->second(nb, x, element);
      nb.create<AffineStoreOp>(loc, y, out, ivs);
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({out}));
  return finishWithCall(builder, ip, funcOp, {input});
}

// --------------------------------------------------------------------------
// LayerNorm (reference: Operators.cc:1076-1251).  Dims before `axis` index the
// groups, dims from `axis` on are normalised together:
//   mean = sum(x)/N;  d = x - mean (stored to the output);  var = sum(d*d)/N;
//   den = sqrt(var + eps);  y = scale * (d / den) + bias.
// scale and bias broadcast over the input by trailing-dimension match.
// --------------------------------------------------------------------------
Value LayerNorm::build(ComputeDAG* graph, Value input, Value scale, Value bias, int64_t axis, const float& eps,
                       MemorySpace ms, const std::string& dtype_) {
  OpBuilder& builder = graph->builder;
  Operand in = describe(input, "LayerNorm", "operand"), sc = describe(scale, "LayerNorm", "scale"),
          bi = describe(bias, "LayerNorm", "bias");
  if (!in.ok || !sc.ok || !bi.ok) return nullptr;
  const int64_t rank = (int64_t)in.shape.size();
  auto broadcastable = [&](const Operand& t, const char* what) {
    if ((int64_t)t.shape.size() > rank) { llvm::errs() << what << " has more dims than the input.\n"; return false; }
    for (size_t i = 0; i < t.shape.size(); ++i) {
      const int64_t d = t.shape[t.shape.size() - 1 - i];
      if (d != in.shape[rank - 1 - i] && d != 1) { llvm::errs() << what << " dim is not equal.\n"; return false; }
    }
    return true;
  };
  if (!broadcastable(sc, "scale") || !broadcastable(bi, "bias")) return nullptr;
  if (axis >= rank || axis <= -rank) {
    llvm::errs() << "axis is out of bounds for array of dimension.\n";
    return nullptr;
  }
  if (axis < 0) axis += rank;
  const std::string dtype = dtype_.empty() ? toStr(in.element) : dtype_;
  Type element = getDType(builder, dtype);
  if (!element || element != in.element || !element.isFloat()) {
    llvm::errs() << "LayerNorm: dtype must be the input's float element type.\n";
    return nullptr;
  }
  std::vector<int64_t> outerShape(in.shape.begin(), in.shape.begin() + axis);
  std::vector<int64_t> innerShape(in.shape.begin() + axis, in.shape.end());
  const int64_t count = std::accumulate(innerShape.begin(), innerShape.end(), (int64_t)1, std::multiplies<int64_t>());

  const std::string funcName = "LayerNorm" + shapeSuffix(in.shape, in.shape.size()) + "_axis_" + std::to_string(axis);
  auto ip = builder.saveInsertionPoint();
  auto funcOp = buildFuction(graph->module, builder, funcName, {in.type, sc.type, bi.type}, {in.type});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, {input, scale, bias});

  builder.setInsertionPointToStart(&body);
  Value argX = body.getArgument(0), argS = body.getArgument(1), argB = body.getArgument(2);
  Value out = ms == MemorySpace::inplace
                  ? argX
                  : builder.create<memref::AllocOp>(builder.getUnknownLoc(), globalMemref(in.shape, element, ms)).getResult();
  auto fullIndex = [](ValueRange outer, ValueRange inner) {
    std::vector<Value> idx(outer.begin(), outer.end());
    idx.insert(idx.end(), inner.begin(), inner.end());
    return idx;
  };
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(outerShape.size()), outerShape, ones(outerShape.size()),
    [&](OpBuilder& ob, Location loc, ValueRange outerIvs) {
      Value countF = ob.create<arith::ConstantOp>(loc, ob.getFloatAttr(element, (double)count));
      Value epsF = ob.create<arith::ConstantOp>(loc, ob.getFloatAttr(element, eps));
      Value zeroF = ob.create<arith::ConstantOp>(loc, ob.getFloatAttr(element, 0));
      // pass 1: sum
      AffineForOp sumNest = buildReductionNest(ob, loc, innerShape, zeroF,
        [&](OpBuilder& nb, Location nloc, ValueRange innerIvs, ValueRange iterArgs) -> Value {
          Value x = nb.create<AffineLoadOp>(nloc, argX, ValueRange(fullIndex(outerIvs, innerIvs)));
          return nb.create<arith::AddFOp>(nloc, x, iterArgs[0]);
        });
      ob.setInsertionPointAfter(sumNest);
      Value mean = ob.create<arith::DivFOp>(loc, sumNest.getResult(0), countF);
      // pass 2: centre, store, sum of squares
      AffineForOp varNest = buildReductionNest(ob, loc, innerShape, zeroF,
        [&](OpBuilder& nb, Location nloc, ValueRange innerIvs, ValueRange iterArgs) -> Value {
          auto idx = fullIndex(outerIvs, innerIvs);
          Value x = nb.create<AffineLoadOp>(nloc, argX, ValueRange(idx));
          Value d = nb.create<arith::SubFOp>(nloc, x, mean);
          nb.create<AffineStoreOp>(nloc, d, out, ValueRange(idx));
          Value sq = nb.create<arith::MulFOp>(nloc, d, d);
          return nb.create<arith::AddFOp>(nloc, sq, iterArgs[0]);
        });
      ob.setInsertionPointAfter(varNest);
      Value var = ob.create<arith::DivFOp>(loc, varNest.getResult(0), countF);
      Value varEps = ob.create<arith::AddFOp>(loc, var, epsF);
      Value den = ob.create<math::SqrtOp>(loc, varEps);
      // pass 3: normalise, scale, shift
      buildAffineLoopNest(ob, loc, zeros(innerShape.size()), innerShape, ones(innerShape.size()),
        [&](OpBuilder& nb, Location nloc, ValueRange innerIvs) {
          auto idx = fullIndex(outerIvs, innerIvs);
          Value zeroIdx;
          auto needsZero = [&](const Operand& t) {
            for (size_t i = 0; i < t.shape.size(); ++i)
              if (t.shape[t.shape.size() - 1 - i] != in.shape[rank - 1 - i]) return true;
            return false;
          };
          if (needsZero(sc) || needsZero(bi)) zeroIdx = nb.create<arith::ConstantIndexOp>(nloc, 0);
          Value d = nb.create<AffineLoadOp>(nloc, out, ValueRange(idx));
          Value g = nb.create<AffineLoadOp>(nloc, argS, ValueRange(broadcastIndices(sc.shape, in.shape, ValueRange(idx), zeroIdx)));
          Value b = nb.create<AffineLoadOp>(nloc, argB, ValueRange(broadcastIndices(bi.shape, in.shape, ValueRange(idx), zeroIdx)));
          Value q = nb.create<arith::DivFOp>(nloc, d, den);
          Value m = nb.create<arith::MulFOp>(nloc, g, q);
          Value y = nb.create<arith::AddFOp>(nloc, m, b);
          nb.create<AffineStoreOp>(nloc, y, out, ValueRange(idx));
        });
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({out}));
  return finishWithCall(builder, ip, funcOp, {input, scale, bias});
}

// --------------------------------------------------------------------------
// Gather (reference: Operators.cc:1253-1352).  The dimension `axis` of the input is
// replaced by the dimensions of `indices` (dropped altogether for a single index,
// shape {1}):  out[o.., i.., r..] = in[o.., indices[i..], r..].
// The index is read with affine.load and used by a memref.load, the one place
// where the IR addresses memory with a loaded value.
// --------------------------------------------------------------------------
Value Gather::build(ComputeDAG* graph, Value input, Value indices, const std::int64_t& axis_, const std::string& dtype_) {
  OpBuilder& builder = graph->builder;
  Operand in = describe(input, "Gather", "input"), ix = describe(indices, "Gather", "indices");
  if (!in.ok || !ix.ok) return nullptr;
  const int64_t rank = (int64_t)in.shape.size();
  int64_t axis = axis_;
  if (axis >= rank || axis < -rank) {
    llvm::errs() << "Can't apply Gather Operation due to axis is greater than shape of input.\n";
    return nullptr;
  }
  if (axis < 0) axis += rank;
  if (!ix.element.isIndex()) {
    llvm::errs() << "Gather: indices must have dtype \"index\".\n";
    return nullptr;
  }
  const std::string dtype = dtype_.empty() ? toStr(in.element) : dtype_;
  Type element = getDType(builder, dtype);
  if (!element || element != in.element) {
    llvm::errs() << "Gather: dtype must be the input's element type.\n";
    return nullptr;
  }
  const bool single = ix.shape.size() == 1 && ix.shape[0] == 1;
  std::vector<int64_t> outShape(in.shape.begin(), in.shape.begin() + axis);
  if (!single) outShape.insert(outShape.end(), ix.shape.begin(), ix.shape.end());
  outShape.insert(outShape.end(), in.shape.begin() + axis + 1, in.shape.end());
  if (outShape.empty()) {
    llvm::errs() << "Gather: a single index into a 1-d input leaves no output dimension.\n";
    return nullptr;
  }

  std::string funcName = "Gather";
  for (auto d : in.shape) funcName += "_" + std::to_string(d);
  funcName += "_indices";
  for (auto d : ix.shape) funcName += "_" + std::to_string(d);
  funcName += "_axis_" + std::to_string(axis);

  auto ip = builder.saveInsertionPoint();
  MemRefType outType = globalMemref(outShape, element);
  auto funcOp = buildFuction(graph->module, builder, funcName, {in.type, ix.type}, {outType});
  Block& body = funcOp.front();
  if (!body.empty()) return finishWithCall(builder, ip, funcOp, {input, indices});

  builder.setInsertionPointToStart(&body);
  Value argX = body.getArgument(0), argI = body.getArgument(1);
  Value out = builder.create<memref::AllocOp>(builder.getUnknownLoc(), outType).getResult();
  const size_t idxRank = single ? 0 : ix.shape.size();
  buildAffineLoopNest(builder, builder.getUnknownLoc(), zeros(outShape.size()), outShape, ones(outShape.size()),
    [&](OpBuilder& nb, Location loc, ValueRange ivRange) {
      const std::vector<Value> ivs(ivRange.begin(), ivRange.end());
      std::vector<Value> where;      // position in `indices`
      if (single) where.push_back(nb.create<arith::ConstantIndexOp>(loc, 0));
      else where.assign(ivs.begin() + axis, ivs.begin() + axis + idxRank);
      Value index = nb.create<AffineLoadOp>(loc, argI, ValueRange(where));
      std::vector<Value> from(ivs.begin(), ivs.begin() + axis);
      from.push_back(index);
      from.insert(from.end(), ivs.begin() + axis + idxRank, ivs.end());
      Value v = nb.create<memref::LoadOp>(loc, argX, ValueRange(from)).getResult();
      nb.create<AffineStoreOp>(loc, v, out, ValueRange(ivs));
    });
  builder.create<func::ReturnOp>(builder.getUnknownLoc(), ValueRange({out}));
  return finishWithCall(builder, ip, funcOp, {input, indices});
}

}  // namespace KernelCodeGen
