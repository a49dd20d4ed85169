// Statement-by-statement lowering of a scheduled function to a gfx950 kernel.
//
// The kernel families of KernelFamilies.cc replace a recognised operator by a hand-shaped kernel and read only the
// tile sizes of its schedule.  This file is the other lowering, the one the reference's backend is
// (src/Backend/CUDA.cc:61-1184: one C statement per affine operation): it prints what the function body says.  The
// outer affine.parallel becomes the grid, the inner one the workgroup, memref.alloc in memory space 2 an LDS array and
// in space 3 a per-lane array that full unrolling turns into registers, affine.for a loop (iter_args become variables
// assigned at the yield), affine.if a condition on its integer set, affine.load/store and their vector forms an
// indexed access with the map written out, gpu.barrier a workgroup barrier, gpu.shuffle a wavefront shuffle.  It
// serves schedules that no family covers (a function scripted with the Rewriter and no operator tag) and makes every
// Rewriter primitive checkable on the device: the kernel computes what the host interpreter computes from the same
// body, operation for operation (floating-point contraction is switched off so that a mulf followed by an addf stays
// two roundings, as written).
#include "backend/ScheduleEmitter.h"

#include <cctype>
#include <cmath>
#include <cstdio>
#include <limits>
#include <set>
#include <sstream>
#include <unordered_map>

namespace KernelCodeGen {
namespace hipgen {

using namespace mlir;

namespace {

// Closed interval an index value is known to lie in.
struct Range {
  bool known = false;
  int64_t lo = 0, hi = 0;
  static Range of(int64_t a, int64_t b) { Range r; r.known = true; r.lo = a; r.hi = b; return r; }
  bool isConstant() const { return known && lo == hi; }
};

int64_t floorDiv(int64_t a, int64_t b) { int64_t q = a / b; return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; }
int64_t ceilDiv(int64_t a, int64_t b) { return -floorDiv(-a, b); }

struct Failure { std::string what; };
[[noreturn]] void fail(const std::string& what) { throw Failure{what}; }

class Emitter {
public:
  Emitter(func::FuncOp f, const std::string& kernelName) : f(f), kernelName(kernelName) {}

  void run(std::string& text, KernelLaunchInfo& info) {
    collectSignature();
    findLevels();
    std::ostringstream head;
    body << "#pragma clang fp contract(" << (f->hasAttr("kcg.fp_contract") && f->getAttr("kcg.fp_contract").i ? "fast" : "off") << ")\n";
    indent = 1;
    // what the function does before the grid level: constants and the like (the result buffers are parameters)
    for (auto& op : f.front().getOperations()) {
      if (&op == grid.getOperation()) { emitGrid(); continue; }
      if (op.getKind() == OpKind::Return) continue;
      if (op.getKind() == OpKind::Alloc) continue;   // handled by collectSignature
      if (op.getKind() == OpKind::AffineParallel) fail("more than one grid-level affine.parallel");
      emitOp(&op);
    }
    head << typedefs.str();
    head << "extern \"C\" __global__ void __launch_bounds__(" << threads << ") " << kernelName << "(";
    for (size_t i = 0; i < params.size(); ++i) head << (i ? ", " : "") << params[i];
    head << ") {\n" << body.str() << "}\n";
    text = head.str();
    info = KernelLaunchInfo();
    info.name = kernelName;
    for (int d = 0; d < 3; ++d) { info.grid[d] = gridDim[d]; info.block[d] = blockDim[d]; }
    info.numArgs = (uint32_t)params.size();
    info.ldsBytes = 0;
  }

private:
  func::FuncOp f;
  std::string kernelName;
  AffineParallelOp grid;
  std::ostringstream body, typedefs;
  std::vector<std::string> params;
  std::unordered_map<detail::ValueImpl*, std::string> names;
  std::unordered_map<detail::ValueImpl*, Range> ranges;
  std::set<std::string> knownTypedefs;
  std::set<detail::ValueImpl*> unrollIvs;      // induction variables that index a per-lane array
  int indent = 1, nextId = 0;
  int64_t threads = 0, ldsBytes = 0;
  uint32_t gridDim[3] = {1, 1, 1}, blockDim[3] = {1, 1, 1};
  bool inWorkgroup = false;

  // ---- names and types ----------------------------------------------------------------------------------------
  std::string pad() const { return std::string((size_t)indent * 2, ' '); }
  std::string fresh(const char* stem) { return stem + std::to_string(nextId++); }

  // Index values are 32-bit like the reference's (src/Backend/CUDA.cc prints `int`), unless some buffer of the function
  // has more elements than that can count: flattened positions appear as intermediate values of the index expressions.
  bool wideIndex = false;
  std::string indexType() const { return wideIndex ? "long" : "int"; }
  std::string scalarType(Type t) const {
    if (t.isIndex()) return indexType();
    return plainType(t);
  }
  static std::string plainType(Type t) {
    if (t.isF32()) return "float";
    if (t.isF16()) return "_Float16";
    if (t.isBF16()) return "__bf16";
    if (t.isF64()) return "double";
    if (t.isIndex()) return "int";
    if (t.isa<IntegerType>()) {
      switch (t.cast<IntegerType>().getWidth()) {
        case 1: return "bool";
        case 8: return "signed char";
        case 16: return "short";
        case 32: return "int";
        case 64: return "long";
      }
    }
    fail("element type without a device type");
  }
  // What an element of a buffer is on the device: index values are 64-bit there, an i1 one byte.
  static std::string storageType(Type t) {
    if (t.isIndex()) return "long";
    if (t.isa<IntegerType>() && t.cast<IntegerType>().getWidth() == 1) return "unsigned char";
    return plainType(t);
  }
  static std::string typeTag(Type t) {
    std::string s = storageType(t);
    for (auto& c : s) if (c == ' ') c = '_';
    return s;
  }
  static int widthOf(Type t) { return t.isa<VectorType>() ? (int)t.cast<VectorType>().getNumElements() : 1; }
  static Type elementOf(Type t) { return t.isa<VectorType>() ? t.cast<VectorType>().getElementType() : t; }
  std::string vectorType(Type element, int width) {
    const std::string name = "kcg_v" + std::to_string(width) + "_" + typeTag(element);
    if (knownTypedefs.insert(name).second)
      typedefs << "typedef " << storageType(element) << " " << name << " __attribute__((ext_vector_type(" << width << ")));\n";
    return name;
  }
  // C type of an SSA value; a vector of one element is a scalar
  std::string valueType(Type t) {
    const int w = widthOf(t);
    return w == 1 ? scalarType(elementOf(t)) : vectorType(elementOf(t), w);
  }

  const std::string& nameOf(Value v) {
    auto it = names.find(v.getImpl());
    if (it == names.end()) fail("use of a value the kernel has not defined (defined outside the function?)");
    return it->second;
  }
  Range rangeOf(Value v) const {
    auto it = ranges.find(v.getImpl());
    return it == ranges.end() ? Range() : it->second;
  }
  // an index operand as text: its literal when it is a known constant
  std::string indexText(Value v) {
    Range r = rangeOf(v);
    if (r.isConstant()) return std::to_string(r.lo);
    return nameOf(v);
  }

  // ---- affine expressions ---------------------------------------------------------------------------------------
  Range evalRange(AffineExpr e, const std::vector<Range>& in, unsigned numDims) const {
    switch (e.getKind()) {
      case AffineExprKind::Constant: { int64_t v = e.evaluate({}, {}); return Range::of(v, v); }
      case AffineExprKind::DimId: return in[e.cast<AffineDimExpr>().getPosition()];
      case AffineExprKind::SymbolId: return in[numDims + e.cast<AffineSymbolExpr>().getPosition()];
      default: break;
    }
    auto bin = e.cast<AffineBinaryOpExpr>();
    Range a = evalRange(bin.getLHS(), in, numDims), b = evalRange(bin.getRHS(), in, numDims);
    if (e.getKind() == AffineExprKind::Mod && b.isConstant() && b.lo > 0) {
      if (a.known && a.lo >= 0 && a.hi < b.lo) return a;
      return Range::of(0, b.lo - 1);
    }
    if (!a.known || !b.known) return Range();
    switch (e.getKind()) {
      case AffineExprKind::Add: return Range::of(a.lo + b.lo, a.hi + b.hi);
      case AffineExprKind::Mul: {
        const int64_t c[4] = {a.lo * b.lo, a.lo * b.hi, a.hi * b.lo, a.hi * b.hi};
        return Range::of(std::min(std::min(c[0], c[1]), std::min(c[2], c[3])), std::max(std::max(c[0], c[1]), std::max(c[2], c[3])));
      }
      case AffineExprKind::FloorDiv:
        if (b.isConstant() && b.lo > 0) return Range::of(floorDiv(a.lo, b.lo), floorDiv(a.hi, b.lo));
        return Range();
      case AffineExprKind::CeilDiv:
        if (b.isConstant() && b.lo > 0) return Range::of(ceilDiv(a.lo, b.lo), ceilDiv(a.hi, b.lo));
        return Range();
      default: return Range();
    }
  }

  // prec: 0 = anything may stand here, 1 = operand of +, 3 = operand of * / % (any binary expression gets brackets)
  std::string exprText(AffineExpr e, const std::vector<std::string>& in, const std::vector<Range>& rin, unsigned numDims, int prec) {
    Range whole = evalRange(e, rin, numDims);
    if (whole.isConstant()) return whole.lo < 0 && prec > 0 ? "(" + std::to_string(whole.lo) + ")" : std::to_string(whole.lo);
    switch (e.getKind()) {
      case AffineExprKind::Constant: return std::to_string(e.evaluate({}, {}));
      case AffineExprKind::DimId: return in[e.cast<AffineDimExpr>().getPosition()];
      case AffineExprKind::SymbolId: return in[numDims + e.cast<AffineSymbolExpr>().getPosition()];
      default: break;
    }
    auto bin = e.cast<AffineBinaryOpExpr>();
    Range a = evalRange(bin.getLHS(), rin, numDims), b = evalRange(bin.getRHS(), rin, numDims);
    std::string s;
    int mine = 2;
    switch (e.getKind()) {
      case AffineExprKind::Add:
        mine = 1;
        if (a.isConstant() && a.lo == 0) return exprText(bin.getRHS(), in, rin, numDims, prec);
        if (b.isConstant() && b.lo == 0) return exprText(bin.getLHS(), in, rin, numDims, prec);
        if (b.isConstant() && b.lo < 0) s = exprText(bin.getLHS(), in, rin, numDims, 1) + " - " + std::to_string(-b.lo);
        else s = exprText(bin.getLHS(), in, rin, numDims, 1) + " + " + exprText(bin.getRHS(), in, rin, numDims, 1);
        break;
      case AffineExprKind::Mul:
        if (a.isConstant() && a.lo == 1) return exprText(bin.getRHS(), in, rin, numDims, prec);
        if (b.isConstant() && b.lo == 1) return exprText(bin.getLHS(), in, rin, numDims, prec);
        if (b.isConstant() && b.lo == -1) { s = "-" + exprText(bin.getLHS(), in, rin, numDims, 3); break; }
        if (a.isConstant() && a.lo == -1) { s = "-" + exprText(bin.getRHS(), in, rin, numDims, 3); break; }
        s = exprText(bin.getLHS(), in, rin, numDims, 3) + " * " + exprText(bin.getRHS(), in, rin, numDims, 3);
        break;
      case AffineExprKind::FloorDiv: case AffineExprKind::CeilDiv: case AffineExprKind::Mod: {
        const bool positive = a.known && a.lo >= 0 && b.known && b.lo > 0;
        const std::string l = exprText(bin.getLHS(), in, rin, numDims, positive ? 3 : 0);
        const std::string r = exprText(bin.getRHS(), in, rin, numDims, positive ? 3 : 0);
        if (e.getKind() == AffineExprKind::FloorDiv) {
          if (!positive) return "kcg_floordiv<" + indexType() + ">(" + l + ", " + r + ")";
          s = l + " / " + r;
        } else if (e.getKind() == AffineExprKind::Mod) {
          if (!positive) return "kcg_floormod<" + indexType() + ">(" + l + ", " + r + ")";
          s = l + " % " + r;
        } else {
          return "kcg_ceildiv<" + indexType() + ">(" + l + ", " + r + ")";
        }
        break;
      }
      default: fail("affine expression kind without a lowering");
    }
    return prec > mine ? "(" + s + ")" : s;
  }

  struct Bound { std::vector<std::string> in; std::vector<Range> rin; };
  Bound bind(const std::vector<Value>& operands) {
    Bound b;
    for (Value v : operands) { b.in.push_back(indexText(v)); b.rin.push_back(rangeOf(v)); }
    return b;
  }
  std::string mapResultText(AffineMap map, unsigned i, const Bound& b, int prec = 0) {
    if (map.getNumInputs() != b.in.size()) fail("affine map has " + std::to_string(map.getNumInputs()) + " inputs but " + std::to_string(b.in.size()) + " operands");
    return exprText(map.getResult(i), b.in, b.rin, map.getNumDims(), prec);
  }
  Range mapResultRange(AffineMap map, unsigned i, const Bound& b) const { return evalRange(map.getResult(i), b.rin, map.getNumDims()); }

  // ---- function signature and launch geometry ---------------------------------------------------------------------
  void collectSignature() {
    if (f.empty()) fail("function has no body");
    f.walk([&](Operation* op) {
      for (unsigned i = 0; i < op->getNumResults(); ++i)
        if (auto mt = op->getResult(i).getType().dyn_cast<MemRefType>())
          wideIndex = wideIndex || mt.getNumElements() > (int64_t)std::numeric_limits<int32_t>::max();
    });
    for (auto a : f.getArguments())
      if (auto mt = a.getType().dyn_cast<MemRefType>())
        wideIndex = wideIndex || mt.getNumElements() > (int64_t)std::numeric_limits<int32_t>::max();
    unsigned n = 0;
    for (auto a : f.getArguments()) {
      auto mt = a.getType().dyn_cast<MemRefType>();
      if (!mt) fail("function arguments other than memrefs have no lowering");
      const std::string name = "arg" + std::to_string(n++);
      names[a.getImpl()] = name;
      params.push_back(storageType(mt.getElementType()) + "* __restrict__ " + name);
    }
    // results the function allocates itself follow the inputs, in the order they are returned
    Operation& ret = f.front().back();
    if (ret.getKind() != OpKind::Return) fail("function body does not end in a return");
    unsigned r = 0;
    for (Value v : ret.getOperands()) {
      if (v.isa<BlockArgument>()) continue;       // written in place
      Operation* def = v.getDefiningOp();
      if (!def || def->getKind() != OpKind::Alloc || def->getBlock() != &f.front()) fail("a returned value is neither an argument nor a buffer the function allocates");
      if (names.count(v.getImpl())) continue;
      auto mt = v.getType().cast<MemRefType>();
      const std::string name = "out" + std::to_string(r++);
      names[v.getImpl()] = name;
      params.push_back(storageType(mt.getElementType()) + "* __restrict__ " + name);
    }
    for (auto& op : f.front().getOperations())
      if (op.getKind() == OpKind::Alloc && !names.count(op.getResult(0).getImpl()))
        fail("a buffer allocated at function level is not returned: temporaries in global memory have no lowering");
  }

  void findLevels() {
    for (auto& op : f.front().getOperations())
      if (auto p = dyn_cast<AffineParallelOp>(op)) { grid = p; break; }
    if (!grid) fail("function has no grid-level affine.parallel");
    if (grid.getNumDims() > 3) fail("grid of more than three dimensions");
    // every workgroup-level affine.parallel directly inside the grid level must have the same extents: the thread
    // ids are the same ones
    std::vector<int64_t> first;
    for (auto& op : grid.getBody()->getOperations())
      if (auto p = dyn_cast<AffineParallelOp>(op)) {
        if (p.getNumDims() > 3) fail("workgroup of more than three dimensions");
        auto e = extents(p);
        if (first.empty()) {
          first = e;
          threads = 1;
          for (auto x : e) threads *= x;
          for (size_t d = 0; d < e.size(); ++d) blockDim[e.size() - 1 - d] = (uint32_t)e[d];
        } else if (e != first) {
          fail("workgroup levels of different extents in one kernel");
        }
      }
    if (threads == 0) fail("function has no workgroup-level affine.parallel inside the grid level");
    if (threads > 1024) fail("workgroup of " + std::to_string(threads) + " threads (the limit is 1024)");
    auto ge = extents(grid);
    for (size_t d = 0; d < ge.size(); ++d) gridDim[ge.size() - 1 - d] = (uint32_t)ge[d];
    // induction variables that (through affine.apply) index a per-lane array: their loops must unroll completely
    f.walk([&](Operation* op) {
      int memIdx = -1;
      switch (op->getKind()) {
        case OpKind::AffineLoad: case OpKind::AffineVectorLoad: case OpKind::MemLoad: memIdx = 0; break;
        case OpKind::AffineStore: case OpKind::AffineVectorStore: case OpKind::MemStore: memIdx = 1; break;
        default: return;
      }
      auto mt = op->getOperand((unsigned)memIdx).getType().dyn_cast<MemRefType>();
      if (!mt || mt.getMemorySpaceAsInt() != 3) return;
      for (unsigned i = (unsigned)memIdx + 1; i < op->getNumOperands(); ++i) markUnroll(op->getOperand(i), 0);
    });
  }
  void markUnroll(Value v, int depth) {
    if (depth > 8) return;
    if (v.isa<BlockArgument>()) { unrollIvs.insert(v.getImpl()); return; }
    Operation* def = v.getDefiningOp();
    if (def && (def->getKind() == OpKind::AffineApply || def->getKind() == OpKind::AddI || def->getKind() == OpKind::MulI || def->getKind() == OpKind::SubI))
      for (Value o : def->getOperands()) markUnroll(o, depth + 1);
  }
  static std::vector<int64_t> extents(AffineParallelOp p) {
    auto lbs = p.getConstantLowerBounds(), ubs = p.getConstantUpperBounds();
    auto steps = p.getSteps();
    std::vector<int64_t> e(ubs.size());
    for (size_t d = 0; d < ubs.size(); ++d) e[d] = (ubs[d] - lbs[d] + steps[d] - 1) / steps[d];
    return e;
  }

  void bindParallelIvs(AffineParallelOp p, const char* builtin) {
    static const char* axis[] = {"x", "y", "z"};
    auto lbs = p.getConstantLowerBounds(), ubs = p.getConstantUpperBounds();
    auto steps = p.getSteps();
    auto ivs = p.getIVs();
    const size_t nd = ivs.size();
    for (size_t d = 0; d < nd; ++d) {
      const std::string name = fresh("i");
      names[ivs[d].getImpl()] = name;
      const int64_t extent = (ubs[d] - lbs[d] + steps[d] - 1) / steps[d];
      ranges[ivs[d].getImpl()] = Range::of(lbs[d], lbs[d] + (extent - 1) * steps[d]);
      body << pad() << "const " << indexType() << " " << name << " = ";
      if (lbs[d] != 0) body << lbs[d] << " + ";
      body << "(" << indexType() << ")" << builtin << "." << axis[nd - 1 - d];
      if (steps[d] != 1) body << " * " << steps[d];
      body << ";\n";
    }
  }

  void emitGrid() {
    bindParallelIvs(grid, "blockIdx");
    bool first = true;
    for (auto& op : grid.getBody()->getOperations()) {
      if (auto p = dyn_cast<AffineParallelOp>(op)) {
        if (!first) body << pad() << "__syncthreads();\n";   // the levels run one after the other
        first = false;
        body << pad() << "{\n";
        ++indent;
        bindParallelIvs(p, "threadIdx");
        inWorkgroup = true;
        emitBlock(p.getBody());
        inWorkgroup = false;
        --indent;
        body << pad() << "}\n";
        continue;
      }
      emitOp(&op);
    }
  }

  void emitBlock(Block* b) {
    for (auto& op : b->getOperations()) emitOp(&op);
  }

  // ---- memory ---------------------------------------------------------------------------------------------------
  std::string linearText(MemRefType mt, const std::vector<std::string>& idx, const std::vector<Range>& ridx) {
    auto shape = mt.getShape();
    const bool wide = mt.getNumElements() > (int64_t)std::numeric_limits<int32_t>::max();
    std::string s;
    int64_t stride = 1;
    std::vector<int64_t> strides(shape.size());
    for (size_t d = shape.size(); d-- > 0;) { strides[d] = stride; stride *= shape[d]; }
    for (size_t d = 0; d < shape.size(); ++d) {
      if (ridx[d].isConstant() && ridx[d].lo == 0) continue;
      std::string term = idx[d];
      if (ridx[d].isConstant()) term = std::to_string(ridx[d].lo * strides[d]);
      else if (strides[d] != 1) term = (wide ? "(long)(" + term + ")" : atom(term)) + " * " + std::to_string(strides[d]);
      else if (wide) term = "(long)(" + term + ")";
      s += (s.empty() ? "" : " + ") + term;
    }
    return s.empty() ? "0" : s;
  }

  // `text` ready to be an operand of *: bracketed unless it is a single name or number
  static std::string atom(const std::string& text) {
    for (char c : text)
      if (!(std::isalnum((unsigned char)c) || c == '_')) return "(" + text + ")";
    return text;
  }

  void emitAccess(Operation* op) {
    const OpKind k = op->getKind();
    const bool isStore = k == OpKind::AffineStore || k == OpKind::AffineVectorStore || k == OpKind::MemStore;
    const bool viaMap = k != OpKind::MemLoad && k != OpKind::MemStore;
    const unsigned memIdx = isStore ? 1 : 0;
    Value mem = op->getOperand(memIdx);
    auto mt = mem.getType().dyn_cast<MemRefType>();
    if (!mt) fail("access to a value that is not a memref");
    std::vector<Value> operands(op->getOperands().begin() + memIdx + 1, op->getOperands().end());
    Bound b = bind(operands);
    std::vector<std::string> idx;
    std::vector<Range> ridx;
    if (viaMap) {
      AffineMap map = op->getAttr("map").map;
      if ((int64_t)map.getNumResults() != mt.getRank()) fail("access map has " + std::to_string(map.getNumResults()) + " results for a memref of rank " + std::to_string(mt.getRank()));
      for (unsigned i = 0; i < map.getNumResults(); ++i) { idx.push_back(mapResultText(map, i, b)); ridx.push_back(mapResultRange(map, i, b)); }
    } else {
      if ((int64_t)operands.size() != mt.getRank()) fail("memref.load/store needs one subscript per dimension");
      idx = b.in; ridx = b.rin;
    }
    const std::string lin = linearText(mt, idx, ridx);
    const std::string& base = nameOf(mem);
    Type valueTy = isStore ? op->getOperand(0).getType() : op->getResult(0).getType();
    const int width = widthOf(valueTy);
    Type element = mt.getElementType();
    if (elementOf(valueTy) != element) fail("access value type differs from the memref's element type");
    const bool perLane = mt.getMemorySpaceAsInt() == 3;
    const bool converts = storageType(element) != scalarType(element);    // index and i1 are stored wider
    if (!isStore) {
      const std::string name = fresh("v");
      names[op->getResult(0).getImpl()] = name;
      body << pad() << "const " << valueType(valueTy) << " " << name << " = ";
      if (width == 1) {
        body << (converts ? "(" + scalarType(element) + ")" : "") << base << "[" << lin << "];\n";
      } else if (perLane || converts) {
        body << "{";
        for (int j = 0; j < width; ++j) body << (j ? ", " : "") << base << "[" << lin << " + " << j << "]";
        body << "};\n";
      } else {
        body << "*(const " << vectorType(element, width) << "*)(" << base << " + " << lin << ");\n";
      }
      return;
    }
    if (!inWorkgroup && !perLane) fail("a store outside the workgroup level would be executed by every thread");
    const std::string& value = nameOf(op->getOperand(0));
    if (width == 1) {
      body << pad() << base << "[" << lin << "] = " << (converts ? "(" + storageType(element) + ")" : "") << value << ";\n";
    } else if (perLane || converts) {
      for (int j = 0; j < width; ++j) body << pad() << base << "[" << lin << " + " << j << "] = " << value << "[" << j << "];\n";
    } else {
      body << pad() << "*(" << vectorType(element, width) << "*)(" << base << " + " << lin << ") = " << value << ";\n";
    }
  }

  void emitAlloc(Operation* op) {
    auto mt = op->getResult(0).getType().cast<MemRefType>();
    const unsigned space = mt.getMemorySpaceAsInt();
    const int64_t n = mt.getNumElements();
    const int64_t bytes = n * ((mt.getElementType().getIntOrFloatBitWidth() + 7) / 8);
    if (space == 2) {
      const std::string name = fresh("lds");
      names[op->getResult(0).getImpl()] = name;
      ldsBytes += (bytes + 15) / 16 * 16;
      if (ldsBytes > 160 * 1024) fail("the schedule's shared buffers need more than the 160 KiB of LDS a workgroup can have");
      body << pad() << "__shared__ __attribute__((aligned(16))) " << storageType(mt.getElementType()) << " " << name << "[" << n << "];\n";
    } else if (space == 3) {
      const std::string name = fresh("reg");
      names[op->getResult(0).getImpl()] = name;
      if (bytes > 2048) fail("a per-lane buffer of " + std::to_string(bytes) + " bytes does not fit the register file");
      body << pad() << storageType(mt.getElementType()) << " " << name << "[" << n << "];\n";
    } else {
      fail("memref.alloc in memory space " + std::to_string(space) + " inside the kernel");
    }
  }

  // ---- control flow -----------------------------------------------------------------------------------------------
  std::string boundText(AffineMap map, const std::vector<Value>& operands, bool lower, Range& r) {
    Bound b = bind(operands);
    std::string s;
    r = Range();
    for (unsigned i = 0; i < map.getNumResults(); ++i) {
      const std::string t = mapResultText(map, i, b);
      Range ri = mapResultRange(map, i, b);
      if (i == 0) { s = t; r = ri; continue; }
      s = std::string(lower ? "max" : "min") + "(" + s + ", " + t + ")";
      if (r.known && ri.known) r = lower ? Range::of(std::max(r.lo, ri.lo), std::max(r.hi, ri.hi)) : Range::of(std::min(r.lo, ri.lo), std::min(r.hi, ri.hi));
      else if (!lower && (r.known || ri.known)) { Range k = r.known ? r : ri; r = Range::of(std::numeric_limits<int32_t>::min(), k.hi); }
      else r = Range();
    }
    return s;
  }

  void emitFor(Operation* op) {
    AffineForOp loop(op);
    Range rl, ru;
    const std::string lb = boundText(loop.getLowerBoundMap(), loop.getLowerBoundOperands(), true, rl);
    const std::string ub = boundText(loop.getUpperBoundMap(), loop.getUpperBoundOperands(), false, ru);
    const int64_t step = loop.getStep();
    if (step <= 0) fail("loop step is not positive");
    // carried values are variables that the yield assigns; the loop's results are those variables after the loop
    auto regionArgs = loop.getRegionIterArgs();
    auto inits = loop.getIterOperands();
    std::vector<std::string> carried;
    for (size_t i = 0; i < regionArgs.size(); ++i) {
      const std::string name = fresh("c");
      carried.push_back(name);
      body << pad() << valueType(regionArgs[i].getType()) << " " << name << " = " << nameOf(inits[i]) << ";\n";
      names[regionArgs[i].getImpl()] = name;
      names[op->getResult((unsigned)i).getImpl()] = name;
    }
    const std::string iv = fresh("i");
    names[loop.getInductionVar().getImpl()] = iv;
    int64_t trips = -1;
    if (rl.isConstant() && ru.isConstant()) trips = ru.lo > rl.lo ? (ru.lo - rl.lo + step - 1) / step : 0;
    if (trips > 0) ranges[loop.getInductionVar().getImpl()] = Range::of(rl.lo, rl.lo + (trips - 1) * step);
    else if (rl.known && ru.known && ru.hi > rl.lo) ranges[loop.getInductionVar().getImpl()] = Range::of(rl.lo, ru.hi - 1);
    const bool tagged = op->hasAttr("affine.loop") && op->getAttr("affine.loop").s == "unroll";
    const bool mustUnroll = unrollIvs.count(loop.getInductionVar().getImpl()) != 0;
    if (mustUnroll && trips < 0) fail("a loop whose index selects a register has no constant trip count");
    // the reference tags every loop of a schedule "unroll", the loop over k included; here a loop unrolls where
    // registers are selected by its index and where it is short, and is left to the compiler otherwise
    if (mustUnroll || (tagged && trips >= 0 && trips <= 16)) body << pad() << "#pragma unroll\n";
    body << pad() << "for (" << indexType() << " " << iv << " = " << lb << "; " << iv << " < " << ub << "; " << iv << " += " << step << ") {\n";
    ++indent;
    emitBlock(loop.getBody());
    Operation* yield = loop.getBody()->getTerminator();
    if (!carried.empty()) {
      if (!yield || yield->getKind() != OpKind::AffineYield || yield->getNumOperands() != carried.size()) fail("loop with iter_args does not yield one value per argument");
      if (carried.size() == 1) {
        body << pad() << carried[0] << " = " << nameOf(yield->getOperand(0)) << ";\n";
      } else {
        std::vector<std::string> tmp;
        for (size_t i = 0; i < carried.size(); ++i) {
          tmp.push_back(fresh("t"));
          body << pad() << "const " << valueType(regionArgs[i].getType()) << " " << tmp.back() << " = " << nameOf(yield->getOperand((unsigned)i)) << ";\n";
        }
        for (size_t i = 0; i < carried.size(); ++i) body << pad() << carried[i] << " = " << tmp[i] << ";\n";
      }
    }
    --indent;
    body << pad() << "}\n";
  }

  void emitIf(Operation* op) {
    AffineIfOp ifOp(op);
    if (op->getNumResults()) fail("affine.if with results");
    IntegerSet set = ifOp.getIntegerSet();
    Bound b = bind(ifOp.getOperands());
    if (set.getNumInputs() != b.in.size()) fail("integer set inputs differ from the affine.if operands");
    std::string cond;
    for (unsigned i = 0; i < set.getNumConstraints(); ++i) {
      const std::string e = exprText(set.getConstraint(i), b.in, b.rin, set.getNumDims(), 1);
      cond += (i ? " && " : "") + e + (set.isEq(i) ? " == 0" : " >= 0");
    }
    if (cond.empty()) cond = "true";
    body << pad() << "if (" << cond << ") {\n";
    ++indent;
    emitBlock(ifOp.getThenBlock());
    --indent;
    if (ifOp.hasElse()) {
      body << pad() << "} else {\n";
      ++indent;
      emitBlock(ifOp.getElseBlock());
      --indent;
    }
    body << pad() << "}\n";
  }

  // ---- values -------------------------------------------------------------------------------------------------------
  static std::string floatLiteral(double v, Type t) {
    if (v != v) return "__builtin_nanf(\"\")";
    if (std::isinf(v)) return v > 0 ? "__builtin_inff()" : "(-__builtin_inff())";
    char buf[64];
    if (t.isF64()) { std::snprintf(buf, sizeof buf, "%.17g", v); std::string s(buf); if (s.find_first_of(".eE") == std::string::npos) s += ".0"; return s; }
    std::snprintf(buf, sizeof buf, "%.9g", (double)(float)v);
    std::string s(buf);
    if (s.find_first_of(".eE") == std::string::npos) s += ".0";
    return s + "f";
  }

  std::string define(Operation* op, unsigned result = 0) {
    const std::string name = fresh("v");
    names[op->getResult(result).getImpl()] = name;
    body << pad() << "const " << valueType(op->getResult(result).getType()) << " " << name << " = ";
    return name;
  }

  // one expression per element: `fn` gets the element's operand texts
  void emitElementwise(Operation* op, const std::function<std::string(const std::vector<std::string>&)>& fn) {
    Type rt = op->getResult(0).getType();
    const int width = widthOf(rt);
    std::vector<std::string> in;
    if (width == 1) {
      for (Value o : op->getOperands()) in.push_back(nameOf(o));
      define(op);
      body << fn(in) << ";\n";
      return;
    }
    define(op);
    body << "{";
    for (int j = 0; j < width; ++j) {
      in.clear();
      for (Value o : op->getOperands()) in.push_back(widthOf(o.getType()) == 1 ? nameOf(o) : nameOf(o) + "[" + std::to_string(j) + "]");
      body << (j ? ", " : "") << fn(in);
    }
    body << "};\n";
  }

  void emitOp(Operation* op) {
    switch (op->getKind()) {
      case OpKind::Alloc: emitAlloc(op); return;
      case OpKind::AffineFor: emitFor(op); return;
      case OpKind::AffineIf: emitIf(op); return;
      case OpKind::AffineParallel: fail("affine.parallel nested deeper than grid and workgroup");
      case OpKind::AffineLoad: case OpKind::AffineStore: case OpKind::AffineVectorLoad: case OpKind::AffineVectorStore:
      case OpKind::MemLoad: case OpKind::MemStore:
        emitAccess(op); return;
      case OpKind::AffineYield: case OpKind::Return: return;
      case OpKind::Barrier:
        if (!inWorkgroup) fail("gpu.barrier outside the workgroup level");
        body << pad() << "__syncthreads();\n";
        return;
      case OpKind::Call: fail("a call inside a scheduled function has no lowering");
      case OpKind::Constant: {
        Attribute a = op->getAttr("value");
        Type t = op->getResult(0).getType();
        if (widthOf(t) != 1) fail("vector constants have no lowering");
        if (t.isIntOrIndex()) ranges[op->getResult(0).getImpl()] = Range::of(a.i, a.i);
        define(op);
        if (t.isFloat()) body << (t.isF32() || t.isF64() ? "" : "(" + scalarType(t) + ")") << floatLiteral(a.kind == Attribute::Float ? a.f : (double)a.i, t) << ";\n";
        else body << a.i << ";\n";
        return;
      }
      case OpKind::AffineApply: {
        AffineMap map = op->getAttr("map").map;
        Bound b = bind(op->getOperands());
        if (map.getNumResults() != 1) fail("affine.apply with more than one result");
        const std::string text = mapResultText(map, 0, b);
        Range r = mapResultRange(map, 0, b);
        if (r.known) ranges[op->getResult(0).getImpl()] = r;
        define(op);
        body << text << ";\n";
        return;
      }
      case OpKind::Shuffle: emitShuffle(op); return;
      default: break;
    }
    Type rt = op->getResult(0).getType();
    Type et = elementOf(rt);
    const std::string ct = scalarType(et);
    const bool f32 = et.isF32();
    // operations in a narrower float type round after every operation, as the type says
    auto binary = [&](const char* sym) {
      emitElementwise(op, [&](const std::vector<std::string>& a) { return "(" + ct + ")(" + a[0] + " " + sym + " " + a[1] + ")"; });
    };
    auto call1 = [&](const std::string& fn32, const std::string& fn64) {
      emitElementwise(op, [&](const std::vector<std::string>& a) {
        if (f32) return fn32 + "(" + a[0] + ")";
        if (et.isF64()) return fn64 + "(" + a[0] + ")";
        return "(" + ct + ")" + fn32 + "((float)" + a[0] + ")";
      });
    };
    switch (op->getKind()) {
      case OpKind::AddF: case OpKind::AddI: binary("+"); return;
      case OpKind::SubF: case OpKind::SubI: binary("-"); return;
      case OpKind::MulF: case OpKind::MulI: binary("*"); return;
      case OpKind::DivF: binary("/"); return;
      case OpKind::MaxF: case OpKind::MinF: {
        const bool mx = op->getKind() == OpKind::MaxF;
        emitElementwise(op, [&](const std::vector<std::string>& a) {   // a NaN operand gives NaN (arith.maxf / minf)
          return "((" + a[0] + " != " + a[0] + " || " + a[1] + " != " + a[1] + ") ? (" + ct + ")__builtin_nanf(\"\") : (" + a[0] + (mx ? " > " : " < ") + a[1] + " ? " + a[0] + " : " + a[1] + "))";
        });
        return;
      }
      case OpKind::PowF:
        emitElementwise(op, [&](const std::vector<std::string>& a) {
          if (f32) return "powf(" + a[0] + ", " + a[1] + ")";
          if (et.isF64()) return "pow(" + a[0] + ", " + a[1] + ")";
          return "(" + ct + ")powf((float)" + a[0] + ", (float)" + a[1] + ")";
        });
        return;
      case OpKind::NegF: emitElementwise(op, [&](const std::vector<std::string>& a) { return "-" + a[0]; }); return;
      case OpKind::Abs: call1("fabsf", "fabs"); return;
      case OpKind::Exp: call1("expf", "exp"); return;
      case OpKind::Exp2: call1("exp2f", "exp2"); return;
      case OpKind::Tanh: call1("tanhf", "tanh"); return;
      case OpKind::Sqrt: call1("sqrtf", "sqrt"); return;
      case OpKind::Log: call1("logf", "log"); return;
      case OpKind::Rsqrt:
        emitElementwise(op, [&](const std::vector<std::string>& a) {
          if (f32) return "(1.0f / sqrtf(" + a[0] + "))";
          if (et.isF64()) return "(1.0 / sqrt(" + a[0] + "))";
          return "(" + ct + ")(1.0f / sqrtf((float)" + a[0] + "))";
        });
        return;
      case OpKind::CmpF: {
        const char* sym = nullptr;
        bool ordered = false;
        switch ((arith::CmpFPredicate)op->getAttr("predicate").i) {
          case arith::CmpFPredicate::OEQ: sym = "=="; break;
          case arith::CmpFPredicate::OGT: sym = ">"; break;
          case arith::CmpFPredicate::OGE: sym = ">="; break;
          case arith::CmpFPredicate::OLT: sym = "<"; break;
          case arith::CmpFPredicate::OLE: sym = "<="; break;
          case arith::CmpFPredicate::ONE: sym = "!="; ordered = true; break;
          default: fail("cmpf predicate without a lowering");
        }
        emitElementwise(op, [&](const std::vector<std::string>& a) {
          std::string s = "(" + a[0] + " " + sym + " " + a[1] + ")";
          if (ordered) s = "(" + s + " && " + a[0] + " == " + a[0] + " && " + a[1] + " == " + a[1] + ")";
          return s;
        });
        return;
      }
      case OpKind::Select:
        emitElementwise(op, [&](const std::vector<std::string>& a) { return "(" + a[0] + " ? " + a[1] + " : " + a[2] + ")"; });
        return;
      // value conversions; the Frontend's "Cast" is an arith.bitcast that the reference prints as static_cast
      // (src/Backend/CUDA.cc:537-548) and the host interpreter executes as one
      case OpKind::ExtF: case OpKind::TruncF: case OpKind::SIToFP: case OpKind::FPToSI: case OpKind::Bitcast:
        emitElementwise(op, [&](const std::vector<std::string>& a) { return "(" + ct + ")" + a[0]; });
        return;
      default: fail(std::string("operation ") + op->getName() + " has no lowering");
    }
  }

  // Lanes exchange inside groups of `width` consecutive threads; the second result tells whether the source lane
  // was inside the group (outside it a lane keeps its own value).
  void emitShuffle(Operation* op) {
    if (!inWorkgroup) fail("gpu.shuffle outside the workgroup level");
    gpu::ShuffleOp sh(op);
    Range w = rangeOf(sh.getWidth());
    if (!w.isConstant() || w.lo <= 0 || w.lo > 64 || (w.lo & (w.lo - 1))) fail("shuffle width must be a constant power of two of at most 64 (one wavefront)");
    if (threads % 64 && threads > 64) fail("shuffles need whole wavefronts");
    if (widthOf(op->getResult(0).getType()) != 1) fail("shuffle of a vector value");
    const std::string off = indexText(sh.getOffset()), width = std::to_string(w.lo), value = nameOf(sh.getValue());
    const std::string lane = fresh("l");
    body << pad() << "const int " << lane << " = (int)((threadIdx.z * blockDim.y + threadIdx.y) * blockDim.x + threadIdx.x) & " << (w.lo - 1) << ";\n";
    std::string fn, src;
    switch (sh.getMode()) {
      case gpu::ShuffleMode::DOWN: fn = "__shfl_down"; src = lane + " + " + off; break;
      case gpu::ShuffleMode::UP: fn = "__shfl_up"; src = lane + " - " + off; break;
      case gpu::ShuffleMode::XOR: fn = "__shfl_xor"; src = "(" + lane + " ^ " + off + ")"; break;
      case gpu::ShuffleMode::IDX: fn = "__shfl"; src = off; break;
    }
    const std::string srcName = fresh("s");
    body << pad() << "const int " << srcName << " = " << src << ";\n";
    const std::string okName = fresh("v");
    names[op->getResult(1).getImpl()] = okName;
    body << pad() << "const bool " << okName << " = " << srcName << " >= 0 && " << srcName << " < " << width << ";\n";
    const std::string got = fresh("g");
    body << pad() << "const " << valueType(op->getResult(0).getType()) << " " << got << " = " << fn << "(" << value << ", " << off << ", " << width << ");\n";
    define(op, 0);
    body << okName << " ? " << got << " : " << value << ";\n";
  }
};

}  // namespace

const char* schedulePrelude() {
  return "#ifndef KCG_SCHEDULE_HELPERS\n"
         "#define KCG_SCHEDULE_HELPERS\n"
         "// floor division and the matching remainder for operands that may be negative (affine floordiv / mod)\n"
         "template <class T> static __device__ __forceinline__ T kcg_floordiv(T a, T b) { const T q = a / b; return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; }\n"
         "template <class T> static __device__ __forceinline__ T kcg_floormod(T a, T b) { const T r = a % b; return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r; }\n"
         "template <class T> static __device__ __forceinline__ T kcg_ceildiv(T a, T b) { return -kcg_floordiv<T>(-a, b); }\n"
         "#endif\n";
}

bool emitSchedule(func::FuncOp f, const std::string& kernelName, std::string& text, KernelLaunchInfo& info, std::string& err) {
  try {
    Emitter e(f, kernelName);
    e.run(text, info);
    text = std::string(schedulePrelude()) + text;
    return true;
  } catch (const Failure& failure) {
    err = failure.what;
    return false;
  }
}

}  // namespace hipgen
}  // namespace KernelCodeGen
