// Host interpreter of the mini affine IR (see include/IR/Interpreter.h).
#include "IR/Interpreter.h"

#include <cmath>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <unordered_map>

using namespace mlir;

namespace KernelCodeGen {

namespace {

float bf16Round(float v) {
  uint32_t u;
  memcpy(&u, &v, 4);
  if ((u & 0x7F800000u) == 0x7F800000u) return v;
  u += 0x7FFFu + ((u >> 16) & 1u);
  u &= 0xFFFF0000u;
  memcpy(&v, &u, 4);
  return v;
}

// nearest value on a grid with `mant` explicit mantissa bits, minimum normal exponent `emin`
double gridRound(double v, int mant, int emin, double maxFinite, bool saturate) {
  if (!std::isfinite(v) || v == 0.0) return v;
  int e;
  (void)std::frexp(v, &e);
  int ulpExp = (e - 1 < emin ? emin : e - 1) - mant;
  double r = std::ldexp(std::nearbyint(std::ldexp(v, -ulpExp)), ulpExp);
  if (std::fabs(r) > maxFinite) return saturate ? std::copysign(maxFinite, v) : std::copysign(INFINITY, v);
  return r;
}

[[noreturn]] void fail(const std::string& msg) { throw std::runtime_error("interpreter: " + msg); }

struct Storage {
  std::vector<int64_t> shape;
  Type element;
  std::vector<double> data;
  int64_t perThread = 0;  // 0: one instance; else number of elements of one thread's instance
  // Shared (workgroup) memory only: who touched each element since which barrier. Thread ids; -1 nobody, -2 all/several.
  bool shared = false;
  std::vector<int32_t> writer, reader;
  std::vector<int64_t> writeEpoch, readEpoch;
  int64_t count() const { int64_t n = 1; for (auto d : shape) n *= d; return n; }
};

struct Val {
  std::vector<double> v;       // uniform: width entries; else nThreads * width
  int width = 1;
  bool uniform = true;
  std::shared_ptr<Storage> mem;  // memref values
  // a scalar operand of a vector operation broadcasts over the lanes of the vector
  double at(int t, int j = 0) const {
    const int jj = width == 1 ? 0 : j;
    return uniform ? v[jj] : v[(size_t)t * width + jj];
  }
};

struct Machine {
  Interpreter& host;
  ModuleOp module;
  std::unordered_map<detail::ValueImpl*, Val> env;
  int nThreads = 1;
  std::vector<char> mask;  // active threads (size nThreads)
  int parallelDepth = 0;
  int64_t epoch = 0;  // barriers passed so far; two accesses with equal epoch have no barrier between them

  // ---- missing-barrier audit ------------------------------------------------------
  // Threads run in lock-step here, so a schedule without barriers still computes the right values. On the GPU the same
  // schedule races. An element of shared memory that one thread writes and another thread reads or overwrites with no
  // barrier in between is counted as a hazard. A store of one value by every thread is not.
  void hazard(const char* kind, Operation* op, int64_t lin, int a, int b) {
    if (host.sharedHazards++ == 0) {
      std::ostringstream os;
      os << kind << " on shared memory without a barrier in " << op->getName() << ": element " << lin << ", threads " << a
         << " and " << b;
      host.firstHazard = os.str();
    }
  }
  // Who performs an access that is the same for every thread (executed once): all active threads, written -2; under
  // a condition that leaves one thread active (`if (tid == 0)`), that thread.
  int everyone() const {
    int only = -1;
    for (int t = 0; t < nThreads; ++t)
      if (mask[t]) { if (only >= 0) return -2; only = t; }
    return only >= 0 ? only : -2;
  }
  void noteRead(Storage& s, int64_t lin, int t, Operation* op) {
    if (!s.shared || nThreads == 1) return;
    const size_t i = (size_t)lin;
    if (s.writeEpoch[i] == epoch && s.writer[i] >= 0 && s.writer[i] != t) hazard("read after write", op, lin, s.writer[i], t);
    if (s.readEpoch[i] != epoch) { s.readEpoch[i] = epoch; s.reader[i] = t; }
    else if (s.reader[i] != t) s.reader[i] = -2;
  }
  void noteWrite(Storage& s, int64_t lin, int t, double value, Operation* op) {
    if (!s.shared || nThreads == 1) return;
    const size_t i = (size_t)lin;
    if (s.readEpoch[i] == epoch && s.reader[i] != -1 && s.reader[i] != t) hazard("write after read", op, lin, s.reader[i], t);
    if (s.writeEpoch[i] == epoch && s.writer[i] != -1 && s.writer[i] != t) {
      const double old = s.data[i];
      if (!(old == value || (std::isnan(old) && std::isnan(value)))) hazard("write after write", op, lin, s.writer[i], t);
    }
    s.writeEpoch[i] = epoch;
    s.writer[i] = t;
  }

  Machine(Interpreter& h, ModuleOp m) : host(h), module(m), mask(1, 1) {}

  Val& get(Value v) {
    auto it = env.find(v.getImpl());
    if (it == env.end()) fail("use of a value that has not been computed");
    return it->second;
  }

  void setScalar(Value v, const std::vector<double>& perThread, bool uniform, int width = 1) {
    Val& d = env[v.getImpl()];
    d.v = perThread;
    d.width = width;
    d.uniform = uniform;
    d.mem = nullptr;
  }

  bool allUniform(Operation* op) {
    for (Value o : op->getOperands())
      if (!get(o).uniform) return false;
    return true;
  }

  // ---- elementwise arithmetic -------------------------------------------------
  double apply1(OpKind k, double a, Type t) {
    double r;
    const bool f32 = t.isF32();
    switch (k) {
      case OpKind::Exp: r = f32 ? (double)expf((float)a) : std::exp(a); break;
      case OpKind::Exp2: r = f32 ? (double)exp2f((float)a) : std::exp2(a); break;
      case OpKind::Tanh: r = f32 ? (double)tanhf((float)a) : std::tanh(a); break;
      case OpKind::Sqrt: r = f32 ? (double)sqrtf((float)a) : std::sqrt(a); break;
      case OpKind::Rsqrt: r = f32 ? (double)(1.0f / sqrtf((float)a)) : 1.0 / std::sqrt(a); break;
      case OpKind::Log: r = f32 ? (double)logf((float)a) : std::log(a); break;
      case OpKind::Abs: r = std::fabs(a); break;
      case OpKind::NegF: r = -a; break;
      default: fail("unsupported unary op");
    }
    return roundToType(r, t);
  }
  double apply2(OpKind k, double a, double b, Type t) {
    double r;
    switch (k) {
      case OpKind::AddF: r = a + b; break;
      case OpKind::SubF: r = a - b; break;
      case OpKind::MulF: r = a * b; break;
      case OpKind::DivF: r = a / b; break;
      case OpKind::MaxF: r = (a != a || b != b) ? NAN : (a > b ? a : b); break;
      case OpKind::MinF: r = (a != a || b != b) ? NAN : (a < b ? a : b); break;
      case OpKind::PowF: r = t.isF32() ? (double)powf((float)a, (float)b) : std::pow(a, b); break;
      case OpKind::AddI: return (double)((int64_t)a + (int64_t)b);
      case OpKind::SubI: return (double)((int64_t)a - (int64_t)b);
      case OpKind::MulI: return (double)((int64_t)a * (int64_t)b);
      default: fail("unsupported binary op");
    }
    // a double sum/product/quotient of two fp32 values rounds to fp32 exactly as the fp32 operation does
    return roundToType(r, t);
  }

  // ---- memory -----------------------------------------------------------------
  int64_t linearIndex(const Storage& s, AffineMap map, const std::vector<int64_t>& inputs, int extent, Operation* op) {
    auto idx = map.evaluate(inputs);
    int64_t lin = 0;
    for (size_t d = 0; d < s.shape.size(); ++d) {
      int64_t i = idx[d];
      int64_t hi = i + (d + 1 == s.shape.size() ? extent - 1 : 0);
      ++host.outOfBoundsChecks;
      if (i < 0 || hi >= s.shape[d]) {
        std::ostringstream os;
        os << "out-of-bounds access in " << op->getName() << ": index " << i << " (+" << extent - 1 << ") in dimension " << d
           << " of extent " << s.shape[d];
        fail(os.str());
      }
      lin = lin * s.shape[d] + i;
    }
    return lin;
  }

  void execAccess(Operation* op) {
    const bool isStore = op->getKind() == OpKind::AffineStore || op->getKind() == OpKind::AffineVectorStore;
    const bool isVector = op->getKind() == OpKind::AffineVectorLoad || op->getKind() == OpKind::AffineVectorStore;
    const unsigned memIdx = isStore ? 1 : 0;
    Val& m = get(op->getOperand(memIdx));
    if (!m.mem) fail("access to a value that is not a memref");
    Storage& s = *m.mem;
    AffineMap map = op->getAttr("map").map;
    int width = 1;
    if (isVector) {
      Type vt = isStore ? op->getOperand(0).getType() : op->getResult(0).getType();
      width = (int)vt.cast<VectorType>().getNumElements();
    }
    const unsigned nIdx = op->getNumOperands() - memIdx - 1;
    std::vector<const Val*> idxVals;
    bool uniformIdx = true;
    for (unsigned i = 0; i < nIdx; ++i) {
      idxVals.push_back(&get(op->getOperand(memIdx + 1 + i)));
      if (!idxVals.back()->uniform) uniformIdx = false;
    }
    const Val* stored = isStore ? &get(op->getOperand(0)) : nullptr;
    const bool uniformAll = uniformIdx && !s.perThread && (!stored || stored->uniform);
    std::vector<int64_t> inputs(nIdx);
    if (!isStore) {
      std::vector<double> out((size_t)(uniformAll ? 1 : nThreads) * width, 0.0);
      for (int t = 0; t < (uniformAll ? 1 : nThreads); ++t) {
        if (!uniformAll && !mask[t]) continue;
        for (unsigned i = 0; i < nIdx; ++i) inputs[i] = (int64_t)idxVals[i]->at(t);
        int64_t lin = linearIndex(s, map, inputs, width, op) + (s.perThread ? (int64_t)t * s.perThread : 0);
        for (int j = 0; j < width; ++j) {
          noteRead(s, lin + j, uniformAll ? everyone() : t, op);
          out[(size_t)t * width + j] = s.data[lin + j];
        }
      }
      setScalar(op->getResult(0), out, uniformAll, width);
    } else {
      if (stored->width != width) fail("stored value width differs from the access width");
      for (int t = 0; t < nThreads; ++t) {
        if (!mask[t]) continue;
        for (unsigned i = 0; i < nIdx; ++i) inputs[i] = (int64_t)idxVals[i]->at(t);
        int64_t lin = linearIndex(s, map, inputs, width, op) + (s.perThread ? (int64_t)t * s.perThread : 0);
        for (int j = 0; j < width; ++j) {
          noteWrite(s, lin + j, uniformAll ? everyone() : t, stored->at(t, j), op);
          s.data[lin + j] = stored->at(t, j);
        }
      }
    }
  }

  // memref.load / memref.store: the subscripts are index values, one per dimension
  void execMemAccess(Operation* op, bool isStore) {
    const unsigned memIdx = isStore ? 1 : 0;
    const Val& m = get(op->getOperand(memIdx));
    if (!m.mem) fail("memref.load/store of a value that is not a memref");
    Storage& s = *m.mem;
    const unsigned nIdx = op->getNumOperands() - memIdx - 1;
    if (nIdx != s.shape.size()) fail("memref.load/store: one subscript per dimension is required");
    std::vector<const Val*> idxVals;
    bool uniformIdx = true;
    for (unsigned i = 0; i < nIdx; ++i) {
      idxVals.push_back(&get(op->getOperand(memIdx + 1 + i)));
      if (!idxVals.back()->uniform) uniformIdx = false;
    }
    const Val* stored = isStore ? &get(op->getOperand(0)) : nullptr;
    const bool uniformAll = uniformIdx && !s.perThread && (!stored || stored->uniform);
    auto linear = [&](int t) {
      int64_t lin = 0;
      for (unsigned i = 0; i < nIdx; ++i) {
        const int64_t v = (int64_t)idxVals[i]->at(t);
        ++host.outOfBoundsChecks;
        if (v < 0 || v >= s.shape[i])
          fail("memref subscript " + std::to_string(v) + " is outside dimension " + std::to_string(i) + " of extent " +
               std::to_string(s.shape[i]));
        lin = lin * s.shape[i] + v;
      }
      return lin + (s.perThread ? (int64_t)t * s.perThread : 0);
    };
    if (!isStore) {
      std::vector<double> out((size_t)(uniformAll ? 1 : nThreads), 0.0);
      for (int t = 0; t < (uniformAll ? 1 : nThreads); ++t) {
        if (!uniformAll && !mask[t]) continue;
        const int64_t lin = linear(t);
        noteRead(s, lin, uniformAll ? everyone() : t, op);
        out[(size_t)t] = s.data[(size_t)lin];
      }
      setScalar(op->getResult(0), out, uniformAll);
    } else {
      for (int t = 0; t < nThreads; ++t) {
        if (!mask[t]) continue;
        const int64_t lin = linear(t);
        noteWrite(s, lin, uniformAll ? everyone() : t, stored->at(t), op);
        s.data[(size_t)lin] = stored->at(t);
      }
    }
  }

  void execAlloc(Operation* op) {
    auto mt = op->getResult(0).getType().cast<MemRefType>();
    auto st = std::make_shared<Storage>();
    st->shape = mt.getShape().vec();
    st->element = mt.getElementType();
    const int64_t n = st->count();
    if (mt.getMemorySpaceAsInt() == 3 && nThreads > 1) {
      st->perThread = n;
      st->data.assign((size_t)n * nThreads, NAN);  // registers start undefined
    } else {
      st->data.assign((size_t)n, mt.getMemorySpaceAsInt() == 1 ? 0.0 : NAN);
    }
    if (mt.getMemorySpaceAsInt() == 2) {
      st->shared = true;
      st->writer.assign((size_t)n, -1);
      st->reader.assign((size_t)n, -1);
      st->writeEpoch.assign((size_t)n, -1);
      st->readEpoch.assign((size_t)n, -1);
    }
    Val& d = env[op->getResult(0).getImpl()];
    d = Val();
    d.mem = st;
  }

  // ---- control flow -------------------------------------------------------------
  void execBlock(Block* b) {
    for (auto& op : b->getOperations()) exec(&op);
  }

  void execFor(Operation* op) {
    AffineForOp loop(op);
    auto bound = [&](AffineMap m, ValueRange operands, bool lower) {
      std::vector<int64_t> in;
      for (Value v : operands) {
        Val& x = get(v);
        if (!x.uniform) fail("loop bound differs between threads");
        in.push_back((int64_t)x.v[0]);
      }
      auto r = m.evaluate(in);
      int64_t best = r[0];
      for (auto x : r) best = lower ? std::max(best, x) : std::min(best, x);
      return best;
    };
    const int64_t lb = bound(loop.getLowerBoundMap(), loop.getLowerBoundOperands(), true);
    const int64_t ub = bound(loop.getUpperBoundMap(), loop.getUpperBoundOperands(), false);
    const int64_t step = loop.getStep();
    auto regionArgs = loop.getRegionIterArgs();
    auto inits = loop.getIterOperands();
    std::vector<Val> carried;
    for (Value v : inits) carried.push_back(get(v));
    Operation* yield = loop.getBody()->getTerminator();
    for (int64_t iv = lb; iv < ub; iv += step) {
      setScalar(loop.getInductionVar(), {(double)iv}, true);
      for (size_t i = 0; i < regionArgs.size(); ++i) env[regionArgs[i].getImpl()] = carried[i];
      execBlock(loop.getBody());
      for (size_t i = 0; i < carried.size(); ++i) {
        Val next = get(yield->getOperand((unsigned)i));
        if (nThreads > 1 && !(next.uniform && carried[i].uniform)) {
          // inactive threads keep their previous value
          Val merged;
          merged.width = next.width;
          merged.uniform = false;
          merged.v.resize((size_t)nThreads * next.width);
          for (int t = 0; t < nThreads; ++t)
            for (int j = 0; j < next.width; ++j)
              merged.v[(size_t)t * next.width + j] = mask[t] ? next.at(t, j) : carried[i].at(t, j);
          carried[i] = merged;
        } else {
          carried[i] = next;
        }
      }
    }
    for (size_t i = 0; i < carried.size(); ++i) env[op->getResult((unsigned)i).getImpl()] = carried[i];
  }

  void execParallel(Operation* op) {
    AffineParallelOp par(op);
    auto lbs = par.getConstantLowerBounds(), ubs = par.getConstantUpperBounds();
    auto steps = par.getSteps();
    auto ivs = par.getIVs();
    const size_t nd = ubs.size();
    std::vector<int64_t> extent(nd);
    int64_t total = 1;
    for (size_t d = 0; d < nd; ++d) { extent[d] = (ubs[d] - lbs[d] + steps[d] - 1) / steps[d]; total *= extent[d]; }
    ++parallelDepth;
    if (parallelDepth == 1) {
      // grid level: one workgroup after the other
      for (int64_t lin = 0; lin < total; ++lin) {
        int64_t rem = lin;
        for (size_t d = nd; d-- > 0;) {
          setScalar(ivs[d], {(double)(lbs[d] + (rem % extent[d]) * steps[d])}, true);
          rem /= extent[d];
        }
        execBlock(par.getBody());
      }
    } else {
      // workgroup level: all threads in lock-step; thread id = row-major position, last dim fastest
      if (nThreads != 1) fail("more than two nested parallel levels");
      nThreads = (int)total;
      mask.assign((size_t)total, 1);
      for (size_t d = 0; d < nd; ++d) {
        std::vector<double> iv((size_t)total);
        for (int64_t lin = 0; lin < total; ++lin) {
          int64_t rem = lin;
          for (size_t e = nd; e-- > d + 1;) rem /= extent[e];
          iv[(size_t)lin] = (double)(lbs[d] + (rem % extent[d]) * steps[d]);
        }
        setScalar(ivs[d], iv, false);
      }
      execBlock(par.getBody());
      nThreads = 1;
      mask.assign(1, 1);
    }
    --parallelDepth;
  }

  void execIf(Operation* op) {
    AffineIfOp ifOp(op);
    IntegerSet set = ifOp.getIntegerSet();
    std::vector<const Val*> in;
    bool uniform = true;
    for (Value v : op->getOperands()) { in.push_back(&get(v)); if (!in.back()->uniform) uniform = false; }
    std::vector<int64_t> inputs(in.size());
    std::vector<char> saved = mask, thenMask(mask.size(), 0), elseMask(mask.size(), 0);
    bool anyThen = false, anyElse = false;
    for (int t = 0; t < nThreads; ++t) {
      if (!saved[t]) continue;
      for (size_t i = 0; i < in.size(); ++i) inputs[i] = (int64_t)in[i]->at(uniform ? 0 : t);
      if (set.contains(inputs)) { thenMask[t] = 1; anyThen = true; } else { elseMask[t] = 1; anyElse = true; }
    }
    if (anyThen) { mask = thenMask; execBlock(ifOp.getThenBlock()); }
    if (anyElse && ifOp.hasElse()) { mask = elseMask; execBlock(ifOp.getElseBlock()); }
    mask = saved;
  }

  void execShuffle(Operation* op) {
    gpu::ShuffleOp sh(op);
    const Val& v = get(sh.getValue());
    const Val& off = get(sh.getOffset());
    const Val& w = get(sh.getWidth());
    std::vector<double> out((size_t)nThreads), valid((size_t)nThreads);
    for (int t = 0; t < nThreads; ++t) {
      const int width = (int)w.at(t), o = (int)off.at(t);
      if (width <= 0 || nThreads % width) fail("shuffle width does not divide the block");
      const int base = t / width * width, lane = t - base;
      int src = lane;
      switch (sh.getMode()) {
        case gpu::ShuffleMode::DOWN: src = lane + o; break;
        case gpu::ShuffleMode::UP: src = lane - o; break;
        case gpu::ShuffleMode::XOR: src = lane ^ o; break;
        case gpu::ShuffleMode::IDX: src = o; break;
      }
      const bool ok = src >= 0 && src < width;
      out[(size_t)t] = v.at(ok ? base + src : t);
      valid[(size_t)t] = ok ? 1.0 : 0.0;
    }
    setScalar(op->getResult(0), out, false);
    setScalar(op->getResult(1), valid, false);
  }

  std::vector<HostTensor> callFunction(func::FuncOp f, const std::vector<std::shared_ptr<Storage>>& args) {
    if (f.empty()) fail("call of a function without a body: " + f.getSymName());
    if (args.size() != f.getNumArguments()) fail("wrong number of arguments for " + f.getSymName());
    for (unsigned i = 0; i < args.size(); ++i) {
      auto mt = f.getArgument(i).getType().dyn_cast<MemRefType>();
      if (!mt) fail("only memref arguments are supported");
      if (mt.getShape().vec() != args[i]->shape || mt.getElementType() != args[i]->element)
        fail("argument " + std::to_string(i) + " of " + f.getSymName() + " has the wrong shape or element type");
      Val& d = env[f.getArgument(i).getImpl()];
      d = Val();
      d.mem = args[i];
    }
    returned.clear();
    execBlock(&f.front());
    std::vector<HostTensor> out;
    for (auto& st : returned) out.push_back(HostTensor{st->shape, st->element, st->data});
    return out;
  }
  std::vector<std::shared_ptr<Storage>> returned;

  void exec(Operation* op) {
    switch (op->getKind()) {
      case OpKind::Alloc: execAlloc(op); return;
      case OpKind::AffineFor: execFor(op); return;
      case OpKind::AffineParallel: execParallel(op); return;
      case OpKind::AffineIf: execIf(op); return;
      case OpKind::AffineLoad: case OpKind::AffineStore: case OpKind::AffineVectorLoad: case OpKind::AffineVectorStore:
        execAccess(op); return;
      case OpKind::MemLoad: execMemAccess(op, false); return;
      case OpKind::MemStore: execMemAccess(op, true); return;
      case OpKind::AffineYield: return;
      case OpKind::Barrier:
        ++host.barriersExecuted;
        ++epoch;
        for (int t = 0; t < nThreads; ++t)
          if (!mask[t]) { hazard("barrier that some threads skip", op, -1, t, t); break; }
        return;
      case OpKind::Shuffle: execShuffle(op); return;
      case OpKind::Return:
        returned.clear();
        for (Value v : op->getOperands()) {
          if (!get(v).mem) fail("only memrefs can be returned");
          returned.push_back(get(v).mem);
        }
        return;
      case OpKind::Constant: {
        Attribute a = op->getAttr("value");
        setScalar(op->getResult(0), {a.kind == Attribute::Float ? a.f : (double)a.i}, true);
        return;
      }
      case OpKind::AffineApply: {
        AffineMap map = op->getAttr("map").map;
        const bool uni = allUniform(op);
        const int n = uni ? 1 : nThreads;
        std::vector<double> out((size_t)n);
        std::vector<int64_t> in(op->getNumOperands());
        for (int t = 0; t < n; ++t) {
          for (unsigned i = 0; i < op->getNumOperands(); ++i) in[i] = (int64_t)get(op->getOperand(i)).at(t);
          out[(size_t)t] = (double)map.evaluate(in)[0];
        }
        setScalar(op->getResult(0), out, uni);
        return;
      }
      default: break;
    }
    // elementwise ops over scalars or vectors
    const bool uni = allUniform(op);
    const int n = uni ? 1 : nThreads;
    Type rt = op->getResult(0).getType();
    Type et = rt.isa<VectorType>() ? rt.cast<VectorType>().getElementType() : rt;
    const int width = rt.isa<VectorType>() ? (int)rt.cast<VectorType>().getNumElements() : 1;
    std::vector<double> out((size_t)n * width);
    auto operand = [&](unsigned i) -> const Val& { return get(op->getOperand(i)); };
    for (int t = 0; t < n; ++t)
      for (int j = 0; j < width; ++j) {
        double r;
        switch (op->getKind()) {
          case OpKind::AddF: case OpKind::SubF: case OpKind::MulF: case OpKind::DivF: case OpKind::MaxF: case OpKind::MinF:
          case OpKind::PowF: case OpKind::AddI: case OpKind::SubI: case OpKind::MulI:
            r = apply2(op->getKind(), operand(0).at(t, j), operand(1).at(t, j), et); break;
          case OpKind::Exp: case OpKind::Exp2: case OpKind::Tanh: case OpKind::Sqrt: case OpKind::Rsqrt: case OpKind::Log:
          case OpKind::Abs: case OpKind::NegF:
            r = apply1(op->getKind(), operand(0).at(t, j), et); break;
          case OpKind::CmpF: {
            const double a = operand(0).at(t, j), b = operand(1).at(t, j);
            switch ((arith::CmpFPredicate)op->getAttr("predicate").i) {
              case arith::CmpFPredicate::OEQ: r = a == b; break;
              case arith::CmpFPredicate::OGT: r = a > b; break;
              case arith::CmpFPredicate::OGE: r = a >= b; break;
              case arith::CmpFPredicate::OLT: r = a < b; break;
              case arith::CmpFPredicate::OLE: r = a <= b; break;
              case arith::CmpFPredicate::ONE: r = a != b && a == a && b == b; break;
              default: fail("unsupported cmpf predicate");
            }
            break;
          }
          case OpKind::Select: r = operand(0).at(t, j) != 0.0 ? operand(1).at(t, j) : operand(2).at(t, j); break;
          case OpKind::ExtF: case OpKind::TruncF: r = roundToType(operand(0).at(t, j), et); break;
          case OpKind::SIToFP: r = roundToType(operand(0).at(t, j), et); break;
          // The Frontend's "Cast" is an arith.bitcast that the backends print as a
          // value conversion (static_cast); both execute it as one.
          case OpKind::FPToSI: case OpKind::Bitcast:
            r = et.isFloat() ? roundToType(operand(0).at(t, j), et) : std::trunc(operand(0).at(t, j)); break;
          default: fail(std::string("unsupported operation ") + op->getName());
        }
        out[(size_t)t * width + j] = r;
      }
    setScalar(op->getResult(0), out, uni, width);
  }
};

}  // namespace

double roundToType(double v, Type type) {
  if (type.isF64()) return v;
  if (type.isF32()) return (double)(float)v;
  if (type.isBF16()) return (double)bf16Round((float)v);
  if (type.isF16()) return gridRound(v, 10, -14, 65504.0, false);
  if (type.isa<Float8E4M3FNType>()) return v != v ? v : gridRound(std::isinf(v) ? std::copysign(448.0, v) : v, 3, -6, 448.0, true);
  if (type.isIntOrIndex()) return std::trunc(v);
  return v;
}

std::vector<HostTensor> Interpreter::run(func::FuncOp func, std::vector<HostTensor>& args) {
  Machine m(*this, module);
  std::vector<std::shared_ptr<Storage>> bound;
  for (auto& a : args) {
    auto st = std::make_shared<Storage>();
    st->shape = a.shape;
    st->element = a.elementType;
    st->data = a.data;
    if ((int64_t)st->data.size() != st->count()) fail("argument data size differs from its shape");
    bound.push_back(st);
  }
  auto out = m.callFunction(func, bound);
  for (size_t i = 0; i < args.size(); ++i) args[i].data = bound[i]->data;  // in-place results are visible to the caller
  return out;
}

std::vector<HostTensor> Interpreter::runGraph(std::vector<HostTensor>& placeholders) {
  std::unordered_map<detail::ValueImpl*, std::shared_ptr<Storage>> values;
  std::vector<std::pair<size_t, std::shared_ptr<Storage>>> boundPlaceholders;
  std::vector<HostTensor> results;
  size_t next = 0;
  for (auto& op : module.getBody()->getOperations()) {
    if (op.getKind() == OpKind::Alloc) {
      auto mt = op.getResult(0).getType().cast<MemRefType>();
      auto st = std::make_shared<Storage>();
      st->shape = mt.getShape().vec();
      st->element = mt.getElementType();
      if (!op.hasAttr("kcg.result") && next < placeholders.size()) {
        if (placeholders[next].shape != st->shape) fail("placeholder " + std::to_string(next) + " has the wrong shape");
        st->data = placeholders[next].data;
        boundPlaceholders.emplace_back(next, st);
        ++next;
      } else {
        st->data.assign((size_t)st->count(), 0.0);
        if (!op.hasAttr("kcg.result")) ++next;
      }
      values[op.getResult(0).getImpl()] = st;
    } else if (op.getKind() == OpKind::Call) {
      func::FuncOp callee;
      const std::string name = op.getAttr("callee").s;
      for (auto& f : module.getBody()->getOperations())
        if (f.getKind() == OpKind::Func && func::FuncOp(&f).getSymName() == name) callee = func::FuncOp(&f);
      if (!callee) fail("call of unknown function " + name);
      Machine m(*this, module);
      std::vector<std::shared_ptr<Storage>> args;
      for (Value v : op.getOperands()) {
        auto it = values.find(v.getImpl());
        if (it == values.end()) fail("call operand is not a graph value");
        args.push_back(it->second);
      }
      m.callFunction(callee, args);
      for (unsigned i = 0; i < op.getNumResults(); ++i) {
        values[op.getResult(i).getImpl()] = m.returned[i];
        results.push_back(HostTensor{m.returned[i]->shape, m.returned[i]->element, m.returned[i]->data});
      }
    }
  }
  for (auto& kv : boundPlaceholders) placeholders[kv.first].data = kv.second->data;
  return results;
}

}  // namespace KernelCodeGen
