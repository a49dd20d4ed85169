// Textual form (MLIR custom syntax) and structural verifier of the mini IR.
#include <sstream>

#include "IR/MLIR.h"

namespace mlir {

namespace {

struct PrintState {
  std::unordered_map<detail::ValueImpl*, std::string> names;
  std::map<std::string, int> used;
  int nextResult = 0;
  int nextArg = 0;

  std::string unique(const std::string& base) {
    int& n = used[base];
    std::string s = n == 0 ? base : base + "_" + std::to_string(n - 1);
    ++n;
    return s;
  }
  std::string name(Value v) {
    auto it = names.find(v.getImpl());
    if (it != names.end()) return it->second;
    return "%<<unknown>>";
  }
  void nameArg(Value v) { names[v.getImpl()] = "%arg" + std::to_string(nextArg++); }
  void nameResult(Operation* op) {
    if (op->getNumResults() == 0) return;
    std::string base;
    if (op->getKind() == OpKind::Constant) {
      Attribute a = op->getAttr("value");
      if (a.kind == Attribute::Integer && a.i >= 0) base = "%c" + std::to_string(a.i);
      else if (a.kind == Attribute::Integer) base = "%c-" + std::to_string(-a.i);
      else base = "%cst";
      if (a.kind == Attribute::Integer && !a.type.isIndex()) base += "_i" + std::to_string(a.type.getIntOrFloatBitWidth());
      names[op->getResult(0).getImpl()] = unique(base);
      return;
    }
    std::string n = "%" + std::to_string(nextResult++);
    if (op->getNumResults() == 1) names[op->getResult(0).getImpl()] = n;
    else
      for (unsigned i = 0; i < op->getNumResults(); ++i) names[op->getResult(i).getImpl()] = n + "#" + std::to_string(i);
  }
};

void indent(std::ostream& os, int n) { for (int i = 0; i < n; ++i) os << "  "; }

// Prints `expr` with d_i replaced by the SSA names of the operands, the way
// MLIR prints the subscripts of affine accesses.
void printBoundExpr(std::ostream& os, AffineExpr e, const std::vector<std::string>& names, unsigned numDims, bool paren) {
  switch (e.getKind()) {
    case AffineExprKind::Constant: os << e.cast<AffineConstantExpr>().getValue(); return;
    case AffineExprKind::DimId: os << names[e.cast<AffineDimExpr>().getPosition()]; return;
    case AffineExprKind::SymbolId: os << "symbol(" << names[numDims + e.cast<AffineSymbolExpr>().getPosition()] << ")"; return;
    default: break;
  }
  auto b = e.cast<AffineBinaryOpExpr>();
  AffineExpr l = b.getLHS(), r = b.getRHS();
  if (paren) os << "(";
  if (e.getKind() == AffineExprKind::Add) {
    printBoundExpr(os, l, names, numDims, false);
    auto rc = r.dyn_cast<AffineConstantExpr>();
    if (rc && rc.getValue() < 0) os << " - " << -rc.getValue();
    else if (r.getKind() == AffineExprKind::Mul && r.cast<AffineBinaryOpExpr>().getRHS() == -1) {
      os << " - ";
      printBoundExpr(os, r.cast<AffineBinaryOpExpr>().getLHS(), names, numDims, true);
    } else {
      os << " + ";
      printBoundExpr(os, r, names, numDims, false);
    }
  } else {
    const char* sym = e.getKind() == AffineExprKind::Mul ? " * " : e.getKind() == AffineExprKind::Mod ? " mod "
                    : e.getKind() == AffineExprKind::FloorDiv ? " floordiv " : " ceildiv ";
    if (e.getKind() == AffineExprKind::Mul && r == -1) { os << "-"; printBoundExpr(os, l, names, numDims, true); }
    else { printBoundExpr(os, l, names, numDims, true); os << sym; printBoundExpr(os, r, names, numDims, true); }
  }
  if (paren) os << ")";
}

void printSubscripts(std::ostream& os, PrintState& st, AffineMap map, const std::vector<Value>& operands) {
  std::vector<std::string> names;
  for (Value v : operands) names.push_back(st.name(v));
  os << "[";
  for (unsigned i = 0; i < map.getNumResults(); ++i) {
    if (i) os << ", ";
    printBoundExpr(os, map.getResult(i), names, map.getNumDims(), false);
  }
  os << "]";
}

void printOp(std::ostream& os, PrintState& st, Operation* op, int level);

void printBlockBody(std::ostream& os, PrintState& st, Block* b, int level, bool skipEmptyYield) {
  for (auto& op : b->getOperations()) {
    if (skipEmptyYield && op.getKind() == OpKind::AffineYield && op.getNumOperands() == 0) continue;
    printOp(os, st, &op, level);
  }
}

void printExtraAttrs(std::ostream& os, Operation* op, std::initializer_list<const char*> elided, const char* prefix) {
  std::vector<std::pair<std::string, Attribute>> rest;
  for (auto& kv : op->getAttrs()) {
    bool skip = false;
    for (auto e : elided) if (kv.first == e) skip = true;
    if (!skip) rest.push_back(kv);
  }
  if (rest.empty()) return;
  os << prefix << "{";
  for (size_t i = 0; i < rest.size(); ++i) {
    if (i) os << ", ";
    os << rest[i].first;
    if (rest[i].second.kind != Attribute::Unit) { os << " = "; rest[i].second.print(os); }
  }
  os << "}";
}

void printOperandList(std::ostream& os, PrintState& st, const std::vector<Value>& vs) {
  for (size_t i = 0; i < vs.size(); ++i) os << (i ? ", " : "") << st.name(vs[i]);
}

const char* predicateName(arith::CmpFPredicate p) {
  static const char* names[] = {"false", "oeq", "ogt", "oge", "olt", "ole", "one", "ord",
                                "ueq", "ugt", "uge", "ult", "ule", "une", "uno", "true"};
  return names[(int)p];
}

void printOp(std::ostream& os, PrintState& st, Operation* op, int level) {
  indent(os, level);
  switch (op->getKind()) {
    case OpKind::Module: {
      os << "module";
      if (op->hasAttr("sym_name")) os << " @" << op->getAttr("sym_name").s;
      os << " {\n";
      printBlockBody(os, st, &op->getRegion(0).front(), level + 1, false);
      indent(os, level);
      os << "}\n";
      return;
    }
    case OpKind::Func: {
      func::FuncOp f(op);
      // SSA names restart in every function, as in MLIR
      PrintState outer = st;
      st.nextResult = 0; st.nextArg = 0; st.used.clear();
      os << "func.func @" << f.getSymName() << "(";
      FunctionType ft = f.getFunctionType();
      if (!f.empty()) {
        auto args = f.getArguments();
        for (size_t i = 0; i < args.size(); ++i) {
          st.nameArg(args[i]);
          os << (i ? ", " : "") << st.name(args[i]) << ": " << args[i].getType();
        }
      } else {
        for (unsigned i = 0; i < ft.getNumInputs(); ++i) os << (i ? ", " : "") << ft.getInput(i);
      }
      os << ")";
      if (ft.getNumResults() == 1) os << " -> " << ft.getResult(0);
      else if (ft.getNumResults() > 1) {
        os << " -> (";
        for (unsigned i = 0; i < ft.getNumResults(); ++i) os << (i ? ", " : "") << ft.getResult(i);
        os << ")";
      }
      printExtraAttrs(os, op, {"sym_name", "function_type"}, " attributes ");
      if (f.empty()) { os << "\n"; }
      else {
        os << " {\n";
        printBlockBody(os, st, &f.front(), level + 1, false);
        indent(os, level);
        os << "}\n";
      }
      // keep names of values defined outside functions (module-level allocs)
      auto inner = st.names;
      st = outer;
      for (auto& kv : inner) st.names.insert(kv);
      return;
    }
    case OpKind::AffineFor: {
      AffineForOp loop(op);
      st.nameResult(op);
      if (op->getNumResults()) os << st.name(op->getResult(0)).substr(0, st.name(op->getResult(0)).find('#')) << " = ";
      st.nameArg(loop.getInductionVar());
      os << "affine.for " << st.name(loop.getInductionVar()) << " = ";
      auto printBound = [&](AffineMap m, ValueRange operands, const char* multi) {
        if (m.isSingleConstant()) { os << m.getSingleConstantResult(); return; }
        if (m.getNumResults() == 1 && m.getNumInputs() == 1 && m.getResult(0) == getAffineDimExpr(0)) { os << st.name(operands[0]); return; }
        if (m.getNumResults() > 1) os << multi << " ";
        os << "affine_map<" << m << ">(";
        printOperandList(os, st, operands);
        os << ")";
      };
      printBound(loop.getLowerBoundMap(), loop.getLowerBoundOperands(), "max");
      os << " to ";
      printBound(loop.getUpperBoundMap(), loop.getUpperBoundOperands(), "min");
      if (loop.getStep() != 1) os << " step " << loop.getStep();
      if (loop.getNumIterOperands()) {
        os << " iter_args(";
        auto ra = loop.getRegionIterArgs();
        auto io = loop.getIterOperands();
        for (size_t i = 0; i < ra.size(); ++i) {
          st.nameArg(ra[i]);
          os << (i ? ", " : "") << st.name(ra[i]) << " = " << st.name(io[i]);
        }
        os << ") -> (";
        for (size_t i = 0; i < ra.size(); ++i) os << (i ? ", " : "") << ra[i].getType();
        os << ")";
      }
      os << " {\n";
      printBlockBody(os, st, loop.getBody(), level + 1, true);
      indent(os, level);
      os << "}";
      printExtraAttrs(os, op, {"lower_bound", "upper_bound", "step", "num_lb_operands", "num_ub_operands"}, " ");
      os << "\n";
      return;
    }
    case OpKind::AffineParallel: {
      AffineParallelOp par(op);
      os << "affine.parallel (";
      auto ivs = par.getIVs();
      for (size_t i = 0; i < ivs.size(); ++i) { st.nameArg(ivs[i]); os << (i ? ", " : "") << st.name(ivs[i]); }
      os << ") = (";
      auto lbs = par.getConstantLowerBounds(), ubs = par.getConstantUpperBounds();
      auto steps = par.getSteps();
      for (size_t i = 0; i < lbs.size(); ++i) os << (i ? ", " : "") << lbs[i];
      os << ") to (";
      for (size_t i = 0; i < ubs.size(); ++i) os << (i ? ", " : "") << ubs[i];
      os << ")";
      bool unit = true;
      for (auto s : steps) if (s != 1) unit = false;
      if (!unit) {
        os << " step (";
        for (size_t i = 0; i < steps.size(); ++i) os << (i ? ", " : "") << steps[i];
        os << ")";
      }
      os << " {\n";
      printBlockBody(os, st, par.getBody(), level + 1, true);
      indent(os, level);
      os << "}";
      printExtraAttrs(os, op, {"lower_bounds", "upper_bounds", "steps"}, " ");
      os << "\n";
      return;
    }
    case OpKind::AffineIf: {
      AffineIfOp ifOp(op);
      os << "affine.if affine_set<";
      ifOp.getIntegerSet().print(os);
      os << ">(";
      printOperandList(os, st, op->getOperands());
      os << ") {\n";
      printBlockBody(os, st, ifOp.getThenBlock(), level + 1, true);
      indent(os, level);
      os << "}";
      if (ifOp.hasElse()) {
        os << " else {\n";
        printBlockBody(os, st, ifOp.getElseBlock(), level + 1, true);
        indent(os, level);
        os << "}";
      }
      os << "\n";
      return;
    }
    default: break;
  }

  st.nameResult(op);
  if (op->getNumResults() == 1) os << st.name(op->getResult(0)) << " = ";
  else if (op->getNumResults() > 1) {
    std::string n = st.name(op->getResult(0));
    os << n.substr(0, n.find('#')) << ":" << op->getNumResults() << " = ";
  }
  auto& operands = op->getOperands();
  switch (op->getKind()) {
    case OpKind::Call: {
      os << "func.call @" << op->getAttr("callee").s << "(";
      printOperandList(os, st, operands);
      os << ") : (";
      for (size_t i = 0; i < operands.size(); ++i) os << (i ? ", " : "") << operands[i].getType();
      os << ") -> ";
      if (op->getNumResults() == 1) os << op->getResult(0).getType();
      else {
        os << "(";
        for (unsigned i = 0; i < op->getNumResults(); ++i) os << (i ? ", " : "") << op->getResult(i).getType();
        os << ")";
      }
      break;
    }
    case OpKind::Return:
      os << "return";
      if (!operands.empty()) {
        os << " ";
        printOperandList(os, st, operands);
        os << " : ";
        for (size_t i = 0; i < operands.size(); ++i) os << (i ? ", " : "") << operands[i].getType();
      }
      break;
    case OpKind::Alloc:
      os << "memref.alloc() : " << op->getResult(0).getType();
      printExtraAttrs(os, op, {}, " ");
      break;
    case OpKind::MemLoad:
      os << "memref.load " << st.name(operands[0]) << "[";
      printOperandList(os, st, std::vector<Value>(operands.begin() + 1, operands.end()));
      os << "] : " << operands[0].getType();
      break;
    case OpKind::MemStore:
      os << "memref.store " << st.name(operands[0]) << ", " << st.name(operands[1]) << "[";
      printOperandList(os, st, std::vector<Value>(operands.begin() + 2, operands.end()));
      os << "] : " << operands[1].getType();
      break;
    case OpKind::AffineLoad:
    case OpKind::AffineVectorLoad:
      os << op->getName() << " " << st.name(operands[0]);
      printSubscripts(os, st, op->getAttr("map").map, std::vector<Value>(operands.begin() + 1, operands.end()));
      os << " : " << operands[0].getType();
      if (op->getKind() == OpKind::AffineVectorLoad) os << ", " << op->getResult(0).getType();
      break;
    case OpKind::AffineStore:
    case OpKind::AffineVectorStore:
      os << op->getName() << " " << st.name(operands[0]) << ", " << st.name(operands[1]);
      printSubscripts(os, st, op->getAttr("map").map, std::vector<Value>(operands.begin() + 2, operands.end()));
      os << " : " << operands[1].getType();
      if (op->getKind() == OpKind::AffineVectorStore) os << ", " << operands[0].getType();
      break;
    case OpKind::AffineApply:
      os << "affine.apply affine_map<" << op->getAttr("map").map << ">(";
      printOperandList(os, st, operands);
      os << ")";
      break;
    case OpKind::AffineYield:
      os << "affine.yield";
      if (!operands.empty()) {
        os << " ";
        printOperandList(os, st, operands);
        os << " : ";
        for (size_t i = 0; i < operands.size(); ++i) os << (i ? ", " : "") << operands[i].getType();
      }
      break;
    case OpKind::Constant:
      os << "arith.constant ";
      op->getAttr("value").print(os);
      break;
    case OpKind::CmpF:
      os << "arith.cmpf " << predicateName((arith::CmpFPredicate)op->getAttr("predicate").i) << ", ";
      printOperandList(os, st, operands);
      os << " : " << operands[0].getType();
      break;
    case OpKind::Bitcast: case OpKind::FPToSI: case OpKind::SIToFP: case OpKind::ExtF: case OpKind::TruncF:
      os << op->getName() << " " << st.name(operands[0]) << " : " << operands[0].getType() << " to " << op->getResult(0).getType();
      break;
    case OpKind::Select:
      os << "arith.select ";
      printOperandList(os, st, operands);
      os << " : " << op->getResult(0).getType();
      break;
    case OpKind::Barrier:
      os << "gpu.barrier";
      break;
    case OpKind::Shuffle: {
      static const char* modes[] = {"xor", "down", "up", "idx"};
      os << "gpu.shuffle " << modes[op->getAttr("mode").i] << " ";
      printOperandList(os, st, operands);
      os << " : " << operands[0].getType();
      break;
    }
    default:
      os << op->getName() << " ";
      printOperandList(os, st, operands);
      if (op->getNumResults()) os << " : " << op->getResult(0).getType();
      break;
  }
  os << "\n";
}

}  // namespace

void Operation::print(std::ostream& os) const {
  PrintState st;
  Operation* self = const_cast<Operation*>(this);
  // give names to values defined above the printed op so that uses resolve
  std::vector<Operation*> chain;
  for (Operation* p = self->getParentOp(); p; p = p->getParentOp()) chain.push_back(p);
  for (auto it = chain.rbegin(); it != chain.rend(); ++it) {
    Operation* p = *it;
    for (unsigned r = 0; r < p->getNumRegions(); ++r)
      for (auto& b : p->getRegion(r).getBlocks()) {
        for (auto a : b->getArguments()) st.nameArg(a);
        for (auto& o : b->getOperations()) {
          if (o.isAncestor(self)) break;
          st.nameResult(&o);
        }
      }
  }
  printOp(os, st, self, 0);
}

// ---------------------------------------------------------------------------
// Verifier
// ---------------------------------------------------------------------------
namespace {
struct Verifier {
  std::string msg;
  bool fail(Operation* op, const std::string& m) {
    std::ostringstream os;
    os << op->getName() << ": " << m;
    msg = os.str();
    return false;
  }

  // A use is legal when the value is defined earlier in the same block or in a
  // block that encloses the user.
  bool dominates(Value v, Operation* user) {
    Block* defBlock = v.getParentBlock();
    Operation* defOp = v.getDefiningOp();
    for (Operation* p = user; p; p = p->getParentOp()) {
      if (p->getBlock() == defBlock) {
        if (!defOp) return true;
        return defOp != p && defOp->isBeforeInBlock(p);
      }
    }
    return false;
  }

  bool checkAccess(Operation* op, unsigned memrefIdx) {
    auto mt = op->getOperand(memrefIdx).getType().dyn_cast<MemRefType>();
    if (!mt) return fail(op, "accessed value is not a memref");
    AffineMap map = op->getAttr("map").map;
    if (!map) return fail(op, "missing access map");
    if (map.getNumResults() != (unsigned)mt.getRank()) return fail(op, "access map rank differs from memref rank");
    if (map.getNumInputs() != op->getNumOperands() - memrefIdx - 1) return fail(op, "access map input count differs from operand count");
    for (unsigned i = memrefIdx + 1; i < op->getNumOperands(); ++i)
      if (!op->getOperand(i).getType().isIndex()) return fail(op, "subscript operand is not of index type");
    return true;
  }

  bool visit(Operation* op) {
    for (unsigned i = 0; i < op->getNumOperands(); ++i) {
      Value v = op->getOperand(i);
      if (!v) return fail(op, "null operand");
      if (!dominates(v, op)) return fail(op, "operand #" + std::to_string(i) + " does not dominate its use");
    }
    switch (op->getKind()) {
      case OpKind::AffineLoad:
        if (!checkAccess(op, 0)) return false;
        if (op->getResult(0).getType() != op->getOperand(0).getType().cast<MemRefType>().getElementType())
          return fail(op, "result type differs from memref element type");
        break;
      case OpKind::AffineVectorLoad: {
        if (!checkAccess(op, 0)) return false;
        auto vt = op->getResult(0).getType().dyn_cast<VectorType>();
        if (!vt || vt.getElementType() != op->getOperand(0).getType().cast<MemRefType>().getElementType())
          return fail(op, "vector element type differs from memref element type");
        break;
      }
      case OpKind::AffineStore:
        if (!checkAccess(op, 1)) return false;
        if (op->getOperand(0).getType() != op->getOperand(1).getType().cast<MemRefType>().getElementType())
          return fail(op, "stored value type differs from memref element type");
        break;
      case OpKind::AffineVectorStore: {
        if (!checkAccess(op, 1)) return false;
        auto vt = op->getOperand(0).getType().dyn_cast<VectorType>();
        if (!vt || vt.getElementType() != op->getOperand(1).getType().cast<MemRefType>().getElementType())
          return fail(op, "vector element type differs from memref element type");
        break;
      }
      case OpKind::AffineFor: {
        AffineForOp loop(op);
        Block* body = loop.getBody();
        if (body->empty() || body->back().getKind() != OpKind::AffineYield) return fail(op, "body must end with affine.yield");
        if (body->back().getNumOperands() != op->getNumResults()) return fail(op, "yield arity differs from the number of loop results");
        if (body->getNumArguments() != 1 + op->getNumResults()) return fail(op, "body argument count differs from 1 + iter_args");
        for (unsigned i = 0; i < op->getNumResults(); ++i)
          if (body->back().getOperand(i).getType() != op->getResult(i).getType()) return fail(op, "yield type differs from result type");
        if (loop.getStep() <= 0) return fail(op, "step must be positive");
        break;
      }
      case OpKind::AffineParallel: {
        Block* body = AffineParallelOp(op).getBody();
        if (body->empty() || body->back().getKind() != OpKind::AffineYield) return fail(op, "body must end with affine.yield");
        break;
      }
      case OpKind::AffineIf: {
        AffineIfOp ifOp(op);
        if (ifOp.getIntegerSet().getNumInputs() != op->getNumOperands()) return fail(op, "set input count differs from operand count");
        break;
      }
      case OpKind::AffineApply:
        if (op->getAttr("map").map.getNumInputs() != op->getNumOperands()) return fail(op, "map input count differs from operand count");
        break;
      case OpKind::AddF: case OpKind::SubF: case OpKind::MulF: case OpKind::DivF: case OpKind::MaxF: case OpKind::MinF:
        // operands have the result type; in a vector operation a scalar operand of the element
        // type is allowed and broadcasts (what a vectorised epilogue does with its constants)
        for (unsigned i = 0; i < 2; ++i) {
          Type ot = op->getOperand(i).getType(), rt = op->getResult(0).getType();
          if (ot != rt && !(rt.isa<VectorType>() && rt.cast<VectorType>().getElementType() == ot))
            return fail(op, "operand and result types differ");
        }
        break;
      case OpKind::Func: {
        func::FuncOp f(op);
        if (!f.empty()) {
          if (f.front().getNumArguments() != f.getFunctionType().getNumInputs()) return fail(op, "entry block arguments differ from the function type");
          if (f.front().empty() || f.front().back().getKind() != OpKind::Return) return fail(op, "function body must end with return");
          Operation& ret = f.front().back();
          if (ret.getNumOperands() != f.getFunctionType().getNumResults()) return fail(op, "return arity differs from the function type");
          for (unsigned i = 0; i < ret.getNumOperands(); ++i)
            if (ret.getOperand(i).getType() != f.getFunctionType().getResult(i)) return fail(op, "return type differs from the function type");
        }
        break;
      }
      default: break;
    }
    for (unsigned r = 0; r < op->getNumRegions(); ++r)
      for (auto& b : op->getRegion(r).getBlocks())
        for (auto& inner : b->getOperations()) {
          if (inner.getBlock() != b.get()) return fail(&inner, "operation's block pointer is stale");
          if (!visit(&inner)) return false;
        }
    return true;
  }
};
}  // namespace

LogicalResult verify(Operation* op, std::string* message) {
  Verifier v;
  if (v.visit(op)) return success();
  if (message) *message = v.msg;
  else std::cerr << "verification failed: " << v.msg << "\n";
  return failure();
}

}  // namespace mlir
