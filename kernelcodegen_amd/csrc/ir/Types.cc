// Types, affine expressions / maps / sets and attributes of the mini affine IR.
#include <cmath>
#include <cstring>
#include <deque>
#include <mutex>

#include "IR/MLIR.h"

namespace mlir {

MLIRContext* getGlobalContext() {
  static MLIRContext ctx;
  return &ctx;
}

// ---------------------------------------------------------------------------
// Type uniquing
// ---------------------------------------------------------------------------
namespace {
std::mutex& internMutex() { static std::mutex m; return m; }

struct TypeKey {
  int kind; unsigned width; std::vector<int64_t> shape; const void* element; int memorySpace;
  std::vector<const void*> inputs, results;
  bool operator<(const TypeKey& o) const {
    return std::tie(kind, width, shape, element, memorySpace, inputs, results) <
           std::tie(o.kind, o.width, o.shape, o.element, o.memorySpace, o.inputs, o.results);
  }
};

const detail::TypeStorage* internType(const detail::TypeStorage& proto) {
  static std::map<TypeKey, std::unique_ptr<detail::TypeStorage>> table;
  TypeKey key{(int)proto.kind, proto.width, proto.shape, proto.element, proto.memorySpace, {}, {}};
  for (auto p : proto.inputs) key.inputs.push_back(p);
  for (auto p : proto.results) key.results.push_back(p);
  std::lock_guard<std::mutex> lock(internMutex());
  auto& slot = table[key];
  if (!slot) slot = std::make_unique<detail::TypeStorage>(proto);
  return slot.get();
}

const detail::TypeStorage* simpleType(detail::TypeStorage::Kind k) {
  detail::TypeStorage p;
  p.kind = k;
  return internType(p);
}
}  // namespace

#define KCG_SIMPLE_GET(NAME, KIND) \
  NAME NAME::get(MLIRContext*) { return NAME(simpleType(detail::TypeStorage::KIND)); }
KCG_SIMPLE_GET(Float16Type, F16)
KCG_SIMPLE_GET(BFloat16Type, BF16)
KCG_SIMPLE_GET(Float32Type, F32)
KCG_SIMPLE_GET(Float64Type, F64)
KCG_SIMPLE_GET(Float8E4M3FNType, F8E4M3FN)
KCG_SIMPLE_GET(IndexType, Index)
#undef KCG_SIMPLE_GET

IntegerType IntegerType::get(MLIRContext*, unsigned width) {
  detail::TypeStorage p;
  p.kind = detail::TypeStorage::Integer;
  p.width = width;
  return IntegerType(internType(p));
}

MemRefType MemRefType::get(ArrayRef<int64_t> shape, Type elementType, LayoutPlaceholder, int memorySpace) {
  assert(elementType && "memref needs an element type");
  detail::TypeStorage p;
  p.kind = detail::TypeStorage::MemRef;
  p.shape = shape.vec();
  p.element = elementType.getImpl();
  p.memorySpace = memorySpace;
  return MemRefType(internType(p));
}

VectorType VectorType::get(ArrayRef<int64_t> shape, Type elementType) {
  detail::TypeStorage p;
  p.kind = detail::TypeStorage::Vector;
  p.shape = shape.vec();
  p.element = elementType.getImpl();
  return VectorType(internType(p));
}

FunctionType FunctionType::get(MLIRContext*, TypeRange inputs, TypeRange results) {
  detail::TypeStorage p;
  p.kind = detail::TypeStorage::Function;
  for (auto t : inputs) p.inputs.push_back(t.getImpl());
  for (auto t : results) p.results.push_back(t.getImpl());
  return FunctionType(internType(p));
}
std::vector<Type> FunctionType::getInputs() const {
  std::vector<Type> r;
  for (auto p : impl->inputs) r.push_back(Type(p));
  return r;
}
std::vector<Type> FunctionType::getResults() const {
  std::vector<Type> r;
  for (auto p : impl->results) r.push_back(Type(p));
  return r;
}

bool Type::isF16() const { return impl && impl->kind == detail::TypeStorage::F16; }
bool Type::isBF16() const { return impl && impl->kind == detail::TypeStorage::BF16; }
bool Type::isF32() const { return impl && impl->kind == detail::TypeStorage::F32; }
bool Type::isF64() const { return impl && impl->kind == detail::TypeStorage::F64; }
bool Type::isIndex() const { return impl && impl->kind == detail::TypeStorage::Index; }
bool Type::isFloat() const {
  if (!impl) return false;
  switch (impl->kind) {
    case detail::TypeStorage::F16: case detail::TypeStorage::BF16: case detail::TypeStorage::F32:
    case detail::TypeStorage::F64: case detail::TypeStorage::F8E4M3FN: return true;
    default: return false;
  }
}
bool Type::isIntOrIndex() const {
  return impl && (impl->kind == detail::TypeStorage::Integer || impl->kind == detail::TypeStorage::Index);
}
unsigned Type::getIntOrFloatBitWidth() const {
  switch (impl->kind) {
    case detail::TypeStorage::F16: case detail::TypeStorage::BF16: return 16;
    case detail::TypeStorage::F32: return 32;
    case detail::TypeStorage::F64: return 64;
    case detail::TypeStorage::F8E4M3FN: return 8;
    case detail::TypeStorage::Integer: return impl->width;
    case detail::TypeStorage::Index: return 64;
    default: assert(false && "not an int or float type"); return 0;
  }
}

void Type::print(std::ostream& os) const {
  if (!impl) { os << "<<null type>>"; return; }
  switch (impl->kind) {
    case detail::TypeStorage::F16: os << "f16"; break;
    case detail::TypeStorage::BF16: os << "bf16"; break;
    case detail::TypeStorage::F32: os << "f32"; break;
    case detail::TypeStorage::F64: os << "f64"; break;
    case detail::TypeStorage::F8E4M3FN: os << "f8E4M3FN"; break;
    case detail::TypeStorage::Index: os << "index"; break;
    case detail::TypeStorage::Integer: os << "i" << impl->width; break;
    case detail::TypeStorage::MemRef:
      os << "memref<";
      for (auto d : impl->shape) os << d << "x";
      Type(impl->element).print(os);
      if (impl->memorySpace) os << ", " << impl->memorySpace;
      os << ">";
      break;
    case detail::TypeStorage::Vector:
      os << "vector<";
      for (auto d : impl->shape) os << d << "x";
      Type(impl->element).print(os);
      os << ">";
      break;
    case detail::TypeStorage::Function: {
      os << "(";
      for (size_t i = 0; i < impl->inputs.size(); ++i) { if (i) os << ", "; Type(impl->inputs[i]).print(os); }
      os << ") -> ";
      if (impl->results.size() == 1) Type(impl->results[0]).print(os);
      else {
        os << "(";
        for (size_t i = 0; i < impl->results.size(); ++i) { if (i) os << ", "; Type(impl->results[i]).print(os); }
        os << ")";
      }
      break;
    }
  }
}
void Type::dump() const { print(std::cerr); std::cerr << "\n"; }

// ---------------------------------------------------------------------------
// Affine expressions
// ---------------------------------------------------------------------------
namespace {
struct ExprKey {
  int kind; const void* lhs; const void* rhs; int64_t value;
  bool operator<(const ExprKey& o) const { return std::tie(kind, lhs, rhs, value) < std::tie(o.kind, o.lhs, o.rhs, o.value); }
};
AffineExpr internExpr(AffineExprKind kind, const detail::AffineExprStorage* lhs, const detail::AffineExprStorage* rhs,
                      int64_t value) {
  static std::map<ExprKey, std::unique_ptr<detail::AffineExprStorage>> table;
  ExprKey key{(int)kind, lhs, rhs, value};
  std::lock_guard<std::mutex> lock(internMutex());
  auto& slot = table[key];
  if (!slot) {
    slot = std::make_unique<detail::AffineExprStorage>();
    slot->kind = kind; slot->lhs = lhs; slot->rhs = rhs; slot->value = value;
  }
  return AffineExpr(slot.get());
}
int64_t floorDivI(int64_t a, int64_t b) { int64_t q = a / b, r = a % b; return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q; }
int64_t ceilDivI(int64_t a, int64_t b) { return -floorDivI(-a, b); }
int64_t modI(int64_t a, int64_t b) { int64_t r = a % b; return r < 0 ? r + (b < 0 ? -b : b) : r; }
bool isConst(AffineExpr e, int64_t* v = nullptr) {
  if (e.getKind() != AffineExprKind::Constant) return false;
  if (v) *v = e.getImpl()->value;
  return true;
}
}  // namespace

AffineExpr getAffineDimExpr(unsigned position, MLIRContext*) { return internExpr(AffineExprKind::DimId, nullptr, nullptr, position); }
AffineExpr getAffineSymbolExpr(unsigned position, MLIRContext*) { return internExpr(AffineExprKind::SymbolId, nullptr, nullptr, position); }
AffineExpr getAffineConstantExpr(int64_t constant, MLIRContext*) { return internExpr(AffineExprKind::Constant, nullptr, nullptr, constant); }

// Light simplification on construction: constant folding, neutral elements and
// constants moved to the right of + and *.  Everything else is kept as written.
AffineExpr getAffineBinaryOpExpr(AffineExprKind kind, AffineExpr lhs, AffineExpr rhs) {
  int64_t a, b;
  const bool ca = isConst(lhs, &a), cb = isConst(rhs, &b);
  switch (kind) {
    case AffineExprKind::Add:
      if (ca && cb) return getAffineConstantExpr(a + b);
      if (ca) { std::swap(lhs, rhs); b = a; }
      if ((ca || cb) && b == 0) return lhs;
      // (x + c1) + c2 -> x + (c1 + c2)
      if ((ca || cb) && lhs.getKind() == AffineExprKind::Add) {
        int64_t c1;
        if (isConst(AffineExpr(lhs.getImpl()->rhs), &c1))
          return getAffineBinaryOpExpr(AffineExprKind::Add, AffineExpr(lhs.getImpl()->lhs), getAffineConstantExpr(c1 + b));
      }
      break;
    case AffineExprKind::Mul:
      if (ca && cb) return getAffineConstantExpr(a * b);
      if (ca) { std::swap(lhs, rhs); b = a; }
      if (ca || cb) {
        if (b == 0) return getAffineConstantExpr(0);
        if (b == 1) return lhs;
      }
      break;
    case AffineExprKind::FloorDiv:
      assert(!(cb && b == 0) && "division by zero in affine expression");
      if (ca && cb) return getAffineConstantExpr(floorDivI(a, b));
      if (cb && b == 1) return lhs;
      break;
    case AffineExprKind::CeilDiv:
      assert(!(cb && b == 0) && "division by zero in affine expression");
      if (ca && cb) return getAffineConstantExpr(ceilDivI(a, b));
      if (cb && b == 1) return lhs;
      break;
    case AffineExprKind::Mod:
      assert(!(cb && b <= 0) && "modulo by a non-positive constant in affine expression");
      if (ca && cb) return getAffineConstantExpr(modI(a, b));
      if (cb && b == 1) return getAffineConstantExpr(0);
      break;
    default: assert(false && "not a binary affine expression kind");
  }
  return internExpr(kind, lhs.getImpl(), rhs.getImpl(), 0);
}

bool AffineExpr::operator==(int64_t v) const { int64_t c; return isConst(*this, &c) && c == v; }
AffineExpr AffineExpr::operator+(int64_t v) const { return *this + getAffineConstantExpr(v); }
AffineExpr AffineExpr::operator+(AffineExpr o) const { return getAffineBinaryOpExpr(AffineExprKind::Add, *this, o); }
AffineExpr AffineExpr::operator-() const { return *this * -1; }
AffineExpr AffineExpr::operator-(int64_t v) const { return *this + (-v); }
AffineExpr AffineExpr::operator-(AffineExpr o) const { return *this + (-o); }
AffineExpr AffineExpr::operator*(int64_t v) const { return *this * getAffineConstantExpr(v); }
AffineExpr AffineExpr::operator*(AffineExpr o) const { return getAffineBinaryOpExpr(AffineExprKind::Mul, *this, o); }
AffineExpr AffineExpr::floorDiv(uint64_t v) const { return floorDiv(getAffineConstantExpr((int64_t)v)); }
AffineExpr AffineExpr::floorDiv(AffineExpr o) const { return getAffineBinaryOpExpr(AffineExprKind::FloorDiv, *this, o); }
AffineExpr AffineExpr::ceilDiv(uint64_t v) const { return ceilDiv(getAffineConstantExpr((int64_t)v)); }
AffineExpr AffineExpr::ceilDiv(AffineExpr o) const { return getAffineBinaryOpExpr(AffineExprKind::CeilDiv, *this, o); }
AffineExpr AffineExpr::operator%(uint64_t v) const { return *this % getAffineConstantExpr((int64_t)v); }
AffineExpr AffineExpr::operator%(AffineExpr o) const { return getAffineBinaryOpExpr(AffineExprKind::Mod, *this, o); }

bool AffineExpr::isSymbolicOrConstant() const {
  switch (getKind()) {
    case AffineExprKind::Constant: case AffineExprKind::SymbolId: return true;
    case AffineExprKind::DimId: return false;
    default: return AffineExpr(expr->lhs).isSymbolicOrConstant() && AffineExpr(expr->rhs).isSymbolicOrConstant();
  }
}
bool AffineExpr::isFunctionOfDim(unsigned position) const {
  switch (getKind()) {
    case AffineExprKind::DimId: return (unsigned)expr->value == position;
    case AffineExprKind::Constant: case AffineExprKind::SymbolId: return false;
    default: return AffineExpr(expr->lhs).isFunctionOfDim(position) || AffineExpr(expr->rhs).isFunctionOfDim(position);
  }
}

AffineExpr AffineExpr::replaceDimsAndSymbols(ArrayRef<AffineExpr> dimRepl, ArrayRef<AffineExpr> symRepl) const {
  switch (getKind()) {
    case AffineExprKind::Constant: return *this;
    case AffineExprKind::DimId: return (size_t)expr->value < dimRepl.size() ? dimRepl[expr->value] : *this;
    case AffineExprKind::SymbolId: return (size_t)expr->value < symRepl.size() ? symRepl[expr->value] : *this;
    default:
      return getAffineBinaryOpExpr(getKind(), AffineExpr(expr->lhs).replaceDimsAndSymbols(dimRepl, symRepl),
                                   AffineExpr(expr->rhs).replaceDimsAndSymbols(dimRepl, symRepl));
  }
}

AffineExpr AffineExpr::shiftDims(unsigned numDims, unsigned shift, unsigned offset) const {
  SmallVector<AffineExpr> dims;
  for (unsigned i = 0; i < offset; ++i) dims.push_back(getAffineDimExpr(i));
  for (unsigned i = offset; i < numDims; ++i) dims.push_back(getAffineDimExpr(i + shift));
  return replaceDimsAndSymbols(dims, {});
}

int64_t AffineExpr::evaluate(ArrayRef<int64_t> dims, ArrayRef<int64_t> syms) const {
  switch (getKind()) {
    case AffineExprKind::Constant: return expr->value;
    case AffineExprKind::DimId: assert((size_t)expr->value < dims.size()); return dims[expr->value];
    case AffineExprKind::SymbolId: assert((size_t)expr->value < syms.size()); return syms[expr->value];
    default: break;
  }
  const int64_t a = AffineExpr(expr->lhs).evaluate(dims, syms), b = AffineExpr(expr->rhs).evaluate(dims, syms);
  switch (getKind()) {
    case AffineExprKind::Add: return a + b;
    case AffineExprKind::Mul: return a * b;
    case AffineExprKind::FloorDiv: return floorDivI(a, b);
    case AffineExprKind::CeilDiv: return ceilDivI(a, b);
    case AffineExprKind::Mod: return modI(a, b);
    default: assert(false); return 0;
  }
}

void AffineExpr::walk(const std::function<void(AffineExpr)>& fn) const {
  if (getKind() <= AffineExprKind::LAST_AFFINE_BINARY_OP) {
    AffineExpr(expr->lhs).walk(fn);
    AffineExpr(expr->rhs).walk(fn);
  }
  fn(*this);
}

namespace {
void printExpr(std::ostream& os, AffineExpr e, bool paren) {
  switch (e.getKind()) {
    case AffineExprKind::Constant: os << e.getImpl()->value; return;
    case AffineExprKind::DimId: os << "d" << e.getImpl()->value; return;
    case AffineExprKind::SymbolId: os << "s" << e.getImpl()->value; return;
    default: break;
  }
  AffineExpr l(e.getImpl()->lhs), r(e.getImpl()->rhs);
  int64_t c;
  if (paren) os << "(";
  if (e.getKind() == AffineExprKind::Add) {
    printExpr(os, l, false);
    // x + (y * -1) prints as x - y, x + (-c) as x - c
    if (isConst(r, &c) && c < 0) os << " - " << -c;
    else if (r.getKind() == AffineExprKind::Mul && isConst(AffineExpr(r.getImpl()->rhs), &c) && c == -1) {
      os << " - "; printExpr(os, AffineExpr(r.getImpl()->lhs), true);
    } else { os << " + "; printExpr(os, r, false); }
  } else {
    const char* sym = e.getKind() == AffineExprKind::Mul ? " * " : e.getKind() == AffineExprKind::Mod ? " mod "
                    : e.getKind() == AffineExprKind::FloorDiv ? " floordiv " : " ceildiv ";
    if (e.getKind() == AffineExprKind::Mul && isConst(r, &c) && c == -1) { os << "-"; printExpr(os, l, true); }
    else { printExpr(os, l, true); os << sym; printExpr(os, r, true); }
  }
  if (paren) os << ")";
}
}  // namespace
void AffineExpr::print(std::ostream& os) const { if (!expr) os << "<<null expr>>"; else printExpr(os, *this, false); }
void AffineExpr::dump() const { print(std::cerr); std::cerr << "\n"; }

// ---------------------------------------------------------------------------
// Affine maps and integer sets
// ---------------------------------------------------------------------------
AffineMap AffineMap::get(unsigned dimCount, unsigned symbolCount, ArrayRef<AffineExpr> results, MLIRContext*) {
  static std::deque<detail::AffineMapStorage> table;
  std::lock_guard<std::mutex> lock(internMutex());
  for (auto& m : table)
    if (m.numDims == dimCount && m.numSymbols == symbolCount && ArrayRef<AffineExpr>(m.results) == results)
      return AffineMap(&m);
  table.emplace_back();
  table.back().numDims = dimCount;
  table.back().numSymbols = symbolCount;
  table.back().results = results.vec();
  return AffineMap(&table.back());
}
AffineMap AffineMap::get(unsigned dimCount, unsigned symbolCount, AffineExpr result) {
  return get(dimCount, symbolCount, ArrayRef<AffineExpr>(result));
}
AffineMap AffineMap::get(unsigned dimCount, unsigned symbolCount, MLIRContext*) {
  return get(dimCount, symbolCount, ArrayRef<AffineExpr>());
}
AffineMap AffineMap::getConstantMap(int64_t val, MLIRContext*) { return get(0, 0, getAffineConstantExpr(val)); }
AffineMap AffineMap::getMultiDimIdentityMap(unsigned numDims, MLIRContext*) {
  SmallVector<AffineExpr> e;
  for (unsigned i = 0; i < numDims; ++i) e.push_back(getAffineDimExpr(i));
  return get(numDims, 0, ArrayRef<AffineExpr>(e));
}
bool AffineMap::isConstant() const {
  for (auto e : map->results) if (e.getKind() != AffineExprKind::Constant) return false;
  return true;
}
int64_t AffineMap::getSingleConstantResult() const {
  assert(isSingleConstant() && "map must have a single constant result");
  return map->results[0].getImpl()->value;
}
SmallVector<int64_t> AffineMap::getConstantResults() const {
  SmallVector<int64_t> r;
  for (auto e : map->results) { assert(e.getKind() == AffineExprKind::Constant); r.push_back(e.getImpl()->value); }
  return r;
}
bool AffineMap::isIdentity() const {
  if (getNumDims() != getNumResults()) return false;
  for (unsigned i = 0; i < getNumResults(); ++i)
    if (map->results[i] != getAffineDimExpr(i)) return false;
  return true;
}
AffineMap AffineMap::replaceDimsAndSymbols(ArrayRef<AffineExpr> dimRepl, ArrayRef<AffineExpr> symRepl, unsigned nd,
                                           unsigned ns) const {
  SmallVector<AffineExpr> r;
  for (auto e : map->results) r.push_back(e.replaceDimsAndSymbols(dimRepl, symRepl));
  return get(nd, ns, ArrayRef<AffineExpr>(r));
}
SmallVector<int64_t> AffineMap::evaluate(ArrayRef<int64_t> inputs) const {
  assert(inputs.size() == getNumInputs() && "wrong number of map inputs");
  ArrayRef<int64_t> dims(inputs.data(), map->numDims), syms(inputs.data() + map->numDims, map->numSymbols);
  SmallVector<int64_t> r;
  for (auto e : map->results) r.push_back(e.evaluate(dims, syms));
  return r;
}
namespace {
void printDimsAndSymbols(std::ostream& os, unsigned nd, unsigned ns) {
  os << "(";
  for (unsigned i = 0; i < nd; ++i) os << (i ? ", d" : "d") << i;
  os << ")";
  if (ns) {
    os << "[";
    for (unsigned i = 0; i < ns; ++i) os << (i ? ", s" : "s") << i;
    os << "]";
  }
}
}  // namespace
void AffineMap::print(std::ostream& os) const {
  if (!map) { os << "<<null map>>"; return; }
  printDimsAndSymbols(os, map->numDims, map->numSymbols);
  os << " -> (";
  for (size_t i = 0; i < map->results.size(); ++i) { if (i) os << ", "; map->results[i].print(os); }
  os << ")";
}
void AffineMap::dump() const { print(std::cerr); std::cerr << "\n"; }

IntegerSet IntegerSet::get(unsigned dimCount, unsigned symbolCount, ArrayRef<AffineExpr> constraints, ArrayRef<bool> eqFlags) {
  assert(constraints.size() == eqFlags.size());
  static std::deque<detail::IntegerSetStorage> table;
  std::lock_guard<std::mutex> lock(internMutex());
  std::vector<bool> flags(eqFlags.begin(), eqFlags.end());
  for (auto& s : table)
    if (s.numDims == dimCount && s.numSymbols == symbolCount && ArrayRef<AffineExpr>(s.constraints) == constraints &&
        s.eqFlags == flags)
      return IntegerSet(&s);
  table.emplace_back();
  table.back().numDims = dimCount;
  table.back().numSymbols = symbolCount;
  table.back().constraints = constraints.vec();
  table.back().eqFlags = flags;
  return IntegerSet(&table.back());
}
bool IntegerSet::contains(ArrayRef<int64_t> inputs) const {
  ArrayRef<int64_t> dims(inputs.data(), set->numDims), syms(inputs.data() + set->numDims, set->numSymbols);
  for (size_t i = 0; i < set->constraints.size(); ++i) {
    const int64_t v = set->constraints[i].evaluate(dims, syms);
    if (set->eqFlags[i] ? v != 0 : v < 0) return false;
  }
  return true;
}
void IntegerSet::print(std::ostream& os) const {
  printDimsAndSymbols(os, set->numDims, set->numSymbols);
  os << " : (";
  for (size_t i = 0; i < set->constraints.size(); ++i) {
    if (i) os << ", ";
    set->constraints[i].print(os);
    os << (set->eqFlags[i] ? " == 0" : " >= 0");
  }
  os << ")";
}

// ---------------------------------------------------------------------------
// Attributes
// ---------------------------------------------------------------------------
bool Attribute::operator==(const Attribute& o) const {
  return kind == o.kind && s == o.s && i == o.i && f == o.f && type == o.type && map == o.map && set == o.set && ints == o.ints;
}

namespace {
float roundToBF16(float v) {
  uint32_t u; memcpy(&u, &v, 4);
  if ((u & 0x7F800000u) == 0x7F800000u) return v;
  u += 0x7FFFu + ((u >> 16) & 1u);
  u &= 0xFFFF0000u;
  memcpy(&v, &u, 4);
  return v;
}
// Nearest binary16 value (ties to even), returned as a float; overflow gives infinity.
float roundToF16(float v) {
  if (!std::isfinite(v) || v == 0.0f) return v;
  int e;
  (void)std::frexp(v, &e);              // v = f * 2^e, f in [0.5, 1)
  int ulpExp = (e - 1 < -14 ? -14 : e - 1) - 10;
  float q = std::nearbyint(std::ldexp(v, -ulpExp));
  float r = std::ldexp(q, ulpExp);
  return std::fabs(r) > 65504.0f ? std::copysign(INFINITY, v) : r;
}
}  // namespace

FloatAttr FloatAttr::get(Type t, double v) {
  FloatAttr a;
  a.kind = Float;
  a.type = t;
  if (t.isF32()) a.f = (double)(float)v;          // the value the element type can hold
  else if (t.isBF16()) a.f = (double)roundToBF16((float)v);
  else if (t.isF16()) a.f = (double)roundToF16((float)v);
  else a.f = v;
  return a;
}

Attribute getIntArrayAttr(ArrayRef<int64_t> v) {
  Attribute a;
  a.kind = Attribute::IntArray;
  a.ints = v.vec();
  return a;
}

void Attribute::print(std::ostream& os) const {
  switch (kind) {
    case None: os << "<<null attr>>"; break;
    case String: os << '"' << s << '"'; break;
    case Integer:
      os << i;
      if (type && !type.isIndex() && !(type.isa<IntegerType>() && type.getIntOrFloatBitWidth() == 64)) { os << " : "; type.print(os); }
      else if (type) { os << " : "; type.print(os); }
      break;
    case Float: {
      char buf[64];
      // MLIR prints the shortest scientific form that round-trips
      if (type.isF32() || type.isBF16() || type.isF16()) snprintf(buf, sizeof buf, "%.6e", f);
      else snprintf(buf, sizeof buf, "%.15e", f);
      if (type.isF32()) { float back = strtof(buf, nullptr); if (back != (float)f) snprintf(buf, sizeof buf, "%.9g", f); }
      os << buf << " : ";
      type.print(os);
      break;
    }
    case Map: os << "affine_map<"; map.print(os); os << ">"; break;
    case Set: os << "affine_set<"; set.print(os); os << ">"; break;
    case TypeKind: type.print(os); break;
    case Unit: os << "unit"; break;
    case IntArray:
      os << "[";
      for (size_t k = 0; k < ints.size(); ++k) os << (k ? ", " : "") << ints[k];
      os << "]";
      break;
  }
}

}  // namespace mlir
