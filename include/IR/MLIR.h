// A small, self-contained affine IR that provides, under the namespace `mlir`,
// the subset of the MLIR 15 C++ API that KernelCodeGen's public headers and
// passes use (the reference's include/IR/MLIR.h is an umbrella include of the
// external LLVM/MLIR tree; this build has no such dependency).
//
// Provided: builtin types (f16/bf16/f32/f64/f8E4M3FN, iN, index, memref,
// vector, function), affine expressions / maps / integer sets, SSA values with
// use lists, operations with regions, the ops of the func, memref, affine,
// arith, math and gpu dialects that the Frontend and the Optimizer create,
// OpBuilder, cloning with a value mapping, walks, a verifier and a textual
// printer in MLIR's syntax.
#pragma once

#include <map>
#include <memory>
#include <set>
#include <unordered_map>

#include "IR/Support.h"

namespace mlir {

using llvm::ArrayRef;
using llvm::SmallVector;
using llvm::StringRef;
using llvm::function_ref;
template <typename T>
using Optional = std::optional<T>;

class Operation;
class Block;
class Region;
class OpBuilder;
class Value;
class AffineMap;
class IntegerSet;

// ---------------------------------------------------------------------------
// Context, location, dialect tags
// ---------------------------------------------------------------------------
class MLIRContext {
public:
  template <typename Dialect>
  Dialect* getOrLoadDialect() { return nullptr; }  // every dialect below is always available
};
MLIRContext* getGlobalContext();

struct Location {};
struct UnknownLoc : Location {};

class AffineDialect {};
namespace memref { class MemRefDialect {}; }
namespace func { class FuncDialect {}; }
namespace arith { class ArithmeticDialect {}; }
namespace gpu { class GPUDialect {}; }
namespace vector { class VectorDialect {}; }
namespace scf { class SCFDialect {}; }
namespace math { class MathDialect {}; }
inline void registerAllPasses() {}

struct LogicalResult {
  bool ok;
  static LogicalResult success() { return {true}; }
  static LogicalResult failure() { return {false}; }
};
inline bool failed(LogicalResult r) { return !r.ok; }
inline bool succeeded(LogicalResult r) { return r.ok; }
inline LogicalResult success() { return LogicalResult::success(); }
inline LogicalResult failure() { return LogicalResult::failure(); }

// ---------------------------------------------------------------------------
// Types (interned; equality is pointer equality)
// ---------------------------------------------------------------------------
namespace detail {
struct TypeStorage {
  enum Kind { F16, BF16, F32, F64, F8E4M3FN, Integer, Index, MemRef, Vector, Function };
  Kind kind;
  unsigned width = 0;                       // Integer
  std::vector<int64_t> shape;               // MemRef, Vector
  const TypeStorage* element = nullptr;     // MemRef, Vector
  int memorySpace = 0;                      // MemRef
  std::vector<const TypeStorage*> inputs;   // Function
  std::vector<const TypeStorage*> results;  // Function
};
}  // namespace detail

class Type {
public:
  Type() = default;
  Type(std::nullptr_t) {}
  explicit Type(const detail::TypeStorage* impl) : impl(impl) {}
  explicit operator bool() const { return impl != nullptr; }
  bool operator==(Type o) const { return impl == o.impl; }
  bool operator!=(Type o) const { return impl != o.impl; }
  bool operator<(Type o) const { return impl < o.impl; }
  template <typename U> bool isa() const { return impl && U::classof(*this); }
  template <typename U> U dyn_cast() const { return isa<U>() ? U(impl) : U(); }
  template <typename U> U cast() const { assert(isa<U>()); return U(impl); }
  bool isF16() const;
  bool isBF16() const;
  bool isF32() const;
  bool isF64() const;
  bool isIndex() const;
  bool isFloat() const;        // any float kind, including the 8-bit one
  bool isIntOrIndex() const;
  unsigned getIntOrFloatBitWidth() const;
  void print(std::ostream& os) const;
  void dump() const;
  const detail::TypeStorage* getImpl() const { return impl; }

protected:
  const detail::TypeStorage* impl = nullptr;
};
inline std::ostream& operator<<(std::ostream& os, Type t) { t.print(os); return os; }

#define KCG_SIMPLE_TYPE(NAME, KIND)                                                        \
  class NAME : public Type {                                                               \
  public:                                                                                  \
    using Type::Type;                                                                      \
    NAME() = default;                                                                      \
    static bool classof(Type t) { return t.getImpl()->kind == detail::TypeStorage::KIND; } \
    static NAME get(MLIRContext* = nullptr);                                               \
  };
KCG_SIMPLE_TYPE(Float16Type, F16)
KCG_SIMPLE_TYPE(BFloat16Type, BF16)
KCG_SIMPLE_TYPE(Float32Type, F32)
KCG_SIMPLE_TYPE(Float64Type, F64)
KCG_SIMPLE_TYPE(Float8E4M3FNType, F8E4M3FN)
KCG_SIMPLE_TYPE(IndexType, Index)
#undef KCG_SIMPLE_TYPE

class FloatType : public Type {
public:
  using Type::Type;
  FloatType() = default;
  static bool classof(Type t) { return t.isFloat(); }
  unsigned getWidth() const { return getIntOrFloatBitWidth(); }
};

class IntegerType : public Type {
public:
  using Type::Type;
  IntegerType() = default;
  static bool classof(Type t) { return t.getImpl()->kind == detail::TypeStorage::Integer; }
  static IntegerType get(MLIRContext*, unsigned width);
  unsigned getWidth() const { return impl->width; }
};

class ShapedType : public Type {
public:
  using Type::Type;
  ShapedType() = default;
  static bool classof(Type t) {
    return t.getImpl()->kind == detail::TypeStorage::MemRef || t.getImpl()->kind == detail::TypeStorage::Vector;
  }
  ArrayRef<int64_t> getShape() const { return impl->shape; }
  Type getElementType() const { return Type(impl->element); }
  int64_t getRank() const { return (int64_t)impl->shape.size(); }
  int64_t getNumElements() const { int64_t n = 1; for (auto d : impl->shape) n *= d; return n; }
  int64_t getDimSize(unsigned i) const { return impl->shape[i]; }
};

// The memory space is kept as the integer the reference passes
// (KernelCodeGen::MemorySpace: global = 1, shared = 2, local = 3).
struct MemorySpaceAttr {
  int value = 0;
  bool operator==(const MemorySpaceAttr& o) const { return value == o.value; }
};

class MemRefType : public ShapedType {
public:
  using ShapedType::ShapedType;
  MemRefType() = default;
  static bool classof(Type t) { return t.getImpl()->kind == detail::TypeStorage::MemRef; }
  struct LayoutPlaceholder { LayoutPlaceholder() = default; };
  static MemRefType get(ArrayRef<int64_t> shape, Type elementType, LayoutPlaceholder = {}, int memorySpace = 0);
  unsigned getMemorySpaceAsInt() const { return (unsigned)impl->memorySpace; }
  MemorySpaceAttr getMemorySpace() const { return {impl->memorySpace}; }
};

class VectorType : public ShapedType {
public:
  using ShapedType::ShapedType;
  VectorType() = default;
  static bool classof(Type t) { return t.getImpl()->kind == detail::TypeStorage::Vector; }
  static VectorType get(ArrayRef<int64_t> shape, Type elementType);
  static VectorType get(int64_t n, Type elementType) { return get(ArrayRef<int64_t>(n), elementType); }
};

class TypeRange : public std::vector<Type> {
public:
  using std::vector<Type>::vector;
  TypeRange() = default;
  TypeRange(const std::vector<Type>& v) : std::vector<Type>(v) {}
  TypeRange(ArrayRef<Type> a) : std::vector<Type>(a.begin(), a.end()) {}
  TypeRange(Type t) : std::vector<Type>(1, t) {}
};

class FunctionType : public Type {
public:
  using Type::Type;
  FunctionType() = default;
  static bool classof(Type t) { return t.getImpl()->kind == detail::TypeStorage::Function; }
  static FunctionType get(MLIRContext*, TypeRange inputs, TypeRange results);
  std::vector<Type> getInputs() const;
  std::vector<Type> getResults() const;
  unsigned getNumInputs() const { return (unsigned)impl->inputs.size(); }
  unsigned getNumResults() const { return (unsigned)impl->results.size(); }
  Type getInput(unsigned i) const { return Type(impl->inputs[i]); }
  Type getResult(unsigned i) const { return Type(impl->results[i]); }
};

// ---------------------------------------------------------------------------
// Affine expressions, maps and integer sets (interned, immutable)
// ---------------------------------------------------------------------------
enum class AffineExprKind { Add, Mul, Mod, FloorDiv, CeilDiv, LAST_AFFINE_BINARY_OP = CeilDiv, Constant, DimId, SymbolId };

namespace detail {
struct AffineExprStorage {
  AffineExprKind kind;
  const AffineExprStorage* lhs = nullptr;
  const AffineExprStorage* rhs = nullptr;
  int64_t value = 0;  // constant value, or dim / symbol position
};
}  // namespace detail

class AffineExpr {
public:
  AffineExpr() = default;
  explicit AffineExpr(const detail::AffineExprStorage* e) : expr(e) {}
  explicit operator bool() const { return expr != nullptr; }
  bool operator==(AffineExpr o) const { return expr == o.expr; }
  bool operator!=(AffineExpr o) const { return expr != o.expr; }
  bool operator==(int64_t v) const;
  AffineExprKind getKind() const { return expr->kind; }
  MLIRContext* getContext() const { return getGlobalContext(); }
  template <typename U> bool isa() const { return expr && U::classof(*this); }
  template <typename U> U dyn_cast() const { return isa<U>() ? U(expr) : U(); }
  template <typename U> U cast() const { assert(isa<U>()); return U(expr); }
  bool isSymbolicOrConstant() const;
  bool isPureAffine() const { return true; }
  bool isFunctionOfDim(unsigned position) const;
  AffineExpr operator+(int64_t v) const;
  AffineExpr operator+(AffineExpr other) const;
  AffineExpr operator-() const;
  AffineExpr operator-(int64_t v) const;
  AffineExpr operator-(AffineExpr other) const;
  AffineExpr operator*(int64_t v) const;
  AffineExpr operator*(AffineExpr other) const;
  AffineExpr floorDiv(uint64_t v) const;
  AffineExpr floorDiv(AffineExpr other) const;
  AffineExpr ceilDiv(uint64_t v) const;
  AffineExpr ceilDiv(AffineExpr other) const;
  AffineExpr operator%(uint64_t v) const;
  AffineExpr operator%(AffineExpr other) const;
  // d_i -> dimReplacements[i], s_i -> symReplacements[i]
  AffineExpr replaceDimsAndSymbols(ArrayRef<AffineExpr> dimReplacements, ArrayRef<AffineExpr> symReplacements = {}) const;
  AffineExpr replaceDims(ArrayRef<AffineExpr> dimReplacements) const { return replaceDimsAndSymbols(dimReplacements, {}); }
  AffineExpr shiftDims(unsigned numDims, unsigned shift, unsigned offset = 0) const;
  // Value at the given dim / symbol assignment; floordiv and mod follow the
  // mathematical (floor) definition.
  int64_t evaluate(ArrayRef<int64_t> dims, ArrayRef<int64_t> syms = {}) const;
  void walk(const std::function<void(AffineExpr)>& fn) const;
  void print(std::ostream& os) const;
  void dump() const;
  const detail::AffineExprStorage* getImpl() const { return expr; }

protected:
  const detail::AffineExprStorage* expr = nullptr;
};
inline std::ostream& operator<<(std::ostream& os, AffineExpr e) { e.print(os); return os; }
inline AffineExpr operator+(int64_t v, AffineExpr e) { return e + v; }
inline AffineExpr operator*(int64_t v, AffineExpr e) { return e * v; }
inline AffineExpr operator-(int64_t v, AffineExpr e) { return (-e) + v; }

class AffineBinaryOpExpr : public AffineExpr {
public:
  using AffineExpr::AffineExpr;
  AffineBinaryOpExpr() = default;
  static bool classof(AffineExpr e) { return e.getKind() <= AffineExprKind::LAST_AFFINE_BINARY_OP; }
  AffineExpr getLHS() const { return AffineExpr(expr->lhs); }
  AffineExpr getRHS() const { return AffineExpr(expr->rhs); }
};
class AffineDimExpr : public AffineExpr {
public:
  using AffineExpr::AffineExpr;
  AffineDimExpr() = default;
  static bool classof(AffineExpr e) { return e.getKind() == AffineExprKind::DimId; }
  unsigned getPosition() const { return (unsigned)expr->value; }
};
class AffineSymbolExpr : public AffineExpr {
public:
  using AffineExpr::AffineExpr;
  AffineSymbolExpr() = default;
  static bool classof(AffineExpr e) { return e.getKind() == AffineExprKind::SymbolId; }
  unsigned getPosition() const { return (unsigned)expr->value; }
};
class AffineConstantExpr : public AffineExpr {
public:
  using AffineExpr::AffineExpr;
  AffineConstantExpr() = default;
  static bool classof(AffineExpr e) { return e.getKind() == AffineExprKind::Constant; }
  int64_t getValue() const { return expr->value; }
};

AffineExpr getAffineDimExpr(unsigned position, MLIRContext* ctx = nullptr);
AffineExpr getAffineSymbolExpr(unsigned position, MLIRContext* ctx = nullptr);
AffineExpr getAffineConstantExpr(int64_t constant, MLIRContext* ctx = nullptr);
AffineExpr getAffineBinaryOpExpr(AffineExprKind kind, AffineExpr lhs, AffineExpr rhs);

namespace detail {
struct AffineMapStorage {
  unsigned numDims = 0, numSymbols = 0;
  std::vector<AffineExpr> results;
};
struct IntegerSetStorage {
  unsigned numDims = 0, numSymbols = 0;
  std::vector<AffineExpr> constraints;
  std::vector<bool> eqFlags;
};
}  // namespace detail

class AffineMap {
public:
  AffineMap() = default;
  explicit AffineMap(const detail::AffineMapStorage* m) : map(m) {}
  static AffineMap get(unsigned dimCount, unsigned symbolCount, ArrayRef<AffineExpr> results, MLIRContext* ctx = nullptr);
  static AffineMap get(unsigned dimCount, unsigned symbolCount, AffineExpr result);
  static AffineMap get(unsigned dimCount, unsigned symbolCount, MLIRContext* ctx = nullptr);
  static AffineMap getConstantMap(int64_t val, MLIRContext* ctx = nullptr);
  static AffineMap getMultiDimIdentityMap(unsigned numDims, MLIRContext* ctx = nullptr);
  explicit operator bool() const { return map != nullptr; }
  bool operator==(AffineMap o) const { return map == o.map; }
  bool operator!=(AffineMap o) const { return map != o.map; }
  MLIRContext* getContext() const { return getGlobalContext(); }
  unsigned getNumDims() const { return map->numDims; }
  unsigned getNumSymbols() const { return map->numSymbols; }
  unsigned getNumInputs() const { return map->numDims + map->numSymbols; }
  unsigned getNumResults() const { return (unsigned)map->results.size(); }
  ArrayRef<AffineExpr> getResults() const { return map->results; }
  AffineExpr getResult(unsigned i) const { return map->results[i]; }
  bool isConstant() const;
  bool isSingleConstant() const { return getNumResults() == 1 && isConstant(); }
  int64_t getSingleConstantResult() const;
  SmallVector<int64_t> getConstantResults() const;
  bool isIdentity() const;
  AffineMap replaceDimsAndSymbols(ArrayRef<AffineExpr> dimReplacements, ArrayRef<AffineExpr> symReplacements,
                                  unsigned numResultDims, unsigned numResultSyms) const;
  SmallVector<int64_t> evaluate(ArrayRef<int64_t> inputs) const;  // dims then symbols
  void print(std::ostream& os) const;
  void dump() const;

private:
  const detail::AffineMapStorage* map = nullptr;
};
inline std::ostream& operator<<(std::ostream& os, AffineMap m) { m.print(os); return os; }

class IntegerSet {
public:
  IntegerSet() = default;
  explicit IntegerSet(const detail::IntegerSetStorage* s) : set(s) {}
  static IntegerSet get(unsigned dimCount, unsigned symbolCount, ArrayRef<AffineExpr> constraints, ArrayRef<bool> eqFlags);
  explicit operator bool() const { return set != nullptr; }
  bool operator==(IntegerSet o) const { return set == o.set; }
  unsigned getNumDims() const { return set->numDims; }
  unsigned getNumSymbols() const { return set->numSymbols; }
  unsigned getNumInputs() const { return set->numDims + set->numSymbols; }
  unsigned getNumConstraints() const { return (unsigned)set->constraints.size(); }
  ArrayRef<AffineExpr> getConstraints() const { return set->constraints; }
  AffineExpr getConstraint(unsigned i) const { return set->constraints[i]; }
  bool isEq(unsigned i) const { return set->eqFlags[i]; }
  SmallVector<bool> getEqFlags() const { return SmallVector<bool>(set->eqFlags.begin(), set->eqFlags.end()); }
  bool contains(ArrayRef<int64_t> inputs) const;
  void print(std::ostream& os) const;

private:
  const detail::IntegerSetStorage* set = nullptr;
};

// ---------------------------------------------------------------------------
// Attributes
// ---------------------------------------------------------------------------
class Attribute {
public:
  enum Kind { None, String, Integer, Float, Map, Set, TypeKind, Unit, IntArray };
  Attribute() = default;
  explicit operator bool() const { return kind != None; }
  bool operator==(const Attribute& o) const;
  Kind kind = None;
  std::string s;
  int64_t i = 0;
  double f = 0.0;
  Type type;
  AffineMap map;
  IntegerSet set;
  std::vector<int64_t> ints;
  template <typename U> bool isa() const { return kind != None && U::classof(*this); }
  template <typename U> U dyn_cast() const { return isa<U>() ? U(*this) : U(); }
  template <typename U> U cast() const { assert(isa<U>()); return U(*this); }
  void print(std::ostream& os) const;
};
class StringAttr : public Attribute {
public:
  StringAttr() = default;
  StringAttr(const Attribute& a) : Attribute(a) {}
  static bool classof(const Attribute& a) { return a.kind == String; }
  static StringAttr get(MLIRContext*, const std::string& v) { StringAttr a; a.kind = String; a.s = v; return a; }
  std::string getValue() const { return s; }
  std::string str() const { return s; }
};
class IntegerAttr : public Attribute {
public:
  IntegerAttr() = default;
  IntegerAttr(const Attribute& a) : Attribute(a) {}
  static bool classof(const Attribute& a) { return a.kind == Integer; }
  static IntegerAttr get(Type t, int64_t v) { IntegerAttr a; a.kind = Integer; a.type = t; a.i = v; return a; }
  int64_t getInt() const { return i; }
  int64_t getValue() const { return i; }
  Type getType() const { return type; }
};
class FloatAttr : public Attribute {
public:
  FloatAttr() = default;
  FloatAttr(const Attribute& a) : Attribute(a) {}
  static bool classof(const Attribute& a) { return a.kind == Float; }
  static FloatAttr get(Type t, double v);  // value is rounded to the precision of `t`
  double getValueAsDouble() const { return f; }
  Type getType() const { return type; }
};
class AffineMapAttr : public Attribute {
public:
  AffineMapAttr() = default;
  AffineMapAttr(const Attribute& a) : Attribute(a) {}
  static bool classof(const Attribute& a) { return a.kind == Map; }
  static AffineMapAttr get(AffineMap m) { AffineMapAttr a; a.kind = Map; a.map = m; return a; }
  AffineMap getValue() const { return map; }
};
class IntegerSetAttr : public Attribute {
public:
  IntegerSetAttr() = default;
  IntegerSetAttr(const Attribute& a) : Attribute(a) {}
  static bool classof(const Attribute& a) { return a.kind == Set; }
  static IntegerSetAttr get(IntegerSet s) { IntegerSetAttr a; a.kind = Set; a.set = s; return a; }
  IntegerSet getValue() const { return set; }
};
class TypeAttr : public Attribute {
public:
  TypeAttr() = default;
  TypeAttr(const Attribute& a) : Attribute(a) {}
  static bool classof(const Attribute& a) { return a.kind == TypeKind; }
  static TypeAttr get(Type t) { TypeAttr a; a.kind = TypeKind; a.type = t; return a; }
  Type getValue() const { return type; }
};
class UnitAttr : public Attribute {
public:
  static bool classof(const Attribute& a) { return a.kind == Unit; }
  static UnitAttr get(MLIRContext* = nullptr) { UnitAttr a; a.kind = Unit; return a; }
};
Attribute getIntArrayAttr(ArrayRef<int64_t> v);

// ---------------------------------------------------------------------------
// Values
// ---------------------------------------------------------------------------
namespace detail {
struct ValueImpl {
  Type type;
  Operation* definingOp = nullptr;  // op result
  Block* ownerBlock = nullptr;      // block argument
  unsigned index = 0;               // result number or argument number
  std::vector<Operation*> users;    // one entry per use (an op using the value twice appears twice)
};
}  // namespace detail

class Value {
public:
  Value() = default;
  Value(std::nullptr_t) {}
  explicit Value(detail::ValueImpl* impl) : impl(impl) {}
  explicit operator bool() const { return impl != nullptr; }
  bool operator==(const Value& o) const { return impl == o.impl; }
  bool operator!=(const Value& o) const { return impl != o.impl; }
  bool operator<(const Value& o) const { return impl < o.impl; }
  Type getType() const { return impl->type; }
  void setType(Type t) { impl->type = t; }
  Operation* getDefiningOp() const { return impl->definingOp; }
  template <typename OpTy> OpTy getDefiningOp() const;
  Block* getParentBlock() const;
  using user_range = std::vector<Operation*>;
  // Distinct users in first-use order.
  user_range getUsers() const;
  bool use_empty() const { return impl->users.empty(); }
  bool hasOneUse() const { return impl->users.size() == 1; }
  size_t getNumUses() const { return impl->users.size(); }
  void replaceAllUsesWith(Value newValue) const;
  void replaceUsesWithIf(Value newValue, const std::function<bool(Operation*)>& shouldReplace) const;
  template <typename U> bool isa() const { return impl && U::classof(*this); }
  template <typename U> U dyn_cast() const { return isa<U>() ? U(impl) : U(); }
  template <typename U> U cast() const { assert(isa<U>()); return U(impl); }
  detail::ValueImpl* getImpl() const { return impl; }
  void dump() const;

protected:
  detail::ValueImpl* impl = nullptr;
};

class BlockArgument : public Value {
public:
  using Value::Value;
  BlockArgument() = default;
  static bool classof(Value v) { return v.getImpl()->ownerBlock != nullptr; }
  unsigned getArgNumber() const { return impl->index; }
  Block* getOwner() const { return impl->ownerBlock; }
};
class OpResult : public Value {
public:
  using Value::Value;
  OpResult() = default;
  static bool classof(Value v) { return v.getImpl()->definingOp != nullptr; }
  unsigned getResultNumber() const { return impl->index; }
  Operation* getOwner() const { return impl->definingOp; }
};

class ValueRange : public std::vector<Value> {
public:
  using Base = std::vector<Value>;
  using Base::Base;
  ValueRange() = default;
  ValueRange(const Base& v) : Base(v) {}
  ValueRange(std::initializer_list<Value> il) : Base(il) {}
  ValueRange(Value v) : Base(1, v) {}
  ValueRange(ArrayRef<Value> a) : Base(a.begin(), a.end()) {}
  template <unsigned N>
  ValueRange(const SmallVector<Value, N>& v) : Base(v.begin(), v.end()) {}
  ValueRange(const std::vector<BlockArgument>& v) { for (auto a : v) push_back(a); }
  std::vector<Type> getTypes() const { std::vector<Type> t; for (auto v : *this) t.push_back(v.getType()); return t; }
  ValueRange drop_front(size_t n = 1) const { return ValueRange(Base(begin() + n, end())); }
};

class BlockAndValueMapping {
public:
  void map(Value from, Value to) { values[from.getImpl()] = to; }
  void map(Block* from, Block* to) { blocks[from] = to; }
  Value lookupOrDefault(Value from) const { auto it = values.find(from.getImpl()); return it == values.end() ? from : it->second; }
  Value lookupOrNull(Value from) const { auto it = values.find(from.getImpl()); return it == values.end() ? Value() : it->second; }
  Value lookup(Value from) const { auto v = lookupOrNull(from); assert(v && "expected a mapping"); return v; }
  bool contains(Value from) const { return values.count(from.getImpl()) != 0; }
  void clear() { values.clear(); blocks.clear(); }

private:
  std::unordered_map<detail::ValueImpl*, Value> values;
  std::unordered_map<Block*, Block*> blocks;
};
using IRMapping = BlockAndValueMapping;

// ---------------------------------------------------------------------------
// Operations, blocks, regions
// ---------------------------------------------------------------------------
enum class OpKind {
  Module, Func, Call, Return,
  Alloc, MemLoad, MemStore,
  AffineFor, AffineParallel, AffineIf, AffineLoad, AffineStore, AffineVectorLoad, AffineVectorStore,
  AffineApply, AffineYield,
  Constant, AddF, SubF, MulF, DivF, MaxF, MinF, NegF, CmpF, Bitcast, AddI, SubI, MulI, Select, FPToSI, SIToFP, ExtF, TruncF,
  Exp, Exp2, Tanh, Sqrt, Rsqrt, Log, PowF, Abs,
  Barrier, Shuffle,
};
const char* getOpName(OpKind kind);

enum class WalkOrder { PreOrder, PostOrder };

class Operation {
public:
  static Operation* create(OpKind kind, ArrayRef<Value> operands, ArrayRef<Type> resultTypes, unsigned numRegions = 0);
  ~Operation();
  Operation(const Operation&) = delete;

  OpKind getKind() const { return kind; }
  std::string getName() const { return getOpName(kind); }
  MLIRContext* getContext() const { return getGlobalContext(); }
  Location getLoc() const { return Location(); }

  // operands
  unsigned getNumOperands() const { return (unsigned)operands.size(); }
  Value getOperand(unsigned i) const { return operands[i]; }
  const std::vector<Value>& getOperands() const { return operands; }
  void setOperand(unsigned i, Value v);
  void setOperands(ValueRange newOperands);
  void insertOperand(unsigned pos, Value v);
  void eraseOperand(unsigned pos);
  void replaceUsesOfWith(Value from, Value to);

  // results
  unsigned getNumResults() const { return (unsigned)results.size(); }
  Value getResult(unsigned i) const { return Value(results[i]); }
  std::vector<Value> getResults() const;
  bool use_empty() const;
  void replaceAllUsesWith(Operation* other);
  void replaceAllUsesWith(ValueRange values);

  // attributes
  void setAttr(const std::string& name, Attribute a) { attrs[name] = a; }
  Attribute getAttr(const std::string& name) const { auto it = attrs.find(name); return it == attrs.end() ? Attribute() : it->second; }
  template <typename A> A getAttrOfType(const std::string& name) const { return getAttr(name).dyn_cast<A>(); }
  bool hasAttr(const std::string& name) const { return attrs.count(name) != 0; }
  void removeAttr(const std::string& name) { attrs.erase(name); }
  const std::map<std::string, Attribute>& getAttrs() const { return attrs; }

  // structure
  unsigned getNumRegions() const { return (unsigned)regions.size(); }
  Region& getRegion(unsigned i) { return *regions[i]; }
  Block* getBlock() const { return block; }
  Operation* getParentOp() const;
  Region* getParentRegion() const;
  template <typename OpTy> OpTy getParentOfType() const;
  Operation* getNextNode() const { return next; }
  Operation* getPrevNode() const { return prev; }
  bool isBeforeInBlock(Operation* other) const;
  bool isAncestor(Operation* other) const;         // `other` is this op or nested inside it
  bool isProperAncestor(Operation* other) const;

  // mutation
  void erase();                    // unlink and delete (results must be unused)
  void remove();                   // unlink only
  void moveBefore(Operation* other);
  void moveAfter(Operation* other);
  void moveBefore(Block* b, Operation* before /*nullptr = end*/);
  void dropAllReferences();
  void dropAllUses();

  Operation* clone() { BlockAndValueMapping m; return clone(m); }
  Operation* clone(BlockAndValueMapping& mapper);

  void walk(const std::function<void(Operation*)>& fn, WalkOrder order = WalkOrder::PostOrder);
  template <WalkOrder Order = WalkOrder::PostOrder, typename Fn> void walk(Fn&& fn);

  void print(std::ostream& os) const;
  void dump() const;
  LogicalResult emitError(const std::string& msg) const;
  Operation* operator->() { return this; }

private:
  Operation() = default;
  friend class Block;
  OpKind kind;
  std::vector<Value> operands;
  std::vector<detail::ValueImpl*> results;
  std::map<std::string, Attribute> attrs;
  std::vector<std::unique_ptr<Region>> regions;
  Block* block = nullptr;
  Operation* prev = nullptr;
  Operation* next = nullptr;
};

// Intrusive list of the operations of a block.  Iteration yields Operation&.
class OpList {
public:
  class iterator {
  public:
    using iterator_category = std::bidirectional_iterator_tag;
    using value_type = Operation;
    using difference_type = std::ptrdiff_t;
    using pointer = Operation*;
    using reference = Operation&;
    iterator() = default;
    iterator(Block* b, Operation* op) : block(b), op(op) {}
    Operation& operator*() const { return *op; }
    Operation* operator->() const { return op; }
    iterator& operator++();
    iterator operator++(int) { iterator t = *this; ++*this; return t; }
    iterator& operator--();
    iterator operator--(int) { iterator t = *this; --*this; return t; }
    bool operator==(const iterator& o) const { return op == o.op && block == o.block; }
    bool operator!=(const iterator& o) const { return !(*this == o); }
    Operation* getNodePtr() const { return op; }
    Block* block = nullptr;
    Operation* op = nullptr;  // nullptr = end()
  };
  explicit OpList(Block* owner) : owner(owner) {}
  iterator begin() const;
  iterator end() const { return iterator(owner, nullptr); }
  size_t size() const;
  bool empty() const;
  Operation& front() const;
  Operation& back() const;
  // Move [first, last) of `other` in front of `where`.
  void splice(iterator where, OpList& other, iterator first, iterator last);
  void splice(iterator where, OpList& other, iterator first);
  void splice(iterator where, OpList& other) { splice(where, other, other.begin(), other.end()); }
  void push_back(Operation* op);
  void push_front(Operation* op);
  void insert(iterator where, Operation* op);

private:
  Block* owner;
};

class Block {
public:
  Block() : ops(this) {}
  ~Block();
  using iterator = OpList::iterator;
  OpList& getOperations() { return ops; }
  iterator begin() { return ops.begin(); }
  iterator end() { return ops.end(); }
  bool empty() const { return head == nullptr; }
  Operation& front() { return *head; }
  Operation& back() { return *tail; }
  Operation* getTerminator() { return tail; }
  void push_back(Operation* op) { insertBefore(op, nullptr); }
  void push_front(Operation* op) { insertBefore(op, head); }
  void insertBefore(Operation* op, Operation* before /*nullptr = end*/);

  BlockArgument addArgument(Type type, Location = Location());
  void addArguments(Type type, Location loc = Location()) { addArgument(type, loc); }
  void addArguments(ArrayRef<Type> types, ArrayRef<Location> = {}) { for (auto t : types) addArgument(t); }
  BlockArgument insertArgument(unsigned pos, Type type);
  void eraseArgument(unsigned pos);
  unsigned getNumArguments() const { return (unsigned)arguments.size(); }
  BlockArgument getArgument(unsigned i) const { return BlockArgument(arguments[i]); }
  std::vector<BlockArgument> getArguments() const;

  Region* getParent() const { return parent; }
  Operation* getParentOp() const;
  template <WalkOrder Order = WalkOrder::PostOrder, typename Fn> void walk(Fn&& fn);

private:
  friend class Operation;
  friend class OpList;
  friend class Region;
  OpList ops;
  Operation* head = nullptr;
  Operation* tail = nullptr;
  std::vector<detail::ValueImpl*> arguments;
  Region* parent = nullptr;
};

class Region {
public:
  explicit Region(Operation* owner) : owner(owner) {}
  bool empty() const { return blocks.empty(); }
  bool hasOneBlock() const { return blocks.size() == 1; }
  Block& front() { return *blocks.front(); }
  Block& back() { return *blocks.back(); }
  Block& emplaceBlock();
  std::vector<std::unique_ptr<Block>>& getBlocks() { return blocks; }
  Operation* getParentOp() const { return owner; }
  void push_back(Block* b);

private:
  Operation* owner;
  std::vector<std::unique_ptr<Block>> blocks;
};

// ---------------------------------------------------------------------------
// Op wrappers
// ---------------------------------------------------------------------------
class OpState {
public:
  OpState() = default;
  OpState(std::nullptr_t) {}
  explicit OpState(Operation* op) : state(op) {}
  explicit operator bool() const { return state != nullptr; }
  operator Operation*() const { return state; }
  Operation* operator->() const { return state; }
  Operation* getOperation() const { return state; }
  MLIRContext* getContext() const { return getGlobalContext(); }
  Location getLoc() const { return Location(); }
  bool operator==(const OpState& o) const { return state == o.state; }
  bool operator!=(const OpState& o) const { return state != o.state; }
  void erase() { state->erase(); state = nullptr; }
  void dump() const { state->dump(); }
  LogicalResult emitError(const std::string& msg) const { return state->emitError(msg); }
  template <WalkOrder Order = WalkOrder::PostOrder, typename Fn> void walk(Fn&& fn) { state->template walk<Order>(std::forward<Fn>(fn)); }

protected:
  Operation* state = nullptr;
};

template <typename OpTy> bool isa(Operation* op) { return op && OpTy::classof(op); }
template <typename OpTy> bool isa(Operation& op) { return OpTy::classof(&op); }
template <typename OpTy> OpTy dyn_cast(Operation* op) { return (op && OpTy::classof(op)) ? OpTy(op) : OpTy(); }
template <typename OpTy> OpTy dyn_cast(Operation& op) { return OpTy::classof(&op) ? OpTy(&op) : OpTy(); }
template <typename OpTy> OpTy dyn_cast(const OpState& op) { return dyn_cast<OpTy>(op.getOperation()); }
template <typename OpTy> OpTy dyn_cast_or_null(Operation* op) { return dyn_cast<OpTy>(op); }
template <typename OpTy> OpTy cast(Operation* op) { assert(isa<OpTy>(op)); return OpTy(op); }

#define KCG_OP_COMMON(NAME, KIND)                                         \
  using OpState::OpState;                                                 \
  NAME() = default;                                                       \
  static bool classof(Operation* op) { return op->getKind() == OpKind::KIND; }

class ModuleOp : public OpState {
public:
  KCG_OP_COMMON(ModuleOp, Module)
  static ModuleOp create(Location, Optional<StringRef> name = std::nullopt);
  Block* getBody() const { return &state->getRegion(0).front(); }
  Optional<StringRef> getName() const;
  std::string getSymName() const;
  ModuleOp clone() const { return ModuleOp(state->clone()); }
  void destroy();  // deletes the module and everything in it
};

namespace func {
class FuncOp : public OpState {
public:
  KCG_OP_COMMON(FuncOp, Func)
  static FuncOp create(OpBuilder& b, Location, StringRef name, FunctionType type);
  std::string getSymName() const { return state->getAttr("sym_name").s; }
  std::string getName() const { return getSymName(); }
  void setName(const std::string& n);
  FunctionType getFunctionType() const { return state->getAttr("function_type").type.cast<FunctionType>(); }
  void setType(FunctionType t) { state->setAttr("function_type", TypeAttr::get(t)); }
  void setFunctionType(FunctionType t) { setType(t); }
  Region& getBody() const { return state->getRegion(0); }
  Block& front() const { return state->getRegion(0).front(); }
  std::vector<BlockArgument> getArguments() const { return front().getArguments(); }
  BlockArgument getArgument(unsigned i) const { return front().getArgument(i); }
  unsigned getNumArguments() const { return front().getNumArguments(); }
  bool empty() const { return state->getRegion(0).empty(); }
};
class CallOp : public OpState {
public:
  KCG_OP_COMMON(CallOp, Call)
  static CallOp create(OpBuilder& b, Location, FuncOp callee, ValueRange operands);
  static CallOp create(OpBuilder& b, Location, StringRef callee, TypeRange results, ValueRange operands);
  std::string getCallee() const { return state->getAttr("callee").s; }
  void setCallee(const std::string& n);
  Value getResult(unsigned i = 0) const { return state->getResult(i); }
  const std::vector<Value>& getOperands() const { return state->getOperands(); }
  Value getOperand(unsigned i) const { return state->getOperand(i); }
};
class ReturnOp : public OpState {
public:
  KCG_OP_COMMON(ReturnOp, Return)
  static ReturnOp create(OpBuilder& b, Location, ValueRange operands = {});
};
}  // namespace func

namespace memref {
class AllocOp : public OpState {
public:
  KCG_OP_COMMON(AllocOp, Alloc)
  static AllocOp create(OpBuilder& b, Location, MemRefType type);
  Value getResult() const { return state->getResult(0); }
  Value getMemref() const { return state->getResult(0); }
  MemRefType getType() const { return state->getResult(0).getType().cast<MemRefType>(); }
};
class LoadOp : public OpState {
public:
  KCG_OP_COMMON(LoadOp, MemLoad)
  static LoadOp create(OpBuilder& b, Location, Value memref, ValueRange indices);
  Value getResult() const { return state->getResult(0); }
  Value getMemRef() const { return state->getOperand(0); }
  Value getMemref() const { return state->getOperand(0); }
  ValueRange getIndices() const;
};
class StoreOp : public OpState {
public:
  KCG_OP_COMMON(StoreOp, MemStore)
  static StoreOp create(OpBuilder& b, Location, Value value, Value memref, ValueRange indices);
  Value getValue() const { return state->getOperand(0); }
  Value getMemRef() const { return state->getOperand(1); }
  ValueRange getIndices() const;
};
}  // namespace memref

// ---- affine ----
class AffineYieldOp : public OpState {
public:
  KCG_OP_COMMON(AffineYieldOp, AffineYield)
  static AffineYieldOp create(OpBuilder& b, Location, ValueRange operands = {});
};

class AffineForOp : public OpState {
public:
  KCG_OP_COMMON(AffineForOp, AffineFor)
  using BodyBuilderFn = std::function<void(OpBuilder&, Location, Value, ValueRange)>;
  // Constant bounds.  The body builder, when given, must create the terminator.
  static AffineForOp create(OpBuilder& b, Location, int64_t lb, int64_t ub, int64_t step = 1,
                            ValueRange iterArgs = {}, BodyBuilderFn bodyBuilder = nullptr);
  // General bounds (single-result maps).
  static AffineForOp create(OpBuilder& b, Location, ValueRange lbOperands, AffineMap lbMap, ValueRange ubOperands,
                            AffineMap ubMap, int64_t step = 1, ValueRange iterArgs = {},
                            BodyBuilderFn bodyBuilder = nullptr);
  Block* getBody() const { return &state->getRegion(0).front(); }
  Region& getRegion() const { return state->getRegion(0); }
  Region& getLoopBody() const { return state->getRegion(0); }
  Value getInductionVar() const { return getBody()->getArgument(0); }
  std::vector<BlockArgument> getRegionIterArgs() const;
  ValueRange getIterOperands() const;
  unsigned getNumIterOperands() const;
  unsigned getNumResults() const { return state->getNumResults(); }
  Value getResult(unsigned i) const { return state->getResult(i); }
  std::vector<Value> getResults() const { return state->getResults(); }
  AffineMap getLowerBoundMap() const { return state->getAttr("lower_bound").map; }
  AffineMap getUpperBoundMap() const { return state->getAttr("upper_bound").map; }
  ValueRange getLowerBoundOperands() const;
  ValueRange getUpperBoundOperands() const;
  void setLowerBound(ValueRange operands, AffineMap map);
  void setUpperBound(ValueRange operands, AffineMap map);
  void setLowerBoundMap(AffineMap map) { state->setAttr("lower_bound", AffineMapAttr::get(map)); }
  void setUpperBoundMap(AffineMap map) { state->setAttr("upper_bound", AffineMapAttr::get(map)); }
  bool hasConstantLowerBound() const { return getLowerBoundMap().isSingleConstant(); }
  bool hasConstantUpperBound() const { return getUpperBoundMap().isSingleConstant(); }
  bool hasConstantBounds() const { return hasConstantLowerBound() && hasConstantUpperBound(); }
  int64_t getConstantLowerBound() const { return getLowerBoundMap().getSingleConstantResult(); }
  int64_t getConstantUpperBound() const { return getUpperBoundMap().getSingleConstantResult(); }
  void setConstantLowerBound(int64_t v) { setLowerBound({}, AffineMap::getConstantMap(v)); }
  void setConstantUpperBound(int64_t v) { setUpperBound({}, AffineMap::getConstantMap(v)); }
  int64_t getStep() const { return state->getAttr("step").i; }
  void setStep(int64_t s);
};

class AffineParallelOp : public OpState {
public:
  KCG_OP_COMMON(AffineParallelOp, AffineParallel)
  // Constant ranges [lb_i, ub_i) with steps; the body gets one index per dim
  // and is terminated by an empty affine.yield.
  static AffineParallelOp create(OpBuilder& b, Location, ArrayRef<int64_t> lbs, ArrayRef<int64_t> ubs,
                                 ArrayRef<int64_t> steps = {});
  // Ranges [0, range_i), step 1 (the form MLIR's (resultTypes, reductions, ranges) builder gives).
  static AffineParallelOp create(OpBuilder& b, Location, TypeRange resultTypes, ArrayRef<int> reductions,
                                 ArrayRef<int64_t> ranges);
  Block* getBody() const { return &state->getRegion(0).front(); }
  Region& getRegion() const { return state->getRegion(0); }
  unsigned getNumDims() const { return (unsigned)state->getAttr("upper_bounds").ints.size(); }
  std::vector<Value> getIVs() const;
  AffineMap getLowerBoundMap(unsigned i) const { return AffineMap::getConstantMap(state->getAttr("lower_bounds").ints[i]); }
  AffineMap getUpperBoundMap(unsigned i) const { return AffineMap::getConstantMap(state->getAttr("upper_bounds").ints[i]); }
  std::vector<int64_t> getConstantLowerBounds() const { return state->getAttr("lower_bounds").ints; }
  std::vector<int64_t> getConstantUpperBounds() const { return state->getAttr("upper_bounds").ints; }
  SmallVector<int64_t> getSteps() const { return SmallVector<int64_t>(state->getAttr("steps").ints); }
  Optional<SmallVector<int64_t>> getConstantRanges() const;
  void setBounds(ArrayRef<int64_t> lbs, ArrayRef<int64_t> ubs, ArrayRef<int64_t> steps);
};

class AffineIfOp : public OpState {
public:
  KCG_OP_COMMON(AffineIfOp, AffineIf)
  static AffineIfOp create(OpBuilder& b, Location, IntegerSet set, ValueRange operands, bool withElseRegion = false);
  IntegerSet getIntegerSet() const { return state->getAttr("condition").set; }
  void setIntegerSet(IntegerSet s) { state->setAttr("condition", IntegerSetAttr::get(s)); }
  void setConditional(IntegerSet s, ValueRange operands);
  const std::vector<Value>& getOperands() const { return state->getOperands(); }
  Block* getThenBlock() const { return &state->getRegion(0).front(); }
  Block* getBody() const { return getThenBlock(); }
  bool hasElse() const { return !state->getRegion(1).empty(); }
  Block* getElseBlock() const { return &state->getRegion(1).front(); }
};

class AffineApplyOp : public OpState {
public:
  KCG_OP_COMMON(AffineApplyOp, AffineApply)
  static AffineApplyOp create(OpBuilder& b, Location, AffineMap map, ValueRange operands);
  AffineMap getAffineMap() const { return state->getAttr("map").map; }
  void setMap(AffineMap m) { state->setAttr("map", AffineMapAttr::get(m)); }
  const std::vector<Value>& getMapOperands() const { return state->getOperands(); }
  const std::vector<Value>& getOperands() const { return state->getOperands(); }
  Value getResult() const { return state->getResult(0); }
};

// Shared accessors of affine.load / affine.vector_load (memref, indices...) and
// affine.store / affine.vector_store (value, memref, indices...).
template <unsigned MemrefOperand>
class AffineMemOpBase : public OpState {
public:
  using OpState::OpState;
  AffineMemOpBase() = default;
  Value getMemRef() const { return state->getOperand(MemrefOperand); }
  Value getMemref() const { return getMemRef(); }
  void setMemRef(Value v) { state->setOperand(MemrefOperand, v); }
  MemRefType getMemRefType() const { return getMemRef().getType().template cast<MemRefType>(); }
  AffineMap getAffineMap() const { return state->getAttr("map").map; }
  AffineMapAttr getAffineMapAttr() const { return AffineMapAttr(state->getAttr("map")); }
  void setMap(AffineMap m) { state->setAttr("map", AffineMapAttr::get(m)); }
  ValueRange getMapOperands() const {
    auto& ops = state->getOperands();
    return ValueRange(std::vector<Value>(ops.begin() + MemrefOperand + 1, ops.end()));
  }
  ValueRange getIndices() const { return getMapOperands(); }
  // Replace memref, map and map operands in one go.
  void setAccess(Value memref, AffineMap map, ValueRange mapOperands) {
    std::vector<Value> ops(state->getOperands().begin(), state->getOperands().begin() + MemrefOperand);
    ops.push_back(memref);
    ops.insert(ops.end(), mapOperands.begin(), mapOperands.end());
    state->setOperands(ops);
    setMap(map);
  }
};

class AffineLoadOp : public AffineMemOpBase<0> {
public:
  using AffineMemOpBase<0>::AffineMemOpBase;
  AffineLoadOp() = default;
  static bool classof(Operation* op) { return op->getKind() == OpKind::AffineLoad; }
  static AffineLoadOp create(OpBuilder& b, Location, Value memref, ValueRange indices);  // identity map
  static AffineLoadOp create(OpBuilder& b, Location, Value memref, AffineMap map, ValueRange mapOperands);
  Value getResult() const { return state->getResult(0); }
  operator Value() const { return getResult(); }
};
class AffineStoreOp : public AffineMemOpBase<1> {
public:
  using AffineMemOpBase<1>::AffineMemOpBase;
  AffineStoreOp() = default;
  static bool classof(Operation* op) { return op->getKind() == OpKind::AffineStore; }
  static AffineStoreOp create(OpBuilder& b, Location, Value value, Value memref, ValueRange indices);
  static AffineStoreOp create(OpBuilder& b, Location, Value value, Value memref, AffineMap map, ValueRange mapOperands);
  Value getValue() const { return state->getOperand(0); }
  Value getValueToStore() const { return state->getOperand(0); }
};
class AffineVectorLoadOp : public AffineMemOpBase<0> {
public:
  using AffineMemOpBase<0>::AffineMemOpBase;
  AffineVectorLoadOp() = default;
  static bool classof(Operation* op) { return op->getKind() == OpKind::AffineVectorLoad; }
  static AffineVectorLoadOp create(OpBuilder& b, Location, VectorType resultType, Value memref, ValueRange indices);
  static AffineVectorLoadOp create(OpBuilder& b, Location, VectorType resultType, Value memref, AffineMap map,
                                   ValueRange mapOperands);
  Value getResult() const { return state->getResult(0); }
  VectorType getVectorType() const { return getResult().getType().cast<VectorType>(); }
  operator Value() const { return getResult(); }
};
class AffineVectorStoreOp : public AffineMemOpBase<1> {
public:
  using AffineMemOpBase<1>::AffineMemOpBase;
  AffineVectorStoreOp() = default;
  static bool classof(Operation* op) { return op->getKind() == OpKind::AffineVectorStore; }
  static AffineVectorStoreOp create(OpBuilder& b, Location, Value value, Value memref, ValueRange indices);
  static AffineVectorStoreOp create(OpBuilder& b, Location, Value value, Value memref, AffineMap map,
                                    ValueRange mapOperands);
  Value getValue() const { return state->getOperand(0); }
  Value getValueToStore() const { return state->getOperand(0); }
  VectorType getVectorType() const { return getValue().getType().cast<VectorType>(); }
};

// ---- arith / math ----
namespace arith {
enum class CmpFPredicate { AlwaysFalse, OEQ, OGT, OGE, OLT, OLE, ONE, ORD, UEQ, UGT, UGE, ULT, ULE, UNE, UNO, AlwaysTrue };

class ConstantOp : public OpState {
public:
  KCG_OP_COMMON(ConstantOp, Constant)
  static ConstantOp create(OpBuilder& b, Location, Attribute value);
  static ConstantOp create(OpBuilder& b, Location, Type type, Attribute value);
  Attribute getValue() const { return state->getAttr("value"); }
  Value getResult() const { return state->getResult(0); }
  Type getType() const { return state->getResult(0).getType(); }
  operator Value() const { return getResult(); }
};
class ConstantIndexOp : public ConstantOp {
public:
  using ConstantOp::ConstantOp;
  ConstantIndexOp() = default;
  static bool classof(Operation* op) { return ConstantOp::classof(op) && op->getResult(0).getType().isIndex(); }
  static ConstantIndexOp create(OpBuilder& b, Location, int64_t value);
  int64_t value() const { return state->getAttr("value").i; }
};
class ConstantIntOp : public ConstantOp {
public:
  using ConstantOp::ConstantOp;
  ConstantIntOp() = default;
  static bool classof(Operation* op) { return ConstantOp::classof(op) && op->getResult(0).getType().isa<IntegerType>(); }
  static ConstantIntOp create(OpBuilder& b, Location, int64_t value, unsigned width);
  static ConstantIntOp create(OpBuilder& b, Location, int64_t value, Type type);
  int64_t value() const { return state->getAttr("value").i; }
};
class ConstantFloatOp : public ConstantOp {
public:
  using ConstantOp::ConstantOp;
  ConstantFloatOp() = default;
  static bool classof(Operation* op) { return ConstantOp::classof(op) && op->getResult(0).getType().isFloat(); }
  static ConstantFloatOp create(OpBuilder& b, Location, double value, FloatType type);
  double value() const { return state->getAttr("value").f; }
};

#define KCG_BINARY_OP(NAME, KIND)                                            \
  class NAME : public OpState {                                              \
  public:                                                                    \
    KCG_OP_COMMON(NAME, KIND)                                                \
    static NAME create(OpBuilder& b, Location, Value lhs, Value rhs);        \
    Value getLhs() const { return state->getOperand(0); }                    \
    Value getRhs() const { return state->getOperand(1); }                    \
    Value getResult() const { return state->getResult(0); }                  \
    operator Value() const { return getResult(); }                           \
  };
#define KCG_UNARY_OP(NAME, KIND)                                             \
  class NAME : public OpState {                                              \
  public:                                                                    \
    KCG_OP_COMMON(NAME, KIND)                                                \
    static NAME create(OpBuilder& b, Location, Value operand);               \
    Value getOperand() const { return state->getOperand(0); }                \
    Value getResult() const { return state->getResult(0); }                  \
    operator Value() const { return getResult(); }                           \
  };
#define KCG_CAST_OP(NAME, KIND)                                              \
  class NAME : public OpState {                                              \
  public:                                                                    \
    KCG_OP_COMMON(NAME, KIND)                                                \
    static NAME create(OpBuilder& b, Location, Type resultType, Value in);   \
    Value getIn() const { return state->getOperand(0); }                     \
    Value getResult() const { return state->getResult(0); }                  \
    operator Value() const { return getResult(); }                           \
  };
KCG_BINARY_OP(AddFOp, AddF)
KCG_BINARY_OP(SubFOp, SubF)
KCG_BINARY_OP(MulFOp, MulF)
KCG_BINARY_OP(DivFOp, DivF)
KCG_BINARY_OP(MaxFOp, MaxF)
KCG_BINARY_OP(MinFOp, MinF)
KCG_BINARY_OP(AddIOp, AddI)
KCG_BINARY_OP(SubIOp, SubI)
KCG_BINARY_OP(MulIOp, MulI)
KCG_UNARY_OP(NegFOp, NegF)
KCG_CAST_OP(BitcastOp, Bitcast)
KCG_CAST_OP(FPToSIOp, FPToSI)
KCG_CAST_OP(SIToFPOp, SIToFP)
KCG_CAST_OP(ExtFOp, ExtF)
KCG_CAST_OP(TruncFOp, TruncF)

class CmpFOp : public OpState {
public:
  KCG_OP_COMMON(CmpFOp, CmpF)
  static CmpFOp create(OpBuilder& b, Location, CmpFPredicate pred, Value lhs, Value rhs);
  CmpFPredicate getPredicate() const { return (CmpFPredicate)state->getAttr("predicate").i; }
  Value getLhs() const { return state->getOperand(0); }
  Value getRhs() const { return state->getOperand(1); }
  Value getResult() const { return state->getResult(0); }
  operator Value() const { return getResult(); }
};
class SelectOp : public OpState {
public:
  KCG_OP_COMMON(SelectOp, Select)
  static SelectOp create(OpBuilder& b, Location, Value cond, Value trueValue, Value falseValue);
  Value getResult() const { return state->getResult(0); }
  operator Value() const { return getResult(); }
};
}  // namespace arith

namespace math {
KCG_UNARY_OP(ExpOp, Exp)
KCG_UNARY_OP(Exp2Op, Exp2)
KCG_UNARY_OP(TanhOp, Tanh)
KCG_UNARY_OP(SqrtOp, Sqrt)
KCG_UNARY_OP(RsqrtOp, Rsqrt)
KCG_UNARY_OP(LogOp, Log)
KCG_UNARY_OP(AbsOp, Abs)
KCG_BINARY_OP(PowFOp, PowF)
}  // namespace math
#undef KCG_BINARY_OP
#undef KCG_UNARY_OP
#undef KCG_CAST_OP

namespace gpu {
enum class ShuffleMode { XOR = 0, UP = 2, DOWN = 1, IDX = 3 };
class BarrierOp : public OpState {
public:
  KCG_OP_COMMON(BarrierOp, Barrier)
  static BarrierOp create(OpBuilder& b, Location);
};
class ShuffleOp : public OpState {
public:
  KCG_OP_COMMON(ShuffleOp, Shuffle)
  // results: shuffled value, validity bit (i1)
  static ShuffleOp create(OpBuilder& b, Location, Value value, Value offset, Value width, ShuffleMode mode);
  static ShuffleOp create(OpBuilder& b, Location, Value value, int32_t offset, int32_t width, ShuffleMode mode);
  ShuffleMode getMode() const { return (ShuffleMode)state->getAttr("mode").i; }
  Value getValue() const { return state->getOperand(0); }
  Value getOffset() const { return state->getOperand(1); }
  Value getWidth() const { return state->getOperand(2); }
  Value getResult(unsigned i = 0) const { return state->getResult(i); }
  Value getShuffleResult() const { return state->getResult(0); }
};
}  // namespace gpu
#undef KCG_OP_COMMON

// ---------------------------------------------------------------------------
// Builder
// ---------------------------------------------------------------------------
class OpBuilder {
public:
  struct InsertPoint {
    Block* block = nullptr;
    Operation* before = nullptr;  // nullptr = end of block
    bool isSet() const { return block != nullptr; }
    Block* getBlock() const { return block; }
  };
  explicit OpBuilder(MLIRContext* ctx = nullptr) { (void)ctx; }
  explicit OpBuilder(Operation* op) { setInsertionPoint(op); }
  OpBuilder(const OpState& op) { setInsertionPoint(op.getOperation()); }
  OpBuilder(Block* block, Block::iterator where) { setInsertionPoint(block, where); }
  static OpBuilder atBlockBegin(Block* b) { OpBuilder r; r.setInsertionPointToStart(b); return r; }
  static OpBuilder atBlockEnd(Block* b) { OpBuilder r; r.setInsertionPointToEnd(b); return r; }
  static OpBuilder atBlockTerminator(Block* b) { OpBuilder r; r.setInsertionPoint(b->getTerminator()); return r; }

  MLIRContext* getContext() const { return getGlobalContext(); }
  Location getUnknownLoc() const { return Location(); }

  void setInsertionPoint(Block* block, Block::iterator where) { ip.block = block; ip.before = where.getNodePtr(); }
  void setInsertionPoint(Operation* op) { ip.block = op->getBlock(); ip.before = op; }
  void setInsertionPointAfter(Operation* op) { ip.block = op->getBlock(); ip.before = op->getNextNode(); }
  void setInsertionPointToStart(Block* b) { ip.block = b; ip.before = b->empty() ? nullptr : &b->front(); }
  void setInsertionPointToEnd(Block* b) { ip.block = b; ip.before = nullptr; }
  void clearInsertionPoint() { ip = InsertPoint(); }
  InsertPoint saveInsertionPoint() const { return ip; }
  void restoreInsertionPoint(InsertPoint p) { ip = p; }
  Block* getInsertionBlock() const { return ip.block; }
  Block::iterator getInsertionPoint() const { return Block::iterator(ip.block, ip.before); }
  Block* getBlock() const { return ip.block; }

  class InsertionGuard {
  public:
    explicit InsertionGuard(OpBuilder& b) : builder(b), saved(b.saveInsertionPoint()) {}
    ~InsertionGuard() { builder.restoreInsertionPoint(saved); }
  private:
    OpBuilder& builder;
    InsertPoint saved;
  };

  Operation* insert(Operation* op);
  template <typename OpTy, typename... Args>
  OpTy create(Location loc, Args&&... args) { return OpTy::create(*this, loc, std::forward<Args>(args)...); }
  Operation* clone(Operation& op, BlockAndValueMapping& mapper) { return insert(op.clone(mapper)); }
  Operation* clone(Operation& op) { return insert(op.clone()); }
  Block* createBlock(Region* parent);

  // types
  FloatType getF16Type() const;
  FloatType getBF16Type() const;
  FloatType getF32Type() const;
  FloatType getF64Type() const;
  FloatType getF8E4M3FNType() const;
  IndexType getIndexType() const;
  IntegerType getI1Type() const;
  IntegerType getI32Type() const;
  IntegerType getI64Type() const;
  IntegerType getIntegerType(unsigned width) const;
  FunctionType getFunctionType(TypeRange inputs, TypeRange results) const;

  // attributes
  FloatAttr getFloatAttr(Type type, double value) const { return FloatAttr::get(type, value); }
  FloatAttr getF32FloatAttr(float value) const;
  FloatAttr getF64FloatAttr(double value) const;
  IntegerAttr getIntegerAttr(Type type, int64_t value) const { return IntegerAttr::get(type, value); }
  IntegerAttr getIndexAttr(int64_t value) const;
  IntegerAttr getI32IntegerAttr(int32_t value) const;
  IntegerAttr getI64IntegerAttr(int64_t value) const;
  StringAttr getStringAttr(const std::string& s) const { return StringAttr::get(nullptr, s); }
  UnitAttr getUnitAttr() const { return UnitAttr::get(); }

  // affine
  AffineExpr getAffineDimExpr(unsigned position) const { return mlir::getAffineDimExpr(position); }
  AffineExpr getAffineSymbolExpr(unsigned position) const { return mlir::getAffineSymbolExpr(position); }
  AffineExpr getAffineConstantExpr(int64_t constant) const { return mlir::getAffineConstantExpr(constant); }
  AffineMap getDimIdentityMap() const { return AffineMap::getMultiDimIdentityMap(1); }
  AffineMap getMultiDimIdentityMap(unsigned rank) const { return AffineMap::getMultiDimIdentityMap(rank); }
  AffineMap getConstantAffineMap(int64_t v) const { return AffineMap::getConstantMap(v); }

private:
  InsertPoint ip;
};

// ---------------------------------------------------------------------------
// Free functions
// ---------------------------------------------------------------------------
// Perfect nest of constant-bound loops; the body builder gets all ivs and must
// not create the terminators (they exist already).
void buildAffineLoopNest(OpBuilder& builder, Location loc, ArrayRef<int64_t> lbs, ArrayRef<int64_t> ubs,
                         ArrayRef<int64_t> steps,
                         function_ref<void(OpBuilder&, Location, ValueRange)> bodyBuilderFn = nullptr);

// Rewrites an affine.parallel to lower bounds 0 and steps 1; uses of an index
// whose range changed go through an affine.apply (d0 * step + lb) placed at
// the start of the body.
void normalizeAffineParallel(AffineParallelOp op);

// Structural checks: operand/result arity, types of affine accesses against
// their memrefs, terminators, dominance of uses inside a block hierarchy.
LogicalResult verify(Operation* op, std::string* message = nullptr);

// Trivial pass plumbing: the code base's "passes" are module walks.
class Pass {
public:
  virtual ~Pass() = default;
  virtual void runOnOperation(ModuleOp module) = 0;
};
class PassManager {
public:
  explicit PassManager(MLIRContext* = nullptr) {}
  void addPass(std::unique_ptr<Pass> p) { passes.push_back(std::move(p)); }
  LogicalResult run(ModuleOp module) { for (auto& p : passes) p->runOnOperation(module); return success(); }
private:
  std::vector<std::unique_ptr<Pass>> passes;
};

// ---------------------------------------------------------------------------
// Template member definitions
// ---------------------------------------------------------------------------
template <typename OpTy> OpTy Value::getDefiningOp() const { return mlir::dyn_cast<OpTy>(getDefiningOp()); }

template <typename OpTy> OpTy Operation::getParentOfType() const {
  for (Operation* p = getParentOp(); p; p = p->getParentOp())
    if (OpTy::classof(p)) return OpTy(p);
  return OpTy();
}

namespace detail {
template <typename T> struct WalkArg;
template <typename C, typename R, typename A> struct WalkArg<R (C::*)(A) const> { using type = A; };
template <typename C, typename R, typename A> struct WalkArg<R (C::*)(A)> { using type = A; };
template <typename Fn> using walk_arg_t = typename WalkArg<decltype(&std::decay_t<Fn>::operator())>::type;
}  // namespace detail

// walk([](OpTy op) {...}) visits only ops of that type; walk([](Operation* op) {...}) visits all.
template <WalkOrder Order, typename Fn> void Operation::walk(Fn&& fn) {
  using Arg = detail::walk_arg_t<Fn>;
  if constexpr (std::is_same<Arg, Operation*>::value) {
    walk(std::function<void(Operation*)>(fn), Order);
  } else {
    walk([&](Operation* op) { if (Arg::classof(op)) fn(Arg(op)); }, Order);
  }
}
template <WalkOrder Order, typename Fn> void Block::walk(Fn&& fn) {
  std::vector<Operation*> snapshot;
  for (Operation* op = head; op; op = op->getNextNode()) snapshot.push_back(op);
  for (Operation* op : snapshot) op->template walk<Order>(fn);
}

}  // namespace mlir
