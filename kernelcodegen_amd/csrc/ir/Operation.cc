// Values, operations, blocks, regions, builder and op constructors of the
// mini affine IR.
#include <algorithm>

#include "IR/MLIR.h"

namespace mlir {

// ---------------------------------------------------------------------------
// Values
// ---------------------------------------------------------------------------
Value::user_range Value::getUsers() const {
  user_range out;
  for (Operation* u : impl->users)
    if (std::find(out.begin(), out.end(), u) == out.end()) out.push_back(u);
  return out;
}

Block* Value::getParentBlock() const {
  if (impl->ownerBlock) return impl->ownerBlock;
  return impl->definingOp ? impl->definingOp->getBlock() : nullptr;
}

void Value::replaceAllUsesWith(Value newValue) const {
  if (newValue == *this) return;
  std::vector<Operation*> users = getUsers();
  for (Operation* u : users) u->replaceUsesOfWith(*this, newValue);
}

void Value::replaceUsesWithIf(Value newValue, const std::function<bool(Operation*)>& shouldReplace) const {
  if (newValue == *this) return;
  std::vector<Operation*> users = getUsers();
  for (Operation* u : users)
    if (shouldReplace(u)) u->replaceUsesOfWith(*this, newValue);
}

void Value::dump() const {
  if (!impl) { std::cerr << "<<null value>>\n"; return; }
  if (impl->definingOp) impl->definingOp->dump();
  else { std::cerr << "<block argument #" << impl->index << "> : "; impl->type.print(std::cerr); std::cerr << "\n"; }
}

namespace {
void addUse(Value v, Operation* user) { if (v) v.getImpl()->users.push_back(user); }
void dropUse(Value v, Operation* user) {
  if (!v) return;
  auto& us = v.getImpl()->users;
  auto it = std::find(us.begin(), us.end(), user);
  assert(it != us.end() && "use list out of sync");
  us.erase(it);
}
}  // namespace

// ---------------------------------------------------------------------------
// Operation
// ---------------------------------------------------------------------------
const char* getOpName(OpKind kind) {
  switch (kind) {
    case OpKind::Module: return "builtin.module";
    case OpKind::Func: return "func.func";
    case OpKind::Call: return "func.call";
    case OpKind::Return: return "func.return";
    case OpKind::Alloc: return "memref.alloc";
    case OpKind::MemLoad: return "memref.load";
    case OpKind::MemStore: return "memref.store";
    case OpKind::AffineFor: return "affine.for";
    case OpKind::AffineParallel: return "affine.parallel";
    case OpKind::AffineIf: return "affine.if";
    case OpKind::AffineLoad: return "affine.load";
    case OpKind::AffineStore: return "affine.store";
    case OpKind::AffineVectorLoad: return "affine.vector_load";
    case OpKind::AffineVectorStore: return "affine.vector_store";
    case OpKind::AffineApply: return "affine.apply";
    case OpKind::AffineYield: return "affine.yield";
    case OpKind::Constant: return "arith.constant";
    case OpKind::AddF: return "arith.addf";
    case OpKind::SubF: return "arith.subf";
    case OpKind::MulF: return "arith.mulf";
    case OpKind::DivF: return "arith.divf";
    case OpKind::MaxF: return "arith.maxf";
    case OpKind::MinF: return "arith.minf";
    case OpKind::NegF: return "arith.negf";
    case OpKind::CmpF: return "arith.cmpf";
    case OpKind::Bitcast: return "arith.bitcast";
    case OpKind::AddI: return "arith.addi";
    case OpKind::SubI: return "arith.subi";
    case OpKind::MulI: return "arith.muli";
    case OpKind::Select: return "arith.select";
    case OpKind::FPToSI: return "arith.fptosi";
    case OpKind::SIToFP: return "arith.sitofp";
    case OpKind::ExtF: return "arith.extf";
    case OpKind::TruncF: return "arith.truncf";
    case OpKind::Exp: return "math.exp";
    case OpKind::Exp2: return "math.exp2";
    case OpKind::Tanh: return "math.tanh";
    case OpKind::Sqrt: return "math.sqrt";
    case OpKind::Rsqrt: return "math.rsqrt";
    case OpKind::Log: return "math.log";
    case OpKind::PowF: return "math.powf";
    case OpKind::Abs: return "math.absf";
    case OpKind::Barrier: return "gpu.barrier";
    case OpKind::Shuffle: return "gpu.shuffle";
  }
  return "unknown";
}

Operation* Operation::create(OpKind kind, ArrayRef<Value> operands, ArrayRef<Type> resultTypes, unsigned numRegions) {
  Operation* op = new Operation();
  op->kind = kind;
  for (Value v : operands) { assert(v && "null operand"); op->operands.push_back(v); addUse(v, op); }
  for (size_t i = 0; i < resultTypes.size(); ++i) {
    auto* r = new detail::ValueImpl();
    r->type = resultTypes[i];
    r->definingOp = op;
    r->index = (unsigned)i;
    op->results.push_back(r);
  }
  for (unsigned i = 0; i < numRegions; ++i) op->regions.push_back(std::make_unique<Region>(op));
  return op;
}

Operation::~Operation() {
  assert(block == nullptr && "operation destroyed while linked into a block");
  for (Value v : operands) dropUse(v, this);
  operands.clear();
  regions.clear();
  for (auto* r : results) {
    assert(r->users.empty() && "operation destroyed while its results are in use");
    delete r;
  }
}

std::vector<Value> Operation::getResults() const {
  std::vector<Value> out;
  for (auto* r : results) out.push_back(Value(r));
  return out;
}

bool Operation::use_empty() const {
  for (auto* r : results) if (!r->users.empty()) return false;
  return true;
}

void Operation::setOperand(unsigned i, Value v) {
  assert(i < operands.size() && v);
  dropUse(operands[i], this);
  operands[i] = v;
  addUse(v, this);
}

void Operation::setOperands(ValueRange newOperands) {
  for (Value v : operands) dropUse(v, this);
  operands.assign(newOperands.begin(), newOperands.end());
  for (Value v : operands) { assert(v); addUse(v, this); }
}

void Operation::insertOperand(unsigned pos, Value v) {
  assert(pos <= operands.size() && v);
  operands.insert(operands.begin() + pos, v);
  addUse(v, this);
}

void Operation::eraseOperand(unsigned pos) {
  assert(pos < operands.size());
  dropUse(operands[pos], this);
  operands.erase(operands.begin() + pos);
}

void Operation::replaceUsesOfWith(Value from, Value to) {
  for (unsigned i = 0; i < operands.size(); ++i)
    if (operands[i] == from) setOperand(i, to);
}

void Operation::replaceAllUsesWith(Operation* other) {
  assert(other->getNumResults() == getNumResults());
  for (unsigned i = 0; i < getNumResults(); ++i) getResult(i).replaceAllUsesWith(other->getResult(i));
}
void Operation::replaceAllUsesWith(ValueRange values) {
  assert(values.size() == getNumResults());
  for (unsigned i = 0; i < getNumResults(); ++i) getResult(i).replaceAllUsesWith(values[i]);
}

Operation* Operation::getParentOp() const { return block ? block->getParentOp() : nullptr; }
Region* Operation::getParentRegion() const { return block ? block->getParent() : nullptr; }

bool Operation::isBeforeInBlock(Operation* other) const {
  assert(block && block == other->block);
  for (const Operation* p = next; p; p = p->next) if (p == other) return true;
  return false;
}
bool Operation::isAncestor(Operation* other) const {
  for (Operation* p = other; p; p = p->getParentOp()) if (p == this) return true;
  return false;
}
bool Operation::isProperAncestor(Operation* other) const { return other != this && isAncestor(other); }

void Operation::remove() {
  if (!block) return;
  if (prev) prev->next = next; else block->head = next;
  if (next) next->prev = prev; else block->tail = prev;
  prev = next = nullptr;
  block = nullptr;
}

void Operation::dropAllReferences() {
  for (Value v : operands) dropUse(v, this);
  operands.clear();
  for (auto& r : regions)
    for (auto& b : r->getBlocks())
      for (Operation* op = b->head; op; op = op->next) op->dropAllReferences();
}

void Operation::dropAllUses() {
  for (auto* r : results) {
    std::vector<Operation*> users = r->users;
    (void)users;
    assert(r->users.empty() && "dropAllUses on a value that is still used");
  }
}

void Operation::erase() {
  remove();
  // operations nested in the regions may use each other's results in any
  // order; drop every reference first so that destruction order is free
  dropAllReferences();
  delete this;
}

void Operation::moveBefore(Operation* other) { moveBefore(other->block, other); }
void Operation::moveAfter(Operation* other) { moveBefore(other->block, other->next); }
void Operation::moveBefore(Block* b, Operation* before) {
  if (before == this) return;  // already in place
  remove();
  b->insertBefore(this, before);
}

Operation* Operation::clone(BlockAndValueMapping& mapper) {
  std::vector<Value> newOperands;
  for (Value v : operands) newOperands.push_back(mapper.lookupOrDefault(v));
  std::vector<Type> types;
  for (auto* r : results) types.push_back(r->type);
  Operation* c = Operation::create(kind, newOperands, types, (unsigned)regions.size());
  c->attrs = attrs;
  for (unsigned i = 0; i < results.size(); ++i) mapper.map(Value(results[i]), Value(c->results[i]));
  for (unsigned ri = 0; ri < regions.size(); ++ri) {
    for (auto& b : regions[ri]->getBlocks()) {
      Block& nb = c->regions[ri]->emplaceBlock();
      mapper.map(b.get(), &nb);
      for (auto* a : b->arguments) mapper.map(Value(a), nb.addArgument(a->type));
      for (Operation* op = b->head; op; op = op->next) nb.push_back(op->clone(mapper));
    }
  }
  return c;
}

void Operation::walk(const std::function<void(Operation*)>& fn, WalkOrder order) {
  if (order == WalkOrder::PreOrder) fn(this);
  for (auto& r : regions)
    for (auto& b : r->getBlocks()) {
      Operation* op = b->head;
      while (op) {
        Operation* nxt = op->next;  // the callback may erase or move `op`
        op->walk(fn, order);
        op = nxt;
      }
    }
  if (order == WalkOrder::PostOrder) fn(this);
}

void Operation::dump() const { print(std::cerr); std::cerr << "\n"; }

LogicalResult Operation::emitError(const std::string& msg) const {
  std::cerr << "error: " << getName() << ": " << msg << "\n";
  return failure();
}

// ---------------------------------------------------------------------------
// OpList / Block / Region
// ---------------------------------------------------------------------------
OpList::iterator& OpList::iterator::operator++() { op = op->getNextNode(); return *this; }
OpList::iterator& OpList::iterator::operator--() { op = op ? op->getPrevNode() : block->getTerminator(); return *this; }
OpList::iterator OpList::begin() const { return iterator(owner, owner->head); }
size_t OpList::size() const { size_t n = 0; for (Operation* p = owner->head; p; p = p->getNextNode()) ++n; return n; }
bool OpList::empty() const { return owner->head == nullptr; }
Operation& OpList::front() const { return *owner->head; }
Operation& OpList::back() const { return *owner->tail; }
void OpList::push_back(Operation* op) { owner->insertBefore(op, nullptr); }
void OpList::push_front(Operation* op) { owner->insertBefore(op, owner->head); }
void OpList::insert(iterator where, Operation* op) { owner->insertBefore(op, where.getNodePtr()); }
void OpList::splice(iterator where, OpList& other, iterator first, iterator last) {
  (void)other;
  Operation* p = first.getNodePtr();
  Operation* stop = last.getNodePtr();
  while (p != stop) {
    Operation* nxt = p->getNextNode();
    p->moveBefore(owner, where.getNodePtr());
    p = nxt;
  }
}
void OpList::splice(iterator where, OpList& other, iterator first) {
  iterator last = first;
  ++last;
  splice(where, other, first, last);
}

Block::~Block() {
  // drop references first: ops may be used by later ops in the same block
  for (Operation* op = head; op; op = op->next) op->dropAllReferences();
  Operation* op = tail;
  while (op) {
    Operation* p = op->prev;
    op->block = nullptr;
    op->prev = op->next = nullptr;
    delete op;
    op = p;
  }
  head = tail = nullptr;
  for (auto* a : arguments) { assert(a->users.empty()); delete a; }
}

void Block::insertBefore(Operation* op, Operation* before) {
  assert(op->block == nullptr && "operation is already in a block");
  assert(!before || before->block == this);
  op->block = this;
  op->next = before;
  op->prev = before ? before->prev : tail;
  if (op->prev) op->prev->next = op; else head = op;
  if (before) before->prev = op; else tail = op;
}

BlockArgument Block::addArgument(Type type, Location) { return insertArgument((unsigned)arguments.size(), type); }

BlockArgument Block::insertArgument(unsigned pos, Type type) {
  auto* a = new detail::ValueImpl();
  a->type = type;
  a->ownerBlock = this;
  arguments.insert(arguments.begin() + pos, a);
  for (unsigned i = 0; i < arguments.size(); ++i) arguments[i]->index = i;
  return BlockArgument(a);
}

void Block::eraseArgument(unsigned pos) {
  assert(pos < arguments.size() && arguments[pos]->users.empty());
  delete arguments[pos];
  arguments.erase(arguments.begin() + pos);
  for (unsigned i = 0; i < arguments.size(); ++i) arguments[i]->index = i;
}

std::vector<BlockArgument> Block::getArguments() const {
  std::vector<BlockArgument> out;
  for (auto* a : arguments) out.push_back(BlockArgument(a));
  return out;
}

Operation* Block::getParentOp() const { return parent ? parent->getParentOp() : nullptr; }

Block& Region::emplaceBlock() {
  blocks.push_back(std::make_unique<Block>());
  blocks.back()->parent = this;
  return *blocks.back();
}
void Region::push_back(Block* b) {
  b->parent = this;
  blocks.emplace_back(b);
}

// ---------------------------------------------------------------------------
// Builder
// ---------------------------------------------------------------------------
Operation* OpBuilder::insert(Operation* op) {
  if (ip.block) ip.block->insertBefore(op, ip.before);
  return op;
}
Block* OpBuilder::createBlock(Region* parent) {
  Block& b = parent->emplaceBlock();
  setInsertionPointToEnd(&b);
  return &b;
}
FloatType OpBuilder::getF16Type() const { return FloatType(Float16Type::get().getImpl()); }
FloatType OpBuilder::getBF16Type() const { return FloatType(BFloat16Type::get().getImpl()); }
FloatType OpBuilder::getF32Type() const { return FloatType(Float32Type::get().getImpl()); }
FloatType OpBuilder::getF64Type() const { return FloatType(Float64Type::get().getImpl()); }
FloatType OpBuilder::getF8E4M3FNType() const { return FloatType(Float8E4M3FNType::get().getImpl()); }
IndexType OpBuilder::getIndexType() const { return IndexType::get(); }
IntegerType OpBuilder::getI1Type() const { return IntegerType::get(nullptr, 1); }
IntegerType OpBuilder::getI32Type() const { return IntegerType::get(nullptr, 32); }
IntegerType OpBuilder::getI64Type() const { return IntegerType::get(nullptr, 64); }
IntegerType OpBuilder::getIntegerType(unsigned width) const { return IntegerType::get(nullptr, width); }
FunctionType OpBuilder::getFunctionType(TypeRange inputs, TypeRange results) const { return FunctionType::get(nullptr, inputs, results); }
FloatAttr OpBuilder::getF32FloatAttr(float v) const { return FloatAttr::get(getF32Type(), v); }
FloatAttr OpBuilder::getF64FloatAttr(double v) const { return FloatAttr::get(getF64Type(), v); }
IntegerAttr OpBuilder::getIndexAttr(int64_t v) const { return IntegerAttr::get(getIndexType(), v); }
IntegerAttr OpBuilder::getI32IntegerAttr(int32_t v) const { return IntegerAttr::get(getI32Type(), v); }
IntegerAttr OpBuilder::getI64IntegerAttr(int64_t v) const { return IntegerAttr::get(getI64Type(), v); }

// ---------------------------------------------------------------------------
// Op constructors
// ---------------------------------------------------------------------------
ModuleOp ModuleOp::create(Location, Optional<StringRef> name) {
  Operation* op = Operation::create(OpKind::Module, {}, {}, 1);
  op->getRegion(0).emplaceBlock();
  if (name) op->setAttr("sym_name", StringAttr::get(nullptr, name->str()));
  return ModuleOp(op);
}
Optional<StringRef> ModuleOp::getName() const {
  if (!state->hasAttr("sym_name")) return std::nullopt;
  return StringRef(state->getAttr("sym_name").s);
}
std::string ModuleOp::getSymName() const { return state->getAttr("sym_name").s; }
void ModuleOp::destroy() {
  if (!state) return;
  state->erase();
  state = nullptr;
}

namespace func {
FuncOp FuncOp::create(OpBuilder& b, Location, StringRef name, FunctionType type) {
  Operation* op = Operation::create(OpKind::Func, {}, {}, 1);
  op->setAttr("sym_name", StringAttr::get(nullptr, name.str()));
  op->setAttr("function_type", TypeAttr::get(type));
  b.insert(op);
  return FuncOp(op);
}
void FuncOp::setName(const std::string& n) { state->setAttr("sym_name", StringAttr::get(nullptr, n)); }

CallOp CallOp::create(OpBuilder& b, Location loc, FuncOp callee, ValueRange operands) {
  return create(b, loc, callee.getSymName(), callee.getFunctionType().getResults(), operands);
}
CallOp CallOp::create(OpBuilder& b, Location, StringRef callee, TypeRange results, ValueRange operands) {
  Operation* op = Operation::create(OpKind::Call, ArrayRef<Value>(operands), ArrayRef<Type>(results));
  op->setAttr("callee", StringAttr::get(nullptr, callee.str()));
  b.insert(op);
  return CallOp(op);
}
void CallOp::setCallee(const std::string& n) { state->setAttr("callee", StringAttr::get(nullptr, n)); }

ReturnOp ReturnOp::create(OpBuilder& b, Location, ValueRange operands) {
  Operation* op = Operation::create(OpKind::Return, ArrayRef<Value>(operands), {});
  b.insert(op);
  return ReturnOp(op);
}
}  // namespace func

namespace memref {
AllocOp AllocOp::create(OpBuilder& b, Location, MemRefType type) {
  Operation* op = Operation::create(OpKind::Alloc, {}, ArrayRef<Type>(type));
  b.insert(op);
  return AllocOp(op);
}
LoadOp LoadOp::create(OpBuilder& b, Location, Value memref, ValueRange indices) {
  std::vector<Value> ops{memref};
  ops.insert(ops.end(), indices.begin(), indices.end());
  Operation* op = Operation::create(OpKind::MemLoad, ops, ArrayRef<Type>(memref.getType().cast<MemRefType>().getElementType()));
  b.insert(op);
  return LoadOp(op);
}
ValueRange LoadOp::getIndices() const { return ValueRange(std::vector<Value>(state->getOperands().begin() + 1, state->getOperands().end())); }
StoreOp StoreOp::create(OpBuilder& b, Location, Value value, Value memref, ValueRange indices) {
  std::vector<Value> ops{value, memref};
  ops.insert(ops.end(), indices.begin(), indices.end());
  Operation* op = Operation::create(OpKind::MemStore, ops, {});
  b.insert(op);
  return StoreOp(op);
}
ValueRange StoreOp::getIndices() const { return ValueRange(std::vector<Value>(state->getOperands().begin() + 2, state->getOperands().end())); }
}  // namespace memref

AffineYieldOp AffineYieldOp::create(OpBuilder& b, Location, ValueRange operands) {
  Operation* op = Operation::create(OpKind::AffineYield, ArrayRef<Value>(operands), {});
  b.insert(op);
  return AffineYieldOp(op);
}

AffineForOp AffineForOp::create(OpBuilder& b, Location loc, int64_t lb, int64_t ub, int64_t step, ValueRange iterArgs,
                                BodyBuilderFn bodyBuilder) {
  return create(b, loc, {}, AffineMap::getConstantMap(lb), {}, AffineMap::getConstantMap(ub), step, iterArgs, bodyBuilder);
}

AffineForOp AffineForOp::create(OpBuilder& b, Location loc, ValueRange lbOperands, AffineMap lbMap, ValueRange ubOperands,
                                AffineMap ubMap, int64_t step, ValueRange iterArgs, BodyBuilderFn bodyBuilder) {
  assert(step > 0 && "affine.for needs a positive step");
  assert(lbMap.getNumInputs() == lbOperands.size() && ubMap.getNumInputs() == ubOperands.size());
  std::vector<Value> ops(lbOperands.begin(), lbOperands.end());
  ops.insert(ops.end(), ubOperands.begin(), ubOperands.end());
  ops.insert(ops.end(), iterArgs.begin(), iterArgs.end());
  Operation* op = Operation::create(OpKind::AffineFor, ops, ArrayRef<Type>(iterArgs.getTypes()), 1);
  op->setAttr("lower_bound", AffineMapAttr::get(lbMap));
  op->setAttr("upper_bound", AffineMapAttr::get(ubMap));
  op->setAttr("step", IntegerAttr::get(IndexType::get(), step));
  op->setAttr("num_lb_operands", IntegerAttr::get(IndexType::get(), (int64_t)lbOperands.size()));
  op->setAttr("num_ub_operands", IntegerAttr::get(IndexType::get(), (int64_t)ubOperands.size()));
  Block& body = op->getRegion(0).emplaceBlock();
  Value iv = body.addArgument(IndexType::get());
  std::vector<Value> regionArgs;
  for (Value v : iterArgs) regionArgs.push_back(body.addArgument(v.getType()));
  b.insert(op);
  OpBuilder::InsertionGuard guard(b);
  b.setInsertionPointToStart(&body);
  if (bodyBuilder) bodyBuilder(b, loc, iv, ValueRange(regionArgs));
  else if (iterArgs.empty()) AffineYieldOp::create(b, loc);
  return AffineForOp(op);
}

std::vector<BlockArgument> AffineForOp::getRegionIterArgs() const {
  auto args = getBody()->getArguments();
  return std::vector<BlockArgument>(args.begin() + 1, args.end());
}
unsigned AffineForOp::getNumIterOperands() const { return state->getNumResults(); }
ValueRange AffineForOp::getIterOperands() const {
  auto& ops = state->getOperands();
  return ValueRange(std::vector<Value>(ops.end() - getNumIterOperands(), ops.end()));
}
ValueRange AffineForOp::getLowerBoundOperands() const {
  auto& ops = state->getOperands();
  return ValueRange(std::vector<Value>(ops.begin(), ops.begin() + state->getAttr("num_lb_operands").i));
}
ValueRange AffineForOp::getUpperBoundOperands() const {
  auto& ops = state->getOperands();
  const int64_t nl = state->getAttr("num_lb_operands").i, nu = state->getAttr("num_ub_operands").i;
  return ValueRange(std::vector<Value>(ops.begin() + nl, ops.begin() + nl + nu));
}
void AffineForOp::setLowerBound(ValueRange operands, AffineMap map) {
  assert(map.getNumInputs() == operands.size() && map.getNumResults() >= 1);
  std::vector<Value> ops(operands.begin(), operands.end());
  ValueRange ub = getUpperBoundOperands(), it = getIterOperands();
  ops.insert(ops.end(), ub.begin(), ub.end());
  ops.insert(ops.end(), it.begin(), it.end());
  state->setOperands(ops);
  state->setAttr("lower_bound", AffineMapAttr::get(map));
  state->setAttr("num_lb_operands", IntegerAttr::get(IndexType::get(), (int64_t)operands.size()));
}
void AffineForOp::setUpperBound(ValueRange operands, AffineMap map) {
  assert(map.getNumInputs() == operands.size() && map.getNumResults() >= 1);
  ValueRange lb = getLowerBoundOperands(), it = getIterOperands();
  std::vector<Value> ops(lb.begin(), lb.end());
  ops.insert(ops.end(), operands.begin(), operands.end());
  ops.insert(ops.end(), it.begin(), it.end());
  state->setOperands(ops);
  state->setAttr("upper_bound", AffineMapAttr::get(map));
  state->setAttr("num_ub_operands", IntegerAttr::get(IndexType::get(), (int64_t)operands.size()));
}
void AffineForOp::setStep(int64_t s) {
  assert(s > 0);
  state->setAttr("step", IntegerAttr::get(IndexType::get(), s));
}

AffineParallelOp AffineParallelOp::create(OpBuilder& b, Location loc, ArrayRef<int64_t> lbs, ArrayRef<int64_t> ubs,
                                          ArrayRef<int64_t> steps) {
  assert(lbs.size() == ubs.size() && (steps.empty() || steps.size() == ubs.size()));
  Operation* op = Operation::create(OpKind::AffineParallel, {}, {}, 1);
  std::vector<int64_t> st = steps.empty() ? std::vector<int64_t>(ubs.size(), 1) : steps.vec();
  op->setAttr("lower_bounds", getIntArrayAttr(lbs));
  op->setAttr("upper_bounds", getIntArrayAttr(ubs));
  op->setAttr("steps", getIntArrayAttr(st));
  Block& body = op->getRegion(0).emplaceBlock();
  for (size_t i = 0; i < ubs.size(); ++i) body.addArgument(IndexType::get());
  b.insert(op);
  OpBuilder::InsertionGuard guard(b);
  b.setInsertionPointToStart(&body);
  AffineYieldOp::create(b, loc);
  return AffineParallelOp(op);
}
AffineParallelOp AffineParallelOp::create(OpBuilder& b, Location loc, TypeRange resultTypes, ArrayRef<int> reductions,
                                          ArrayRef<int64_t> ranges) {
  assert(resultTypes.empty() && reductions.empty() && "reductions are not supported");
  std::vector<int64_t> lbs(ranges.size(), 0);
  return create(b, loc, lbs, ranges, {});
}
std::vector<Value> AffineParallelOp::getIVs() const {
  std::vector<Value> out;
  for (auto a : getBody()->getArguments()) out.push_back(a);
  return out;
}
Optional<SmallVector<int64_t>> AffineParallelOp::getConstantRanges() const {
  SmallVector<int64_t> out;
  auto lbs = getConstantLowerBounds(), ubs = getConstantUpperBounds();
  for (size_t i = 0; i < ubs.size(); ++i) out.push_back(ubs[i] - lbs[i]);
  return out;
}
void AffineParallelOp::setBounds(ArrayRef<int64_t> lbs, ArrayRef<int64_t> ubs, ArrayRef<int64_t> steps) {
  state->setAttr("lower_bounds", getIntArrayAttr(lbs));
  state->setAttr("upper_bounds", getIntArrayAttr(ubs));
  state->setAttr("steps", getIntArrayAttr(steps));
}

AffineIfOp AffineIfOp::create(OpBuilder& b, Location loc, IntegerSet set, ValueRange operands, bool withElseRegion) {
  assert(set.getNumInputs() == operands.size());
  Operation* op = Operation::create(OpKind::AffineIf, ArrayRef<Value>(operands), {}, 2);
  op->setAttr("condition", IntegerSetAttr::get(set));
  Block& thenB = op->getRegion(0).emplaceBlock();
  b.insert(op);
  OpBuilder::InsertionGuard guard(b);
  b.setInsertionPointToStart(&thenB);
  AffineYieldOp::create(b, loc);
  if (withElseRegion) {
    Block& elseB = op->getRegion(1).emplaceBlock();
    b.setInsertionPointToStart(&elseB);
    AffineYieldOp::create(b, loc);
  }
  return AffineIfOp(op);
}
void AffineIfOp::setConditional(IntegerSet s, ValueRange operands) {
  assert(s.getNumInputs() == operands.size());
  state->setOperands(operands);
  setIntegerSet(s);
}

AffineApplyOp AffineApplyOp::create(OpBuilder& b, Location, AffineMap map, ValueRange operands) {
  assert(map.getNumResults() == 1 && map.getNumInputs() == operands.size());
  Operation* op = Operation::create(OpKind::AffineApply, ArrayRef<Value>(operands), ArrayRef<Type>(IndexType::get()));
  op->setAttr("map", AffineMapAttr::get(map));
  b.insert(op);
  return AffineApplyOp(op);
}

namespace {
Operation* makeLoad(OpBuilder& b, OpKind kind, Type resultType, Value memref, AffineMap map, ValueRange mapOperands) {
  auto mt = memref.getType().dyn_cast<MemRefType>();
  assert(mt && "affine access needs a memref");
  assert(map.getNumResults() == (unsigned)mt.getRank() && map.getNumInputs() == mapOperands.size() &&
         "access map does not match the memref rank or the operand count");
  std::vector<Value> ops{memref};
  ops.insert(ops.end(), mapOperands.begin(), mapOperands.end());
  Operation* op = Operation::create(kind, ops, ArrayRef<Type>(resultType));
  op->setAttr("map", AffineMapAttr::get(map));
  b.insert(op);
  return op;
}
Operation* makeStore(OpBuilder& b, OpKind kind, Value value, Value memref, AffineMap map, ValueRange mapOperands) {
  auto mt = memref.getType().dyn_cast<MemRefType>();
  assert(mt && "affine access needs a memref");
  assert(map.getNumResults() == (unsigned)mt.getRank() && map.getNumInputs() == mapOperands.size() &&
         "access map does not match the memref rank or the operand count");
  std::vector<Value> ops{value, memref};
  ops.insert(ops.end(), mapOperands.begin(), mapOperands.end());
  Operation* op = Operation::create(kind, ops, {});
  op->setAttr("map", AffineMapAttr::get(map));
  b.insert(op);
  return op;
}
}  // namespace

AffineLoadOp AffineLoadOp::create(OpBuilder& b, Location loc, Value memref, ValueRange indices) {
  return create(b, loc, memref, AffineMap::getMultiDimIdentityMap((unsigned)indices.size()), indices);
}
AffineLoadOp AffineLoadOp::create(OpBuilder& b, Location, Value memref, AffineMap map, ValueRange mapOperands) {
  Type elt = memref.getType().cast<MemRefType>().getElementType();
  return AffineLoadOp(makeLoad(b, OpKind::AffineLoad, elt, memref, map, mapOperands));
}
AffineStoreOp AffineStoreOp::create(OpBuilder& b, Location loc, Value value, Value memref, ValueRange indices) {
  return create(b, loc, value, memref, AffineMap::getMultiDimIdentityMap((unsigned)indices.size()), indices);
}
AffineStoreOp AffineStoreOp::create(OpBuilder& b, Location, Value value, Value memref, AffineMap map, ValueRange mapOperands) {
  return AffineStoreOp(makeStore(b, OpKind::AffineStore, value, memref, map, mapOperands));
}
AffineVectorLoadOp AffineVectorLoadOp::create(OpBuilder& b, Location loc, VectorType t, Value memref, ValueRange indices) {
  return create(b, loc, t, memref, AffineMap::getMultiDimIdentityMap((unsigned)indices.size()), indices);
}
AffineVectorLoadOp AffineVectorLoadOp::create(OpBuilder& b, Location, VectorType t, Value memref, AffineMap map,
                                              ValueRange mapOperands) {
  return AffineVectorLoadOp(makeLoad(b, OpKind::AffineVectorLoad, t, memref, map, mapOperands));
}
AffineVectorStoreOp AffineVectorStoreOp::create(OpBuilder& b, Location loc, Value value, Value memref, ValueRange indices) {
  return create(b, loc, value, memref, AffineMap::getMultiDimIdentityMap((unsigned)indices.size()), indices);
}
AffineVectorStoreOp AffineVectorStoreOp::create(OpBuilder& b, Location, Value value, Value memref, AffineMap map,
                                                ValueRange mapOperands) {
  return AffineVectorStoreOp(makeStore(b, OpKind::AffineVectorStore, value, memref, map, mapOperands));
}

namespace arith {
ConstantOp ConstantOp::create(OpBuilder& b, Location loc, Attribute value) {
  assert(value.type && "constant attribute needs a type");
  return create(b, loc, value.type, value);
}
ConstantOp ConstantOp::create(OpBuilder& b, Location, Type type, Attribute value) {
  Operation* op = Operation::create(OpKind::Constant, {}, ArrayRef<Type>(type));
  op->setAttr("value", value);
  b.insert(op);
  return ConstantOp(op);
}
ConstantIndexOp ConstantIndexOp::create(OpBuilder& b, Location loc, int64_t value) {
  return ConstantIndexOp(ConstantOp::create(b, loc, IntegerAttr::get(IndexType::get(), value)).getOperation());
}
ConstantIntOp ConstantIntOp::create(OpBuilder& b, Location loc, int64_t value, unsigned width) {
  return ConstantIntOp(ConstantOp::create(b, loc, IntegerAttr::get(IntegerType::get(nullptr, width), value)).getOperation());
}
ConstantIntOp ConstantIntOp::create(OpBuilder& b, Location loc, int64_t value, Type type) {
  return ConstantIntOp(ConstantOp::create(b, loc, IntegerAttr::get(type, value)).getOperation());
}
ConstantFloatOp ConstantFloatOp::create(OpBuilder& b, Location loc, double value, FloatType type) {
  return ConstantFloatOp(ConstantOp::create(b, loc, FloatAttr::get(type, value)).getOperation());
}

#define KCG_BINARY_CREATE(NS, NAME, KIND)                                                    \
  NS::NAME NS::NAME::create(OpBuilder& b, Location, Value lhs, Value rhs) {                  \
    assert(lhs.getType() == rhs.getType() && "binary op operands must have the same type");  \
    Operation* op = Operation::create(OpKind::KIND, {lhs, rhs}, ArrayRef<Type>(lhs.getType())); \
    b.insert(op);                                                                            \
    return NS::NAME(op);                                                                     \
  }
#define KCG_UNARY_CREATE(NS, NAME, KIND)                                                     \
  NS::NAME NS::NAME::create(OpBuilder& b, Location, Value v) {                               \
    Operation* op = Operation::create(OpKind::KIND, {v}, ArrayRef<Type>(v.getType()));       \
    b.insert(op);                                                                            \
    return NS::NAME(op);                                                                     \
  }
#define KCG_CAST_CREATE(NS, NAME, KIND)                                                      \
  NS::NAME NS::NAME::create(OpBuilder& b, Location, Type t, Value v) {                       \
    Operation* op = Operation::create(OpKind::KIND, {v}, ArrayRef<Type>(t));                 \
    b.insert(op);                                                                            \
    return NS::NAME(op);                                                                     \
  }
}  // namespace arith
KCG_BINARY_CREATE(arith, AddFOp, AddF)
KCG_BINARY_CREATE(arith, SubFOp, SubF)
KCG_BINARY_CREATE(arith, MulFOp, MulF)
KCG_BINARY_CREATE(arith, DivFOp, DivF)
KCG_BINARY_CREATE(arith, MaxFOp, MaxF)
KCG_BINARY_CREATE(arith, MinFOp, MinF)
KCG_BINARY_CREATE(arith, AddIOp, AddI)
KCG_BINARY_CREATE(arith, SubIOp, SubI)
KCG_BINARY_CREATE(arith, MulIOp, MulI)
KCG_UNARY_CREATE(arith, NegFOp, NegF)
KCG_CAST_CREATE(arith, BitcastOp, Bitcast)
KCG_CAST_CREATE(arith, FPToSIOp, FPToSI)
KCG_CAST_CREATE(arith, SIToFPOp, SIToFP)
KCG_CAST_CREATE(arith, ExtFOp, ExtF)
KCG_CAST_CREATE(arith, TruncFOp, TruncF)
KCG_UNARY_CREATE(math, ExpOp, Exp)
KCG_UNARY_CREATE(math, Exp2Op, Exp2)
KCG_UNARY_CREATE(math, TanhOp, Tanh)
KCG_UNARY_CREATE(math, SqrtOp, Sqrt)
KCG_UNARY_CREATE(math, RsqrtOp, Rsqrt)
KCG_UNARY_CREATE(math, LogOp, Log)
KCG_UNARY_CREATE(math, AbsOp, Abs)
KCG_BINARY_CREATE(math, PowFOp, PowF)
#undef KCG_BINARY_CREATE
#undef KCG_UNARY_CREATE
#undef KCG_CAST_CREATE

namespace arith {
CmpFOp CmpFOp::create(OpBuilder& b, Location, CmpFPredicate pred, Value lhs, Value rhs) {
  Operation* op = Operation::create(OpKind::CmpF, {lhs, rhs}, ArrayRef<Type>(IntegerType::get(nullptr, 1)));
  op->setAttr("predicate", IntegerAttr::get(IntegerType::get(nullptr, 64), (int64_t)pred));
  b.insert(op);
  return CmpFOp(op);
}
SelectOp SelectOp::create(OpBuilder& b, Location, Value cond, Value t, Value f) {
  assert(t.getType() == f.getType());
  Operation* op = Operation::create(OpKind::Select, {cond, t, f}, ArrayRef<Type>(t.getType()));
  b.insert(op);
  return SelectOp(op);
}
}  // namespace arith

namespace gpu {
BarrierOp BarrierOp::create(OpBuilder& b, Location) {
  Operation* op = Operation::create(OpKind::Barrier, {}, {});
  b.insert(op);
  return BarrierOp(op);
}
ShuffleOp ShuffleOp::create(OpBuilder& b, Location, Value value, Value offset, Value width, ShuffleMode mode) {
  Operation* op = Operation::create(OpKind::Shuffle, {value, offset, width},
                                    {value.getType(), Type(IntegerType::get(nullptr, 1))});
  op->setAttr("mode", IntegerAttr::get(IntegerType::get(nullptr, 64), (int64_t)mode));
  b.insert(op);
  return ShuffleOp(op);
}
ShuffleOp ShuffleOp::create(OpBuilder& b, Location loc, Value value, int32_t offset, int32_t width, ShuffleMode mode) {
  Value off = arith::ConstantIntOp::create(b, loc, offset, 32).getResult();
  Value w = arith::ConstantIntOp::create(b, loc, width, 32).getResult();
  return create(b, loc, value, off, w, mode);
}
}  // namespace gpu

// ---------------------------------------------------------------------------
// Free functions
// ---------------------------------------------------------------------------
void buildAffineLoopNest(OpBuilder& builder, Location loc, ArrayRef<int64_t> lbs, ArrayRef<int64_t> ubs,
                         ArrayRef<int64_t> steps, function_ref<void(OpBuilder&, Location, ValueRange)> bodyBuilderFn) {
  assert(lbs.size() == ubs.size() && lbs.size() == steps.size());
  OpBuilder::InsertionGuard guard(builder);
  std::vector<Value> ivs;
  if (lbs.empty()) {
    if (bodyBuilderFn) bodyBuilderFn(builder, loc, ValueRange(ivs));
    return;
  }
  for (size_t i = 0; i < lbs.size(); ++i) {
    AffineForOp loop = AffineForOp::create(builder, loc, lbs[i], ubs[i], steps[i]);
    ivs.push_back(loop.getInductionVar());
    builder.setInsertionPointToStart(loop.getBody());
  }
  if (bodyBuilderFn) bodyBuilderFn(builder, loc, ValueRange(ivs));
}

void normalizeAffineParallel(AffineParallelOp op) {
  auto lbs = op.getConstantLowerBounds(), ubs = op.getConstantUpperBounds();
  auto steps = op.getSteps();
  bool normal = true;
  for (size_t i = 0; i < ubs.size(); ++i) if (lbs[i] != 0 || steps[i] != 1) normal = false;
  if (normal) return;
  OpBuilder b = OpBuilder::atBlockBegin(op.getBody());
  std::vector<int64_t> newLbs(ubs.size(), 0), newUbs(ubs.size()), newSteps(ubs.size(), 1);
  auto ivs = op.getIVs();
  for (size_t i = 0; i < ubs.size(); ++i) {
    newUbs[i] = (ubs[i] - lbs[i] + steps[i] - 1) / steps[i];
    if (lbs[i] == 0 && steps[i] == 1) continue;
    AffineExpr e = getAffineDimExpr(0) * steps[i] + lbs[i];
    AffineApplyOp apply = AffineApplyOp::create(b, Location(), AffineMap::get(1, 0, e), ValueRange(ivs[i]));
    ivs[i].replaceUsesWithIf(apply.getResult(), [&](Operation* user) { return user != apply.getOperation(); });
  }
  op.setBounds(newLbs, newUbs, newSteps);
}

}  // namespace mlir
