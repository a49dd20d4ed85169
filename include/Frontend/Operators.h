#pragma once
// Frontend: operator builders.  Each builder emits one func.func that holds the
// operator's naive affine loop nest (tagged func.state = "cpu") plus a
// func.call at the graph's insertion point, and returns the call's result.
// Signatures follow the reference (include/Frontend/Operators.h:17-133).
// Additions: element types "bfloat16" and "float8_e4m3"; a narrower operand is
// extended to the accumulate type `dtype` inside the nest.

#include <functional>
#include <map>
#include <string>
#include <vector>

#include "IR/IR.h"
#include "enum.h"
#include "log.h"

namespace KernelCodeGen {

using loopfunc = std::function<mlir::Value(mlir::OpBuilder&, mlir::Location, mlir::ValueRange, mlir::ValueRange)>;

// Finds the function called `funcName` in `module` or creates it (empty body,
// one entry block argument per input type) at the start of the module.
mlir::func::FuncOp buildFuction(mlir::ModuleOp module, mlir::OpBuilder& builder, const std::string& funcName,
                                const std::vector<mlir::Type>& inputsTypes, const std::vector<mlir::Type>& outputsTypes);

// The graph under construction: a builder positioned in `module`, where every create<Op>() leaves one function
// with the operator's naive nest and one call to it.
struct ComputeDAG {
  ComputeDAG() = default;
  explicit ComputeDAG(mlir::OpBuilder& b) : builder(b) {}

  // create<Matmul>(A, B), create<Relu>(x, MemorySpace::inplace), ...: forwards to the operator's build().
  template <typename OperatorType, typename... Args>
  mlir::Value create(Args&&... args) {
    return OperatorType::build(this, std::forward<Args>(args)...);
  }

  // At Log::Debug: the module's text under a caption, then the verifier (a failure is fatal).
  void dump(const std::string& caption = "") {
    if (!KCGLog::debug()) return;
    const std::string rule(59, '-');
    llvm::errs() << rule << "\n           " << caption << "\n" << rule << "\n";
    module->dump();
    const bool ok = !mlir::failed(mlir::verify(module));
    if (!ok) module->emitError("graph verification error");
    assert(ok && "graph verification error");
  }

  mlir::OpBuilder builder;
  mlir::ModuleOp module;
};

// Element type by name: "float32", "float64", "float16", "bfloat16", "float8_e4m3", "int64", "int32", "int16",
// "index", "bool"; a null type for any other string.  toStr is the inverse ("" for a type without a name).
mlir::Type getDType(mlir::OpBuilder& builder, const std::string& dtype);
std::string toStr(mlir::Type type);

// CRTP base of the operators: Operator<T>::build forwards to T::build.
template <typename T>
struct Operator {
  template <typename... Args>
  static mlir::Value build(ComputeDAG* graph, Args&&... args) {
    return T::build(graph, std::forward<Args>(args)...);
  }
};

// Scalar kernels of Binary and ElementWise, looked up by operation name.
using BinaryScalarFn = std::function<mlir::Value(mlir::OpBuilder&, mlir::Value, mlir::Value)>;
using UnaryScalarFn = std::function<mlir::Value(mlir::OpBuilder&, mlir::Value, mlir::Type)>;

// A graph input: memref<shape x dtype> in global memory.
struct PlaceHolder : Operator<PlaceHolder> {
  static mlir::Value build(ComputeDAG* graph, const std::vector<int64_t>& shape, const std::string& dtype);
};

// C[m][n] = sum_k A[m][k] * B[k][n], both operands row-major; `dtype` names the accumulate type ("" = A's).
struct Matmul : Operator<Matmul> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value lhs, mlir::Value rhs, const std::string& dtype = {""});
  // (scaleA[0] * scaleB[0]) * lhs * rhs: the quantised product, with one fp32 scale per tensor as graph values
  // (placeholders of shape {1}, float32).  Not in the reference, whose element types stop at fp16.
  static mlir::Value build(ComputeDAG* graph, mlir::Value lhs, mlir::Value rhs, mlir::Value scaleLhs, mlir::Value scaleRhs,
                           const std::string& dtype = {""});
};

// max(0, x); with MemorySpace::inplace the input buffer is overwritten and returned.
struct Relu : Operator<Relu> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, MemorySpace space, const std::string& dtype = {""});
};

// Matmul over the two innermost dimensions with leading batch dimensions; either operand may be column-major.
struct BatchedMatmul : Operator<BatchedMatmul> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value lhs, Layout lhsLayout, mlir::Value rhs, Layout rhsLayout,
                           const std::string& dtype = {""});
  // the same with per-tensor fp32 scales as graph values (see Matmul)
  static mlir::Value build(ComputeDAG* graph, mlir::Value lhs, Layout lhsLayout, mlir::Value rhs, Layout rhsLayout,
                           mlir::Value scaleLhs, mlir::Value scaleRhs, const std::string& dtype = {""});
};

// exp(x) / sum exp(x) over the last axis (any other axis is refused, as in the reference).
struct Softmax : Operator<Softmax> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, int axis = -1, MemorySpace space = MemorySpace::global,
                           const std::string& dtype = {""});
};

// Declared for source compatibility; the reference's builder is empty and this one reports "unsupported".
struct Transpose : Operator<Transpose> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input);
};

// Z = X op Y with numpy-style broadcasting; op is one of the keys of operationMap
// ("Add", "Sub", "Mul", "Div", "Pow", "Equal", "Greater").
struct Binary : Operator<Binary> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value lhs, mlir::Value rhs, std::string operation,
                           MemorySpace space = MemorySpace::global, const std::string& dtype = {""});
  static mlir::Value add(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static mlir::Value sub(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static mlir::Value mul(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static mlir::Value div(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static mlir::Value pow(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static mlir::Value equal(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static mlir::Value greater(mlir::OpBuilder& builder, mlir::Value x, mlir::Value y);
  static std::map<std::string, BinaryScalarFn> operationMap;
};

// y = f(x) element by element; f is one of the keys of operationMap
// ("Tanh", "Sqrt", "Log", "Relu", "Cast", "Gelu").
struct ElementWise : Operator<ElementWise> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, std::string operation, MemorySpace space,
                           const std::string& dtype = {""});
  static mlir::Value tanh(mlir::OpBuilder& builder, mlir::Value x, mlir::Type type);
  static mlir::Value sqrt(mlir::OpBuilder& builder, mlir::Value x, mlir::Type type);
  static mlir::Value log(mlir::OpBuilder& builder, mlir::Value x, mlir::Type type);
  static mlir::Value relu(mlir::OpBuilder& builder, mlir::Value x, mlir::Type type);
  static mlir::Value cast(mlir::OpBuilder& builder, mlir::Value x, mlir::Type type);
  static mlir::Value gelu(mlir::OpBuilder& builder, mlir::Value x, mlir::Type type);
  static std::map<std::string, UnaryScalarFn> operationMap;
};

// Normalisation over the dimensions from `axis` on: (x - mean) / sqrt(var + eps) * scale + bias.
struct LayerNorm : Operator<LayerNorm> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, mlir::Value scale, mlir::Value bias, int64_t axis,
                           const float& eps = 1e-5, MemorySpace space = MemorySpace::global,
                           const std::string& dtype = {""});
};

// Rows of `input` along `axis` picked by `indices` (element type "index").
struct Gather : Operator<Gather> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, mlir::Value indices, const std::int64_t& axis = 0,
                           const std::string& dtype = {""});
};

}  // namespace KernelCodeGen
