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

// Builds the graph and owns the graph module.
struct ComputeDAG {
  ComputeDAG(mlir::OpBuilder& builder_) : builder(builder_) {}
  ComputeDAG() = default;

  template <typename OperatorType, typename... Args>
  mlir::Value create(Args&&... args) {
    return OperatorType::build(this, std::forward<Args>(args)...);
  }

  void dump(const std::string& info = "") {
    if (KCGLog::level == Log::Release) return;
    llvm::errs() << "-----------------------------------------------------------\n";
    llvm::errs() << "           " << info << "\n";
    llvm::errs() << "-----------------------------------------------------------\n";
    module->dump();
    if (mlir::failed(mlir::verify(module))) {
      module->emitError("graph verification error");
      assert(false);
    }
  }

  mlir::OpBuilder builder;
  mlir::ModuleOp module;
};

// "float32", "float64", "float16", "bfloat16", "float8_e4m3", "int64", "int32",
// "int16", "index", "bool"; a null type for anything else.
mlir::Type getDType(mlir::OpBuilder& builder, const std::string& dtype);
// Inverse of getDType; "" for a type without a name.
std::string toStr(mlir::Type type);

template <typename T>
struct Operator {
  template <typename... Args>
  static mlir::Value build(ComputeDAG* graph, Args&&... args) {
    return T::build(graph, std::forward<Args>(args)...);
  }
};

struct PlaceHolder : Operator<PlaceHolder> {
  static mlir::Value build(ComputeDAG* graph, const std::vector<int64_t>& shapes, const std::string& dtype);
};

struct Matmul : Operator<Matmul> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value A, mlir::Value B, const std::string& dtype = {""});
};

struct Relu : Operator<Relu> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, MemorySpace ms, const std::string& dtype = {""});
};

struct BatchedMatmul : Operator<BatchedMatmul> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value A, Layout layoutA, mlir::Value B, Layout layoutB,
                           const std::string& dtype = {""});
};

// Softmax over the last axis.
struct Softmax : Operator<Softmax> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, int axis = -1, MemorySpace ms = MemorySpace::global,
                           const std::string& dtype = {""});
};

struct Transpose : Operator<Transpose> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input);
};

struct Binary : Operator<Binary> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value A, mlir::Value B, std::string operation,
                           MemorySpace ms = MemorySpace::global, const std::string& dtype = {""});
  static mlir::Value add(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static mlir::Value mul(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static mlir::Value div(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static mlir::Value sub(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static mlir::Value pow(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static mlir::Value equal(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static mlir::Value greater(mlir::OpBuilder& builder, mlir::Value elem_1, mlir::Value elem_2);
  static std::map<std::string, std::function<mlir::Value(mlir::OpBuilder&, mlir::Value, mlir::Value)>> operationMap;
};

struct ElementWise : Operator<ElementWise> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, std::string operation, MemorySpace ms,
                           const std::string& dtype = {""});
  static mlir::Value tanh(mlir::OpBuilder& builder, mlir::Value elem, mlir::Type type);
  static mlir::Value sqrt(mlir::OpBuilder& builder, mlir::Value elem, mlir::Type type);
  static mlir::Value log(mlir::OpBuilder& builder, mlir::Value elem, mlir::Type type);
  static mlir::Value relu(mlir::OpBuilder& builder, mlir::Value elem, mlir::Type type);
  static mlir::Value cast(mlir::OpBuilder& builder, mlir::Value elem, mlir::Type type);
  static mlir::Value gelu(mlir::OpBuilder& builder, mlir::Value elem, mlir::Type type);
  static std::map<std::string, std::function<mlir::Value(mlir::OpBuilder&, mlir::Value, mlir::Type)>> operationMap;
};

struct LayerNorm : Operator<LayerNorm> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, mlir::Value scale, mlir::Value bias, int64_t axis,
                           const float& eps = 1e-5, MemorySpace ms = MemorySpace::global, const std::string& dtype_ = {""});
};

struct Gather : Operator<Gather> {
  static mlir::Value build(ComputeDAG* graph, mlir::Value input, mlir::Value indices, const std::int64_t& axis = 0,
                           const std::string& dtype_ = {""});
};

}  // namespace KernelCodeGen
