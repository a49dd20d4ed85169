#pragma once
// Collectors over a module (reference: include/Optimizer/Analyzer.h:42-82).

#include <string>
#include <vector>

#include "IR/IR.h"

namespace KernelCodeGen {

// Strict weak orders on op handles by address, for std::set / std::map keys.
struct CompareLoop {
  bool operator()(const mlir::AffineForOp& x, const mlir::AffineForOp& y) const {
    return x.getOperation() < y.getOperation();
  }
};
struct CompareFunc {
  bool operator()(const mlir::func::FuncOp& x, const mlir::func::FuncOp& y) const {
    return x.getOperation() < y.getOperation();
  }
};
struct CompareFuncCall {
  bool operator()(const mlir::func::CallOp& x, const mlir::func::CallOp& y) const {
    return x.getOperation() < y.getOperation();
  }
};

struct Analyzer {
  Analyzer() = default;

  // Loops whose parent is a function or the module.
  static std::vector<mlir::AffineForOp> collectOutermostLoop(mlir::ModuleOp& module);

  // Extent of every dimension of a normalised affine.parallel and their product.
  static std::vector<int64_t> getParallelNumber(mlir::AffineParallelOp parallelLevel, int64_t& totalNumber) {
    totalNumber = 1;
    std::vector<int64_t> result;
    for (unsigned i = 0; i < parallelLevel.getNumDims(); ++i) {
      auto map = parallelLevel.getUpperBoundMap(i);
      assert(map.isSingleConstant());
      totalNumber *= map.getSingleConstantResult();
      result.push_back(map.getSingleConstantResult());
    }
    return result;
  }

  // Functions whose name contains `targetFuncName`, in module order.
  static std::vector<mlir::func::FuncOp> collectFunctions(mlir::ModuleOp& module, const std::string& targetFuncName = {""});
  // All loops of a function in pre-order.
  static std::vector<mlir::AffineForOp> collectFuncLoops(mlir::func::FuncOp funcOp);
  // All calls at any depth of the module, in pre-order.
  static std::vector<mlir::func::CallOp> collectFuncCalls(mlir::ModuleOp& module);
  // The function called exactly `targetFuncName`, or a null handle.
  static mlir::func::FuncOp getTargetFunction(mlir::ModuleOp& module, const std::string& targetFuncName);
  static int getUsersNumber(mlir::Value::user_range users);

  // Last direct child of `father` of type OpType (null handle if none).
  template <typename OpType, typename ParentOpType>
  static OpType getLastOp(ParentOpType father) {
    OpType res;
    for (auto& op : father.getBody()->getOperations())
      if (mlir::isa<OpType>(op)) res = mlir::dyn_cast<OpType>(op);
    return res;
  }
};

}  // namespace KernelCodeGen
