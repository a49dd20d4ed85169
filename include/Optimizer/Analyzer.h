#pragma once
// Collectors over a module (reference: include/Optimizer/Analyzer.h:42-82).

#include <string>
#include <vector>

#include "IR/IR.h"

namespace KernelCodeGen {

// Strict weak order on op handles by the address of the operation, for std::set / std::map keys.  The three
// names are the reference's.
template <typename OpHandle>
struct CompareByOperation {
  bool operator()(const OpHandle& lhs, const OpHandle& rhs) const { return lhs.getOperation() < rhs.getOperation(); }
};
using CompareLoop = CompareByOperation<mlir::AffineForOp>;
using CompareFunc = CompareByOperation<mlir::func::FuncOp>;
using CompareFuncCall = CompareByOperation<mlir::func::CallOp>;

struct Analyzer {
  Analyzer() = default;

  // Loops whose parent is a function or the module.
  static std::vector<mlir::AffineForOp> collectOutermostLoop(mlir::ModuleOp& module);

  // Extent of every dimension of a normalised affine.parallel (constant upper bounds) and, in `totalNumber`,
  // their product.
  static std::vector<int64_t> getParallelNumber(mlir::AffineParallelOp parallelLevel, int64_t& totalNumber) {
    std::vector<int64_t> extents(parallelLevel.getNumDims());
    totalNumber = 1;
    for (unsigned dim = 0; dim < extents.size(); ++dim) {
      const auto bound = parallelLevel.getUpperBoundMap(dim);
      assert(bound.isSingleConstant() && "affine.parallel with a non-constant extent");
      extents[dim] = bound.getSingleConstantResult();
      totalNumber *= extents[dim];
    }
    return extents;
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

  // Last direct child of `father` that is an OpType; a null handle if there is none.
  template <typename OpType, typename ParentOpType>
  static OpType getLastOp(ParentOpType father) {
    OpType last;
    for (auto& child : father.getBody()->getOperations())
      if (auto typed = mlir::dyn_cast<OpType>(child)) last = typed;
    return last;
  }
};

}  // namespace KernelCodeGen
