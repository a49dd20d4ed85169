#include "Optimizer/Analyzer.h"

namespace KernelCodeGen {

using namespace mlir;

std::vector<AffineForOp> Analyzer::collectOutermostLoop(ModuleOp& module) {
  std::vector<AffineForOp> result;
  module.walk<WalkOrder::PreOrder>([&](AffineForOp loop) {
    Operation* parent = loop->getParentOp();
    if (isa<func::FuncOp>(parent) || isa<ModuleOp>(parent)) result.push_back(loop);
  });
  return result;
}

std::vector<func::FuncOp> Analyzer::collectFunctions(ModuleOp& module, const std::string& targetFuncName) {
  std::vector<func::FuncOp> result;
  module.walk<WalkOrder::PreOrder>([&](func::FuncOp f) {
    if (targetFuncName.empty() || f.getSymName().find(targetFuncName) != std::string::npos) result.push_back(f);
  });
  return result;
}

std::vector<AffineForOp> Analyzer::collectFuncLoops(func::FuncOp funcOp) {
  std::vector<AffineForOp> result;
  funcOp.walk<WalkOrder::PreOrder>([&](AffineForOp loop) { result.push_back(loop); });
  return result;
}

std::vector<func::CallOp> Analyzer::collectFuncCalls(ModuleOp& module) {
  std::vector<func::CallOp> result;
  module.walk<WalkOrder::PreOrder>([&](func::CallOp call) { result.push_back(call); });
  return result;
}

func::FuncOp Analyzer::getTargetFunction(ModuleOp& module, const std::string& targetFuncName) {
  func::FuncOp result;
  module.walk<WalkOrder::PreOrder>([&](func::FuncOp f) {
    if (!result && f.getSymName() == targetFuncName) result = f;
  });
  return result;
}

int Analyzer::getUsersNumber(Value::user_range users) { return (int)users.size(); }

}  // namespace KernelCodeGen
