// CPU execution of IR functions: the naive nests the Frontend emits
// (func.state = "cpu") and the GPU schedules the optimizers produce
// (func.state = "gpu": affine.parallel grid { affine.parallel block { ... } }).
//
// The reference declares a CPU lowering (Rewriter::loweringAffineDialect,
// include/Optimizer/Rewriter.h:236) but never implements it
// (src/Optimizer/Rewriter.cc:1615-1622).  This interpreter gives the IR an
// executable meaning on the host: scalar code runs op by op with the rounding of
// its element type; a block-level affine.parallel runs all its threads in
// lock-step (every operation is evaluated for all active threads before the
// next one starts), which makes gpu.barrier a no-op and gives gpu.shuffle its
// cross-lane meaning.  It is a verification tool for rewrites and schedules,
// not a fast path.
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "IR/MLIR.h"

namespace KernelCodeGen {

// Dense row-major tensor on the host.  Values are held as doubles that are
// always exactly representable in the element type.
struct HostTensor {
  std::vector<int64_t> shape;
  mlir::Type elementType;
  std::vector<double> data;
  int64_t numElements() const { int64_t n = 1; for (auto d : shape) n *= d; return n; }
};

class Interpreter {
public:
  // Wave width used by gpu.shuffle segments and reported in diagnostics.
  explicit Interpreter(mlir::ModuleOp module) : module(module) {}

  // Runs one function.  `args` are bound to the entry block arguments (shapes
  // and element types must match); returns the tensors the function returns
  // (an argument returned by the function is returned by value).
  // Throws std::runtime_error on malformed IR or out-of-bounds accesses.
  std::vector<HostTensor> run(mlir::func::FuncOp func, std::vector<HostTensor>& args);

  // Runs the module-level graph: every memref.alloc at module scope is a
  // placeholder, bound in order to `placeholders` (missing ones are zero-filled),
  // except the result buffers the Frontend creates itself (tagged kcg.result),
  // which start at zero; every func.call is executed in order.
  // Returns the value of each call result, in call order.
  std::vector<HostTensor> runGraph(std::vector<HostTensor>& placeholders);

  // Statistics of the last run.
  int64_t barriersExecuted = 0;
  int64_t outOfBoundsChecks = 0;
  // Threads of a workgroup run in lock-step here, so gpu.barrier orders nothing and a
  // schedule that lacks one still computes the right values. This counts what would
  // race on the GPU: an element of shared memory written by one thread and read or
  // overwritten (with another value) by a different thread with no barrier between,
  // and a barrier that only part of the workgroup reaches. firstHazard names the first.
  int64_t sharedHazards = 0;
  std::string firstHazard;

private:
  mlir::ModuleOp module;
};

// Rounds `v` to the nearest value of `type` (ties to even); integers truncate.
double roundToType(double v, mlir::Type type);

}  // namespace KernelCodeGen
