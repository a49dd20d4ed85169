// Lowering of a scheduled function to a gfx950 kernel one statement per operation, the way the reference's
// backend prints CUDA (src/Backend/CUDA.cc:61-1184).  Used for functions no kernel family covers and wherever the
// caller asks for the schedule itself to run (attribute kcg.lowering = "schedule" on the function or the module).
#pragma once

#include <string>

#include "Backend/HIP.h"

namespace KernelCodeGen {
namespace hipgen {

// Kernel text for `f` (grid level = its outer affine.parallel, workgroup level = the affine.parallel inside it);
// parameters are the function's arguments in order, then the buffers it allocates and returns.  Fills the name,
// the launch geometry and the argument count of `info`.  On a construct without a lowering returns false and says
// which in `err`.
bool emitSchedule(mlir::func::FuncOp f, const std::string& kernelName, std::string& text, KernelLaunchInfo& info, std::string& err);

}  // namespace hipgen
}  // namespace KernelCodeGen
