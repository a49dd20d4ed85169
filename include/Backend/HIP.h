#pragma once
// gfx950 HIP backend.  Takes the place of the reference's CUDA pretty-printer
// (include/Backend/CUDA.h:6, src/Backend/CUDA.cc): instead of one C statement
// per affine operation, a scheduled function is recognised (operator, shapes
// and element types from the signature, tile sizes from the schedule) and
// lowered to a kernel shaped for CDNA4: MFMA register tiles fed from padded
// LDS tiles for GEMM, one-pass register-resident rows with wavefront
// reductions for LayerNorm, 128-bit coalesced streams for elementwise maps.

#include <string>
#include <vector>

#include "IR/IR.h"

namespace KernelCodeGen {

// Machine-readable form of the "// grid dims:(..), block dims:(..)" comment the
// reference prints above each kernel (src/Backend/CUDA.cc:1031-1036).
struct KernelLaunchInfo {
  std::string name;               // extern "C" symbol: kernel0, kernel1, ...
  std::string function;           // IR function the kernel implements
  std::string lowering;           // "family <name>" or "schedule"; behind "schedule", in brackets, why a kernel family
                                  // that knows the operator was not used, when that is so
  uint32_t grid[3] = {1, 1, 1};   // x, y, z
  uint32_t block[3] = {1, 1, 1};  // x, y, z
  uint32_t ldsBytes = 0;          // dynamic LDS (static LDS is declared in the source)
  uint32_t numArgs = 0;           // device pointers: function inputs in order, then outputs
  uint32_t numScalars = 0;        // trailing fp32 scalars
  int64_t workspaceBytes = 0;     // > 0: one more pointer behind the outputs, a scratch buffer the workgroups share
                                  // (first 4096 bytes zero before the first launch; launches leave them zero)
  int workspaceArg = -1;          // its position among the pointer arguments
  std::vector<int64_t> argBytes;  // size in bytes of each pointer argument
  std::vector<int> argTypes;      // element type of each pointer argument (KCG_DT_* of kcg_hip.h)
  // What the kernel computes, for a host-side check of its output (KernelCodeGenerator::adaptor): the
  // operator ("gemm", "layernorm", "elementwise", "softmax", "fmha", "binary", "gather"; empty = no check),
  // its integer and floating parameters in the order the adaptor's check routine of that name reads them,
  // the pointer argument that receives the result, and the range the synthetic inputs are drawn from.
  std::string check;
  std::vector<int64_t> checkInts;
  std::vector<double> checkFloats;
  int outputArg = -1;
  double fillLo = -1.0, fillHi = 1.0;
  double flops = 0.0;             // algorithmic flops per launch
  double bytes = 0.0;             // algorithmic HBM bytes per launch
};

// One kernel per scheduled function (func.state = "gpu"), numbered kernel0,
// kernel1, ... in module order, numbering restarting at every call.  Each
// kernel is preceded by the launch-geometry comment.  Functions that are not
// scheduled produce no kernel; when such a function is called from the module body (an operator no
// optimizer has scheduled), its name is appended to `skipped` so that the caller can tell a complete
// translation from a partial one.  On an operator the backend cannot lower the result is empty and
// `error` (when given) says why.
std::string HIPGen(mlir::ModuleOp& module);
std::string HIPGen(mlir::ModuleOp& module, std::vector<KernelLaunchInfo>& infos, std::string* error = nullptr,
                   std::vector<std::string>* skipped = nullptr);

}  // namespace KernelCodeGen
