// gfx950 kernel families: parameterised HIP source for the operators the
// optimizers schedule.  The HIP backend turns a scheduled function into a
// KernelSpec (shapes and dtypes from the memref types, tile sizes from the
// optimizer's config map) and asks the family for source text plus the launch
// geometry.  The reference's backend (src/Backend/CUDA.cc) prints one CUDA
// statement per affine op instead; here the tile/split/reorder decisions select
// and size a hand-shaped CDNA4 kernel.
#pragma once

#include <cstdint>
#include <map>
#include <string>

#include "Backend/HIP.h"

namespace KernelCodeGen {
namespace hipgen {

struct KernelSpec {
  std::string family;                      // "layernorm", "elementwise", "gemm_f32", "gemm_bf16", ...
  std::string name;                        // kernel symbol, "kernel0", ...
  std::map<std::string, int64_t> p;        // integer parameters (shapes, tiles, flags)
  std::map<std::string, double> f;         // floating parameters (eps, scale)
  std::map<std::string, std::string> s;    // string parameters (element types)

  int64_t get(const std::string& key, int64_t dflt) const {
    auto it = p.find(key);
    return it == p.end() ? dflt : it->second;
  }
  bool has(const std::string& key) const { return p.count(key) != 0; }
};

using KernelCodeGen::KernelLaunchInfo;

// Text every emitted translation unit starts with (types, wave reductions,
// GELU, tile mapping).
const std::string& prelude();

// Appends nothing itself: returns the kernel text for `spec` in `src` (without
// the prelude) and fills `info`.  Missing tile parameters are chosen for
// gfx950; the chosen values are written back into `spec.p`.  On failure
// returns false with a message in `err`.
bool emitKernel(KernelSpec& spec, std::string& src, KernelLaunchInfo& info, std::string& err);

}  // namespace hipgen
}  // namespace KernelCodeGen
