/*
 * kcg_codegen.h -- C ABI over the code generator in libkcg_hip.so, for hosts
 * that cannot include the C++ headers (KernelCodeGen.h and friends).
 *
 * The reference has no foreign-function interface: its users link the C++
 * library kcg_runtime and call KernelCodeGenerator directly (test/test.cc:8-49).
 * Each entry point below names the C++ member it forwards to.
 */
#ifndef KCG_CODEGEN_H
#define KCG_CODEGEN_H

#include <stddef.h>
#include <stdint.h>

#include "kcg_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Source text every emitted translation unit starts with.  Static storage. */
const char *kcg_prelude(void);

/* One kernel of a gfx950 kernel family ("layernorm", "elementwise",
 * "gemm_f32", "gemm_bf16", "gemm_fp8", "fmha_bf16") from explicit parameters: the layer
 * HIPGen() sits on (it replaces the per-op printers of src/Backend/CUDA.cc:386-1149).
 * Integer, floating and string parameters are passed as parallel key/value
 * arrays, like the reference's std::map<std::string,int> config tables
 * (include/KernelCodeGen.h:35-58).  On success *src_out is a malloc'ed string
 * (kernel text without the prelude; free with kcg_free_string) and *info is
 * filled.  On failure returns non-zero and copies a message to err. */
int kcg_emit_kernel(const char *family, const char *name,
                    const char *const *ikeys, const int64_t *ivals, int ni,
                    const char *const *fkeys, const double *fvals, int nf,
                    const char *const *skeys, const char *const *svals, int ns,
                    char **src_out, kcg_launch_info *info, char *err, size_t err_cap);

void kcg_free_string(char *s);

#ifdef __cplusplus
}
#endif
#endif /* KCG_CODEGEN_H */
