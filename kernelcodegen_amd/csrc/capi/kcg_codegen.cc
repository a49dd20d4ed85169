// C facade over the code generator (declared in include/kcg_codegen.h).
#include "kcg_codegen.h"

#include <cstdlib>
#include <cstring>
#include <string>

#include "backend/KernelFamilies.h"

using namespace KernelCodeGen;

namespace {
void copyErr(const std::string& msg, char* err, size_t cap) {
  if (!err || cap == 0) return;
  size_t n = msg.size() < cap - 1 ? msg.size() : cap - 1;
  memcpy(err, msg.data(), n);
  err[n] = '\0';
}

char* dupString(const std::string& s) {
  char* p = (char*)malloc(s.size() + 1);
  if (p) memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

void fillInfo(const hipgen::KernelLaunchInfo& in, kcg_launch_info* out) {
  memset(out, 0, sizeof *out);
  strncpy(out->name, in.name.c_str(), sizeof(out->name) - 1);
  for (int i = 0; i < 3; ++i) {
    out->grid[i] = in.grid[i];
    out->block[i] = in.block[i];
  }
  out->lds_bytes = in.ldsBytes;
  out->num_args = in.numArgs;
  out->num_scalars = in.numScalars;
  out->flops = in.flops;
  out->bytes = in.bytes;
}
}  // namespace

extern "C" {

const char* kcg_prelude(void) { return hipgen::prelude().c_str(); }

int kcg_emit_kernel(const char* family, const char* name, const char* const* ikeys, const int64_t* ivals, int ni,
                    const char* const* fkeys, const double* fvals, int nf, const char* const* skeys,
                    const char* const* svals, int ns, char** src_out, kcg_launch_info* info, char* err,
                    size_t err_cap) {
  if (err && err_cap) err[0] = '\0';
  if (!family || !name || !src_out || !info || ni < 0 || nf < 0 || ns < 0 || (ni && (!ikeys || !ivals)) ||
      (nf && (!fkeys || !fvals)) || (ns && (!skeys || !svals))) {
    copyErr("invalid argument", err, err_cap);
    return KCG_ERR_INVALID_ARGUMENT;
  }
  *src_out = nullptr;
  try {
    hipgen::KernelSpec spec;
    spec.family = family;
    spec.name = name;
    for (int i = 0; i < ni; ++i) spec.p[ikeys[i]] = ivals[i];
    for (int i = 0; i < nf; ++i) spec.f[fkeys[i]] = fvals[i];
    for (int i = 0; i < ns; ++i) spec.s[skeys[i]] = svals[i];
    std::string src, msg;
    hipgen::KernelLaunchInfo li;
    if (!hipgen::emitKernel(spec, src, li, msg)) {
      copyErr(msg, err, err_cap);
      return KCG_ERR_INVALID_ARGUMENT;
    }
    char* out = dupString(src);
    if (!out) return KCG_ERR_OUT_OF_HOST_MEMORY;
    *src_out = out;
    fillInfo(li, info);
    return KCG_OK;
  } catch (const std::exception& e) {
    copyErr(e.what(), err, err_cap);
    return KCG_ERR_INVALID_ARGUMENT;
  }
}

void kcg_free_string(char* s) { free(s); }

}  // extern "C"
