// kcg_hip_launch_scratch (declared in include/kcg_hip.h): launches a kernel that needs a workspace on a
// scratch array that is part of the library's own device image, so that the call allocates nothing.
// This is the one translation unit of the library that holds device code; it is compiled by hipcc for gfx950.
#include <hip/hip_runtime.h>

#include <atomic>

#include "kcg_hip.h"
#include "runtime/kcg_handles.h"

// The scratch array.  Every GPU the library runs on holds its own copy, at its own address, from the moment
// the device image is loaded until the process ends.  In host code the name below is only a handle for
// hipGetSymbolAddress, never an address to hand to a kernel.
static __device__ __align__(256) unsigned char kcg_scratch[KCG_SCRATCH_MAX_BYTES];

// Counters at the start of a workspace have to be zero when a kernel starts.  The kernels leave them zero, but a
// launch that was aborted may not have; a fill kernel (not a memset node, which a caller's graph capture must
// not record) clears them in front of every launch.
static __global__ void kcg_scratch_clear(unsigned* p, unsigned count) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) p[i] = 0u;
}

namespace {
constexpr int kMaxDevices = 64;
// device address of kcg_scratch, per device ordinal; two threads that set up the same device at the same time both
// store the address hipGetSymbolAddress gives for it
std::atomic<void*> scratchOfDevice[kMaxDevices] = {};
inline int hipErr(hipError_t e) { return e == hipSuccess ? KCG_OK : (KCG_ERR_DOMAIN_HIP | (int)e); }
}  // namespace

extern "C" int kcg_scratch_setup(void) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return hipErr(e);
  if (device < 0 || device >= kMaxDevices) return KCG_ERR_NO_DEVICE;
  if (scratchOfDevice[device].load(std::memory_order_acquire)) return KCG_OK;
  void* ptr = nullptr;
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(kcg_scratch));
  if (e != hipSuccess) return hipErr(e);
  if (!ptr) return KCG_ERR_NO_DEVICE;
  scratchOfDevice[device].store(ptr, std::memory_order_release);
  return KCG_OK;
}

extern "C" int kcg_hip_launch_scratch(kcg_kernel_t kernel, const uint32_t grid[3], const uint32_t block[3],
                                      uint32_t lds_bytes, void* stream, void** args, int num_args, int scratch_arg,
                                      size_t scratch_bytes) {
  constexpr int kMaxArgs = 16;
  if (!kernel || !grid || !block || !args || num_args <= 0 || num_args > kMaxArgs || scratch_arg < 0 || scratch_arg >= num_args)
    return KCG_ERR_INVALID_ARGUMENT;
  for (int i = 0; i < 3; ++i)
    if (grid[i] == 0 || block[i] == 0) return KCG_ERR_INVALID_ARGUMENT;
  if ((uint64_t)block[0] * block[1] * block[2] > 1024) return KCG_ERR_INVALID_ARGUMENT;
  if (scratch_bytes > (size_t)KCG_SCRATCH_MAX_BYTES) return KCG_ERR_SCRATCH_TOO_LARGE;
  int rc = kcg_scratch_setup();
  if (rc != KCG_OK) return rc;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return hipErr(e);
  void* scratch = scratchOfDevice[device].load(std::memory_order_acquire);   // the address on this device; never the array's name
  hipStream_t s = (hipStream_t)stream;
  const unsigned counters = (unsigned)((scratch_bytes < 4096 ? scratch_bytes : 4096) / sizeof(unsigned));
  if (counters) {
    // the launch's own return code: hipGetLastError would also hand over (and clear) an error that an earlier,
    // unrelated call of this thread left behind
    unsigned* base = (unsigned*)scratch;
    unsigned count = counters;
    void* clearArgs[] = {&base, &count};
    e = hipLaunchKernel((const void*)kcg_scratch_clear, dim3((counters + 255) / 256), dim3(256), clearArgs, 0, s);
    if (e != hipSuccess) return hipErr(e);
  }
  void* patched[kMaxArgs];
  for (int i = 0; i < num_args; ++i) patched[i] = args[i];
  patched[scratch_arg] = &scratch;
  return hipErr(hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes, s,
                                      patched, nullptr));
}
