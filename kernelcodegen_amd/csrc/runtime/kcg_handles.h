// Handle types of the C ABI (include/kcg_hip.h), shared by the runtime's translation units.
#pragma once

#include <hip/hip_runtime_api.h>

#include <vector>

struct kcg_kernel_s {
  hipFunction_t fn;
};
struct kcg_module_s {
  hipModule_t mod;
  std::vector<kcg_kernel_s *> kernels;  // handles handed out by get_kernel, released with the module
};
struct kcg_event_s {
  hipEvent_t ev;
};
struct kcg_graph_s {
  hipGraphExec_t exec;
  size_t nodes;
};

// Looks up, once per device, the address of the library's static scratch array on the current device
// (kcg_scratch.hip).  Called by kcg_hip_init and by the first kcg_hip_launch_scratch on a device.
extern "C" int kcg_scratch_setup(void);
