"""kernelcodegen_amd -- MI355X (gfx950) native re-implementation of the
KernelCodeGen hot path: operator builders, affine rewrite passes, a HIP
emitter and a C-ABI runtime over hipRTC/hipModule.  This package is the thin
Python host layer over libkcg_hip.so; all work happens in the library."""
from ._lib import lib, KcgError, LaunchInfo  # noqa: F401
from .runtime import (emit_kernel, prelude, compile_source, Module, Kernel,  # noqa: F401
                      compile_to_code)
