"""ctypes binding of libkcg_hip.so.  There is no fallback: if the library is
missing or does not load, importing a function from it raises."""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libkcg_hip.so")


class KcgError(RuntimeError):
    def __init__(self, code, what="", log=""):
        self.code = code
        self.log = log
        msg = "%s: %s (code 0x%x)" % (what, strerror(code), code)
        if log:
            msg += "\n" + log
        super().__init__(msg)


class LaunchInfo(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3),
                ("lds_bytes", C.c_uint32), ("num_args", C.c_uint32), ("num_scalars", C.c_uint32),
                ("workspace_bytes", C.c_uint64), ("flops", C.c_double), ("bytes", C.c_double)]

    def as_dict(self):
        return {"name": self.name.decode(), "grid": list(self.grid), "block": list(self.block),
                "lds_bytes": self.lds_bytes, "num_args": self.num_args, "num_scalars": self.num_scalars,
                "workspace_bytes": self.workspace_bytes,
                "flops": self.flops, "bytes": self.bytes}


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is not built; run `python -m kernelcodegen_amd.build`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        _declare(L)
        _lib = L
    return _lib


def strerror(code):
    return lib().kcg_hip_strerror(code).decode()


def check(code, what="", log=""):
    if code != 0:
        raise KcgError(code, what, log)


def _declare(L):
    vp, sz, u32p = C.c_void_p, C.c_size_t, C.POINTER(C.c_uint32)
    cpp = C.POINTER(C.c_char_p)
    L.kcg_hip_strerror.restype = C.c_char_p
    L.kcg_hip_strerror.argtypes = [C.c_int]
    L.kcg_hip_init.argtypes = [C.c_int]
    L.kcg_hip_device_count.argtypes = [C.POINTER(C.c_int)]
    L.kcg_hip_device_name.argtypes = [C.c_int, C.c_char_p, sz]
    L.kcg_hip_compile_to_code.argtypes = [C.c_char_p, cpp, C.c_int, C.POINTER(vp), C.POINTER(sz), C.c_char_p, sz]
    L.kcg_hip_compile_to_code_cached.argtypes = [C.c_char_p, cpp, C.c_int, C.c_int, C.POINTER(vp), C.POINTER(sz),
                                                 C.c_char_p, sz]
    L.kcg_hip_compile_cached.argtypes = [C.c_char_p, cpp, C.c_int, C.POINTER(vp), C.c_char_p, sz]
    L.kcg_hip_cache_dir.argtypes = [C.c_char_p, sz]
    L.kcg_hip_time_rotating.argtypes = [vp, u32p, u32p, C.c_uint32, vp, C.POINTER(C.POINTER(vp)), C.c_int, C.c_int,
                                        C.c_float, C.c_int, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.kcg_hip_launch_sequence.argtypes = [vp, u32p, u32p, C.c_uint32, vp, C.POINTER(C.POINTER(vp)), C.c_int, C.c_int,
                                          C.c_int]
    L.kcg_hip_launch_scratch.argtypes = [vp, u32p, u32p, C.c_uint32, vp, C.POINTER(vp), C.c_int, C.c_int, sz]
    L.kcg_hip_memcpy_d2d.argtypes = [vp, vp, sz]
    L.kcg_dtype_size.argtypes = [C.c_int]
    L.kcg_dtype_size.restype = sz
    L.kcg_host_fill.argtypes = [vp, sz, C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_float, C.c_float, C.c_float]
    L.kcg_host_to_f32.argtypes = [vp, C.POINTER(C.c_float), sz, C.c_int]
    L.kcg_host_from_f32.argtypes = [C.POINTER(C.c_float), vp, sz, C.c_int, C.c_float]
    L.kcg_hip_compiler_info.argtypes = [C.c_char_p, C.c_size_t]
    L.kcg_hip_compiler_info.restype = C.c_int
    L.kcg_hip_free_code.argtypes = [vp]
    L.kcg_hip_free_code.restype = None
    L.kcg_hip_load_code.argtypes = [vp, sz, C.POINTER(vp)]
    L.kcg_hip_compile.argtypes = [C.c_char_p, cpp, C.c_int, C.POINTER(vp), C.c_char_p, sz]
    L.kcg_hip_get_kernel.argtypes = [vp, C.c_char_p, C.POINTER(vp)]
    L.kcg_hip_launch.argtypes = [vp, u32p, u32p, C.c_uint32, vp, C.POINTER(vp)]
    L.kcg_hip_time_launches.argtypes = [vp, u32p, u32p, C.c_uint32, vp, C.POINTER(vp), C.c_int, C.c_int,
                                        C.POINTER(C.c_float)]
    L.kcg_hip_module_destroy.argtypes = [vp]
    L.kcg_hip_malloc.argtypes = [C.POINTER(vp), sz]
    L.kcg_hip_free.argtypes = [vp]
    L.kcg_hip_memcpy_h2d.argtypes = [vp, vp, sz]
    L.kcg_hip_memcpy_d2h.argtypes = [vp, vp, sz]
    L.kcg_hip_memset.argtypes = [vp, C.c_int, sz]
    L.kcg_hip_stream_synchronize.argtypes = [vp]
    L.kcg_hip_device_synchronize.argtypes = []
    L.kcg_hip_stream_create.argtypes = [C.POINTER(vp)]
    L.kcg_hip_stream_destroy.argtypes = [vp]
    L.kcg_hip_graph_begin_capture.argtypes = [vp]
    L.kcg_hip_graph_end_capture.argtypes = [vp, C.POINTER(vp)]
    L.kcg_hip_graph_launch.argtypes = [vp, vp]
    L.kcg_hip_graph_num_nodes.argtypes = [vp, C.POINTER(sz)]
    L.kcg_hip_graph_destroy.argtypes = [vp]
    L.kcg_hip_event_create.argtypes = [C.POINTER(vp)]
    L.kcg_hip_event_record.argtypes = [vp, vp]
    L.kcg_hip_event_synchronize.argtypes = [vp]
    L.kcg_hip_event_elapsed_ms.argtypes = [vp, vp, C.POINTER(C.c_float)]
    L.kcg_hip_event_destroy.argtypes = [vp]
    L.kcg_prelude.restype = C.c_char_p
    L.kcg_emit_kernel.argtypes = [C.c_char_p, C.c_char_p, cpp, C.POINTER(C.c_int64), C.c_int,
                                  cpp, C.POINTER(C.c_double), C.c_int, cpp, cpp, C.c_int,
                                  C.POINTER(vp), C.POINTER(LaunchInfo), C.c_char_p, sz]
    L.kcg_free_string.argtypes = [vp]
    L.kcg_free_string.restype = None


def _declare_generator(L):
    vp, sz = C.c_void_p, C.c_size_t
    cpp = C.POINTER(C.c_char_p)
    i64p = C.POINTER(C.c_int64)
    L.kcg_generator_create.restype = vp
    L.kcg_generator_create.argtypes = [C.c_char_p]
    L.kcg_generator_destroy.argtypes = [vp]
    L.kcg_generator_destroy.restype = None
    L.kcg_generator_create_graph.argtypes = [vp, C.c_char_p]
    L.kcg_generator_error.argtypes = [vp]
    L.kcg_generator_error.restype = C.c_char_p
    L.kcg_generator_set_log_mode.argtypes = [vp, C.c_int]
    L.kcg_generator_set_log_mode.restype = None
    L.kcg_placeholder.argtypes = [vp, i64p, C.c_int, C.c_char_p]
    L.kcg_matmul.argtypes = [vp, C.c_int, C.c_int, C.c_char_p]
    L.kcg_batched_matmul.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_char_p]
    L.kcg_matmul_scaled.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_char_p]
    L.kcg_batched_matmul_scaled.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_char_p]
    L.kcg_softmax.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_char_p]
    L.kcg_relu.argtypes = [vp, C.c_int, C.c_int, C.c_char_p]
    L.kcg_elementwise.argtypes = [vp, C.c_int, C.c_char_p, C.c_int, C.c_char_p]
    L.kcg_binary.argtypes = [vp, C.c_int, C.c_int, C.c_char_p, C.c_int, C.c_char_p]
    L.kcg_layernorm.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_float, C.c_int, C.c_char_p]
    L.kcg_gather.argtypes = [vp, C.c_int, C.c_int, C.c_int64, C.c_char_p]
    L.kcg_add_optimizer.argtypes = [vp, C.c_char_p]
    L.kcg_set_configs.argtypes = [vp, C.c_char_p, C.c_int, C.POINTER(C.c_int), cpp, C.POINTER(C.c_int)]
    L.kcg_optimize.argtypes = [vp]
    L.kcg_get_configs.argtypes = [vp, C.c_char_p]
    L.kcg_get_configs.restype = C.c_char_p
    L.kcg_set_lowering.argtypes = [vp, C.c_char_p]
    L.kcg_set_lowering.restype = C.c_int
    L.kcg_codegen.argtypes = [vp]
    L.kcg_codegen.restype = C.c_char_p
    L.kcg_adaptor.argtypes = [vp, C.c_char_p]
    L.kcg_adaptor.restype = C.c_char_p
    L.kcg_num_kernels.argtypes = [vp]
    L.kcg_kernel_info.argtypes = [vp, C.c_int, C.POINTER(LaunchInfo)]
    L.kcg_kernel_function.argtypes = [vp, C.c_int]
    L.kcg_kernel_function.restype = C.c_char_p
    L.kcg_kernel_lowering.argtypes = [vp, C.c_int]
    L.kcg_kernel_lowering.restype = C.c_char_p
    L.kcg_kernel_arg_bytes.argtypes = [vp, C.c_int, i64p, C.c_int]
    L.kcg_kernel_arg_types.argtypes = [vp, C.c_int, C.POINTER(C.c_int), C.c_int]
    L.kcg_num_skipped.argtypes = [vp]
    L.kcg_skipped_function.argtypes = [vp, C.c_int]
    L.kcg_skipped_function.restype = C.c_char_p
    L.kcg_num_evaluations.argtypes = [vp]
    L.kcg_evaluation.argtypes = [vp, C.c_int, cpp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_float),
                                 C.POINTER(C.c_int), cpp]
    L.kcg_evaluation_config.argtypes = [vp, C.c_int, C.c_char_p]
    L.kcg_evaluate.argtypes = [vp]
    L.kcg_evaluate.restype = C.c_float
    L.kcg_module_plan.argtypes = [vp, C.c_int]
    L.kcg_module_plan.restype = C.c_char_p
    L.kcg_dump.argtypes = [vp, C.c_int]
    L.kcg_dump.restype = C.c_char_p
    L.kcg_verify.argtypes = [vp, C.c_int]
    L.kcg_function_state.argtypes = [vp, C.c_int, C.c_char_p]
    L.kcg_function_state.restype = C.c_char_p
    L.kcg_interpret.argtypes = [vp, C.c_int, C.POINTER(C.POINTER(C.c_float)), i64p, C.c_int, C.POINTER(C.c_float), C.c_int64]
    L.kcg_interpret.restype = C.c_int64
    L.kcg_fmha_map_evaluate.argtypes = [C.c_char_p, i64p, C.c_int, i64p, C.c_int]
    L.kcg_fmha_map_evaluate.restype = C.c_int


_declare_base = _declare


def _declare(L):  # noqa: F811
    _declare_base(L)
    _declare_generator(L)
