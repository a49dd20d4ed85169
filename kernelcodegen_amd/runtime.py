"""Host-side helpers over the C ABI: emit a kernel, compile it with hipRTC (or
pick up a code object built ahead of time), load it, launch it on torch's
current stream.  torch supplies device memory and the stream handle only."""
import ctypes as C
import os

from . import _lib
from ._lib import LaunchInfo, check, lib



def prelude():
    return lib().kcg_prelude().decode()


def _cstr_array(items):
    arr = (C.c_char_p * max(1, len(items)))()
    for i, s in enumerate(items):
        arr[i] = s.encode()
    return arr


DTYPES = {"f32": 0, "bf16": 1, "f8e4m3": 2, "f16": 3, "f64": 4, "i32": 5, "i64": 6, "i16": 7, "i8": 8}
_NUMPY = {0: "float32", 1: "uint16", 2: "uint8", 3: "uint16", 4: "float64", 5: "int32", 6: "int64", 7: "int16", 8: "int8"}
SEED = 0x4B4347


def host_fill(shape, dtype="f32", dist="uniform", stream=0, p0=-1.0, p1=1.0, scale=1.0, seed=SEED):
    """Seeded synthetic operand as a numpy array (bf16 / f16 as uint16 bits, e4m3 as uint8 bits): element i of
    `stream` comes from splitmix64(seed + (stream << 40) + i); uniform(p0, p1) or normal(mean p0, deviation p1)."""
    import numpy as np
    code = DTYPES[dtype]
    out = np.empty(shape, dtype=_NUMPY[code])
    check(lib().kcg_host_fill(out.ctypes.data, out.size, code, {"uniform": 0, "normal": 1}[dist], seed, stream,
                              p0, p1, scale), "kcg_host_fill")
    return out


def host_from_f32(x, dtype, scale=1.0):
    """fp32 array * scale -> bits of `dtype` (round to nearest even; e4m3 saturates at 448)."""
    import numpy as np
    x = np.ascontiguousarray(x, dtype=np.float32)
    code = DTYPES[dtype]
    out = np.empty(x.shape, dtype=_NUMPY[code])
    check(lib().kcg_host_from_f32(x.ctypes.data_as(C.POINTER(C.c_float)), out.ctypes.data, x.size, code, scale),
          "kcg_host_from_f32")
    return out


def host_to_f32(bits, dtype):
    import numpy as np
    bits = np.ascontiguousarray(bits)
    out = np.empty(bits.shape, dtype=np.float32)
    check(lib().kcg_host_to_f32(bits.ctypes.data, out.ctypes.data_as(C.POINTER(C.c_float)), bits.size, DTYPES[dtype]),
          "kcg_host_to_f32")
    return out


def emit_kernel(family, name="kernel0", **params):
    """Returns (kernel text without the prelude, launch-info dict)."""
    ik, iv, fk, fv, sk, sv = [], [], [], [], [], []
    for k, v in params.items():
        if isinstance(v, bool):
            ik.append(k), iv.append(int(v))
        elif isinstance(v, int):
            ik.append(k), iv.append(v)
        elif isinstance(v, float):
            fk.append(k), fv.append(v)
        elif isinstance(v, str):
            sk.append(k), sv.append(v)
        else:
            raise TypeError("parameter %s has unsupported type %r" % (k, type(v)))
    src = C.c_void_p()
    info = LaunchInfo()
    err = C.create_string_buffer(1024)
    ivals = (C.c_int64 * max(1, len(iv)))(*iv)
    fvals = (C.c_double * max(1, len(fv)))(*fv)
    rc = lib().kcg_emit_kernel(family.encode(), name.encode(), _cstr_array(ik), ivals, len(ik),
                               _cstr_array(fk), fvals, len(fk), _cstr_array(sk), _cstr_array(sv), len(sk),
                               C.byref(src), C.byref(info), err, len(err))
    if rc != 0:
        raise _lib.KcgError(rc, "kcg_emit_kernel(%s)" % family, err.value.decode())
    try:
        text = C.string_at(src.value).decode()
    finally:
        lib().kcg_free_string(src)
    return text, info.as_dict()


_compiler = None


def compiler_info():
    """Which hipRTC compiles the kernels (file and how the shim loaded it)."""
    global _compiler
    if _compiler is None:
        buf = C.create_string_buffer(512)
        _lib.check(lib().kcg_hip_compiler_info(buf, len(buf)), "kcg_hip_compiler_info")
        _compiler = buf.value.decode()
    return _compiler


def cache_dir():
    """Directory of the on-disk code-object cache (KCG_CACHE_DIR, or `_cache` beside the library)."""
    buf = C.create_string_buffer(4096)
    _lib.check(lib().kcg_hip_cache_dir(buf, len(buf)), "kcg_hip_cache_dir")
    return buf.value.decode()


def compile_to_code(src, opts=(), use_cache=True, refresh=False):
    """Full source text -> gfx950 code object bytes (hipRTC; needs no GPU).  Code
    objects are cached on disk by the library, keyed by compiler, source and options; `refresh`
    compiles even when the cache holds the object and rewrites it."""
    code, size = C.c_void_p(), C.c_size_t()
    log = C.create_string_buffer(1 << 16)
    if use_cache:
        rc = lib().kcg_hip_compile_to_code_cached(src.encode(), _cstr_array(list(opts)), len(opts), int(refresh),
                                                  C.byref(code), C.byref(size), log, len(log))
    else:
        rc = lib().kcg_hip_compile_to_code(src.encode(), _cstr_array(list(opts)), len(opts), C.byref(code),
                                           C.byref(size), log, len(log))
    if rc != 0:
        raise _lib.KcgError(rc, "kcg_hip_compile_to_code", log.value.decode(errors="replace"))
    try:
        return C.string_at(code.value, size.value)
    finally:
        lib().kcg_hip_free_code(code)


class Kernel:
    def __init__(self, module, handle, info=None):
        self.module, self.handle, self.info = module, handle, info

    @staticmethod
    def _pack(args):
        holders = []
        for a in args:
            if hasattr(a, "data_ptr"):
                holders.append(C.c_void_p(a.data_ptr()))
            elif isinstance(a, float):
                holders.append(C.c_float(a))
            elif isinstance(a, int):
                holders.append(C.c_void_p(a))
            else:
                raise TypeError("unsupported kernel argument %r" % type(a))
        arr = (C.c_void_p * len(holders))(*[C.cast(C.pointer(h), C.c_void_p) for h in holders])
        return holders, arr

    @staticmethod
    def _stream(stream):
        if stream is None:
            import torch
            return C.c_void_p(torch.cuda.current_stream().cuda_stream)
        return C.c_void_p(stream)

    def _dims(self, grid, block):
        grid = grid if grid is not None else self.info["grid"]
        block = block if block is not None else self.info["block"]
        return (C.c_uint32 * 3)(*grid), (C.c_uint32 * 3)(*block)

    def workspace(self):
        """The scratch buffer of a kernel whose launch info reports workspace_bytes: one zero-initialised device
        tensor per Kernel object, shared by its launches (which therefore must not overlap in time)."""
        if getattr(self, "_workspace", None) is None:
            import torch
            self._workspace = torch.zeros(int(self.info["workspace_bytes"]), dtype=torch.uint8, device="cuda")
        return self._workspace

    def _complete(self, args):
        """Inserts the workspace behind the output pointers when the caller has left it out."""
        info = self.info or {}
        if info.get("workspace_bytes", 0) and len(args) == info["num_args"] - 1:
            at = info["num_args"] - info["num_scalars"] - 1
            args = tuple(args[:at]) + (self.workspace(),) + tuple(args[at:])
        return args

    def launch(self, *args, grid=None, block=None, lds_bytes=None, stream=None):
        g, b = self._dims(grid, block)
        lds = self.info["lds_bytes"] if lds_bytes is None else lds_bytes
        holders, arr = self._pack(self._complete(args))
        check(lib().kcg_hip_launch(self.handle, g, b, lds, self._stream(stream), arr), "kcg_hip_launch")

    def arg_sets(self, sets):
        """Packs several argument lists for launch_sequence / time_rotating; keep the result alive while in use."""
        packed = [self._pack(self._complete(a)) for a in sets]
        arr = (C.POINTER(C.c_void_p) * len(packed))(*[C.cast(p[1], C.POINTER(C.c_void_p)) for p in packed])
        return packed, arr, len(packed)

    def launch_sequence(self, packed_sets, first, count, grid=None, block=None, lds_bytes=None, stream=None):
        """`count` launches from inside the library, launch i on argument set (first + i) % len(sets)."""
        g, b = self._dims(grid, block)
        lds = self.info["lds_bytes"] if lds_bytes is None else lds_bytes
        _, arr, n = packed_sets
        check(lib().kcg_hip_launch_sequence(self.handle, g, b, lds, self._stream(stream), arr, n, first, count),
              "kcg_hip_launch_sequence")

    def time_rotating(self, packed_sets, warmup=3, warmup_ms=30.0, runs=7, launches_per_run=3, grid=None, block=None,
                      lds_bytes=None, stream=None):
        """(median, minimum) per-launch duration in ms over `runs` event-timed groups, operand sets in turn."""
        g, b = self._dims(grid, block)
        lds = self.info["lds_bytes"] if lds_bytes is None else lds_bytes
        _, arr, n = packed_sets
        med, low = C.c_float(), C.c_float()
        check(lib().kcg_hip_time_rotating(self.handle, g, b, lds, self._stream(stream), arr, n, warmup, warmup_ms, runs,
                                          launches_per_run, C.byref(med), C.byref(low)), "kcg_hip_time_rotating")
        return med.value, low.value

    def launch_scratch(self, *args, grid=None, block=None, lds_bytes=None, stream=None):
        """launch() of a kernel that takes a workspace, on the library's own scratch array instead of a buffer
        of the caller's (kcg_hip_launch_scratch): allocates nothing.  `args` are the kernel's arguments without
        the workspace.  Launches that overlap in time on one GPU race on the array."""
        info = self.info
        if not info.get("workspace_bytes", 0):
            raise ValueError("the kernel takes no workspace")
        at = info["num_args"] - info["num_scalars"] - 1
        full = tuple(args[:at]) + (0,) + tuple(args[at:])
        g, b = self._dims(grid, block)
        lds = info["lds_bytes"] if lds_bytes is None else lds_bytes
        holders, arr = self._pack(full)
        check(lib().kcg_hip_launch_scratch(self.handle, g, b, lds, self._stream(stream), arr, len(full), at,
                                           int(info["workspace_bytes"])), "kcg_hip_launch_scratch")

    def time(self, *args, warmup=3, iters=20, grid=None, block=None, lds_bytes=None, stream=None):
        """Average kernel duration in ms from HIP events on the launch stream."""
        g, b = self._dims(grid, block)
        lds = self.info["lds_bytes"] if lds_bytes is None else lds_bytes
        holders, arr = self._pack(self._complete(args))
        ms = C.c_float()
        check(lib().kcg_hip_time_launches(self.handle, g, b, lds, self._stream(stream), arr, warmup, iters,
                                          C.byref(ms)), "kcg_hip_time_launches")
        return ms.value


class Graph:
    """A recorded sequence of kernel launches (kcg_hip_graph_*), replayed with one call:

        g = Graph()
        with g:                                   # launches on g.stream are recorded, not run
            kernel_a.launch(x, y, stream=g.stream)
            kernel_b.launch(y, z, stream=g.stream)
        g.launch()                                # runs both, on torch's current stream unless one is given

    The device pointers are fixed at capture, so the tensors must stay alive and in place.  A kernel that takes a
    workspace must have it before the capture starts (Kernel.workspace()): allocating inside a capture is an error."""

    def __init__(self):
        s = C.c_void_p()
        check(lib().kcg_hip_stream_create(C.byref(s)), "kcg_hip_stream_create")
        self._stream, self._h = s, None

    @property
    def stream(self):
        return self._stream.value

    def __enter__(self):
        if self._h is not None:
            raise RuntimeError("the graph has been recorded already")
        check(lib().kcg_hip_graph_begin_capture(self._stream), "kcg_hip_graph_begin_capture")
        return self

    def __exit__(self, exc_type, exc, tb):
        h = C.c_void_p()
        rc = lib().kcg_hip_graph_end_capture(self._stream, C.byref(h))
        if exc_type is None:
            check(rc, "kcg_hip_graph_end_capture")
            self._h = h
        elif rc == 0 and h:
            lib().kcg_hip_graph_destroy(h)
        return False

    def num_nodes(self):
        n = C.c_size_t()
        check(lib().kcg_hip_graph_num_nodes(self._h, C.byref(n)), "kcg_hip_graph_num_nodes")
        return n.value

    def launch(self, stream=None):
        if self._h is None:
            raise RuntimeError("nothing has been recorded")
        check(lib().kcg_hip_graph_launch(self._h, Kernel._stream(stream)), "kcg_hip_graph_launch")

    def destroy(self):
        if self._h is not None:
            check(lib().kcg_hip_graph_destroy(self._h), "kcg_hip_graph_destroy")
            self._h = None
        if self._stream is not None:
            check(lib().kcg_hip_stream_destroy(self._stream), "kcg_hip_stream_destroy")
            self._stream = None


class Module:
    """A loaded code object.  `infos` maps kernel name -> launch info."""

    def __init__(self, code, infos=None):
        self.infos = {i["name"]: i for i in (infos or [])}
        handle = C.c_void_p()
        buf = C.create_string_buffer(code, len(code))
        check(lib().kcg_hip_load_code(buf, len(code), C.byref(handle)), "kcg_hip_load_code")
        self.handle = handle
        self._kernels = {}

    def kernel(self, name):
        if name not in self._kernels:
            h = C.c_void_p()
            check(lib().kcg_hip_get_kernel(self.handle, name.encode(), C.byref(h)), "kcg_hip_get_kernel(%s)" % name)
            self._kernels[name] = Kernel(self, h, self.infos.get(name))
        return self._kernels[name]

    def destroy(self):
        if self.handle:
            check(lib().kcg_hip_module_destroy(self.handle), "kcg_hip_module_destroy")
            self.handle = None
            self._kernels = {}


def compile_source(src, infos=None, opts=()):
    """Full source text -> loaded Module on the current device."""
    return Module(compile_to_code(src, opts), infos)


_kernel_cache = {}


def get_kernel(family, **params):
    """Emit + compile + load one kernel of a family; memoised per process."""
    key = (family, tuple(sorted(params.items())))
    if key not in _kernel_cache:
        text, info = emit_kernel(family, "kernel0", **params)
        mod = compile_source(prelude() + text, [info])
        _kernel_cache[key] = mod.kernel("kernel0")
    return _kernel_cache[key]
