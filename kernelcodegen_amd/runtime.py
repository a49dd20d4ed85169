"""Host-side helpers over the C ABI: emit a kernel, compile it with hipRTC (or
pick up a code object built ahead of time), load it, launch it on torch's
current stream.  torch supplies device memory and the stream handle only."""
import ctypes as C
import hashlib
import os

from . import _lib
from ._lib import LaunchInfo, check, lib

_PKG = os.path.dirname(os.path.abspath(__file__))
CACHE_DIR = os.path.join(_PKG, "_cache")


def prelude():
    return lib().kcg_prelude().decode()


def _cstr_array(items):
    arr = (C.c_char_p * max(1, len(items)))()
    for i, s in enumerate(items):
        arr[i] = s.encode()
    return arr


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


def _cache_path(src, opts):
    h = hashlib.sha256()
    h.update(compiler_info().encode() + b"\0")
    h.update(src.encode())
    for o in opts:
        h.update(b"\0" + o.encode())
    return os.path.join(CACHE_DIR, h.hexdigest()[:32] + ".hsaco")


def compile_to_code(src, opts=(), use_cache=True, refresh=False):
    """Full source text -> gfx950 code object bytes (hipRTC; needs no GPU).  Code
    objects are cached on disk by the hash of compiler, source and options; `refresh`
    compiles even when the cache holds the object and rewrites it."""
    path = _cache_path(src, opts)
    if use_cache and not refresh and os.path.exists(path):
        with open(path, "rb") as f:
            return f.read()
    code, size = C.c_void_p(), C.c_size_t()
    log = C.create_string_buffer(1 << 16)
    rc = lib().kcg_hip_compile_to_code(src.encode(), _cstr_array(list(opts)), len(opts), C.byref(code),
                                       C.byref(size), log, len(log))
    if rc != 0:
        raise _lib.KcgError(rc, "kcg_hip_compile_to_code", log.value.decode(errors="replace"))
    try:
        blob = C.string_at(code.value, size.value)
    finally:
        lib().kcg_hip_free_code(code)
    if use_cache:
        os.makedirs(CACHE_DIR, exist_ok=True)
        tmp = path + ".tmp%d" % os.getpid()
        with open(tmp, "wb") as f:
            f.write(blob)
        os.replace(tmp, path)
    return blob


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

    def launch(self, *args, grid=None, block=None, lds_bytes=None, stream=None):
        g, b = self._dims(grid, block)
        lds = self.info["lds_bytes"] if lds_bytes is None else lds_bytes
        holders, arr = self._pack(args)
        check(lib().kcg_hip_launch(self.handle, g, b, lds, self._stream(stream), arr), "kcg_hip_launch")

    def time(self, *args, warmup=3, iters=20, grid=None, block=None, lds_bytes=None, stream=None):
        """Average kernel duration in ms from HIP events on the launch stream."""
        g, b = self._dims(grid, block)
        lds = self.info["lds_bytes"] if lds_bytes is None else lds_bytes
        holders, arr = self._pack(args)
        ms = C.c_float()
        check(lib().kcg_hip_time_launches(self.handle, g, b, lds, self._stream(stream), arr, warmup, iters,
                                          C.byref(ms)), "kcg_hip_time_launches")
        return ms.value


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
