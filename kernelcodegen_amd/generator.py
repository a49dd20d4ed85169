"""Python mirror of the C++ entry point (include/KernelCodeGen.h) over the C
facade: the same calls in the same order as a C++ user of the library makes.

    gen = KernelCodeGenerator("ROCm")
    graph = gen.createGraph("demo")
    gen.opts.append("Matmul")                      # generator.opts.push_back(make_unique<MatmulOptimizer>())
    A = graph.create("PlaceHolder", [m, k], "float32")
    B = graph.create("PlaceHolder", [k, n], "float32")
    C = graph.create("Matmul", A, B)
    module = gen.optimize(graph)
    source = gen.codegen(module)
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import LaunchInfo, lib


class MemorySpace:
    global_ = 1
    shared = 2
    local = 3
    constant = 4
    unallocated = 5
    inplace = 6


class Layout:
    rowMajor = 0
    colMajor = 1


class GeneratorError(RuntimeError):
    pass


class ComputeDAG:
    def __init__(self, gen):
        self._gen = gen

    def _check(self, vid):
        if vid < 0:
            raise GeneratorError(lib().kcg_generator_error(self._gen._h).decode().strip())
        return vid

    def create(self, op, *args, **kw):
        h, L = self._gen._h, lib()
        dtype = kw.get("dtype", "")
        if op == "PlaceHolder":
            shape, dt = args
            arr = (C.c_int64 * len(shape))(*shape)
            return self._check(L.kcg_placeholder(h, arr, len(shape), dt.encode()))
        if op == "Matmul":
            # (A, B[, dtype]) or, with one fp32 scale per tensor as graph values, (A, B, scaleA, scaleB[, dtype])
            a, b = args[:2]
            if len(args) >= 4 and not isinstance(args[2], str):
                dtype = args[4] if len(args) > 4 else dtype
                return self._check(L.kcg_matmul_scaled(h, a, b, args[2], args[3], dtype.encode()))
            dtype = args[2] if len(args) > 2 else dtype
            return self._check(L.kcg_matmul(h, a, b, dtype.encode()))
        if op == "BatchedMatmul":
            # (A, layoutA, B, layoutB[, dtype]) or (A, layoutA, B, layoutB, scaleA, scaleB[, dtype])
            a, la, b, lb = args[:4]
            if len(args) >= 6 and not isinstance(args[4], str):
                dtype = args[6] if len(args) > 6 else dtype
                return self._check(L.kcg_batched_matmul_scaled(h, a, la, b, lb, args[4], args[5], dtype.encode()))
            dtype = args[4] if len(args) > 4 else dtype
            return self._check(L.kcg_batched_matmul(h, a, la, b, lb, dtype.encode()))
        if op == "Softmax":
            x = args[0]
            axis = args[1] if len(args) > 1 else -1
            ms = args[2] if len(args) > 2 else MemorySpace.global_
            return self._check(L.kcg_softmax(h, x, axis, ms, dtype.encode()))
        if op == "Relu":
            x, ms = args[:2]
            return self._check(L.kcg_relu(h, x, ms, dtype.encode()))
        if op == "ElementWise":
            x, operation, ms = args[:3]
            dtype = args[3] if len(args) > 3 else dtype
            return self._check(L.kcg_elementwise(h, x, operation.encode(), ms, dtype.encode()))
        if op == "Binary":
            a, b, operation = args[:3]
            ms = args[3] if len(args) > 3 else MemorySpace.global_
            return self._check(L.kcg_binary(h, a, b, operation.encode(), ms, dtype.encode()))
        if op == "LayerNorm":
            x, scale, bias, axis = args[:4]
            eps = args[4] if len(args) > 4 else 1e-5
            ms = args[5] if len(args) > 5 else MemorySpace.global_
            return self._check(L.kcg_layernorm(h, x, scale, bias, axis, eps, ms, dtype.encode()))
        if op == "Gather":
            x, indices = args[:2]
            axis = args[2] if len(args) > 2 else 0
            return self._check(L.kcg_gather(h, x, indices, axis, dtype.encode()))
        raise GeneratorError("unknown operator %s" % op)

    def dump(self):
        return self._gen._dump(0)


class Module:
    """Handle of the optimized module held by the generator."""

    def __init__(self, gen):
        self._gen = gen

    def dump(self):
        return self._gen._dump(1)


class _Opts(list):
    def __init__(self, gen):
        super().__init__()
        self._gen = gen

    def append(self, name):
        if lib().kcg_add_optimizer(self._gen._h, name.encode()) != 0:
            raise GeneratorError(lib().kcg_generator_error(self._gen._h).decode())
        super().append(name)

    push_back = append


class KernelCodeGenerator:
    def __init__(self, platform="ROCm"):
        self._h = C.c_void_p(lib().kcg_generator_create(platform.encode()))
        if not self._h:
            raise GeneratorError("could not create the generator")
        self.opts = _Opts(self)
        self._graph = None

    def __del__(self):
        try:
            if self._h:
                lib().kcg_generator_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def _err(self):
        return lib().kcg_generator_error(self._h).decode().strip()

    def createGraph(self, name):
        if lib().kcg_generator_create_graph(self._h, name.encode()) != 0:
            raise GeneratorError(self._err())
        self._graph = ComputeDAG(self)
        return self._graph

    def getGraph(self):
        return self._graph

    def setLogMode(self, level):
        lib().kcg_generator_set_log_mode(self._h, level)

    def setConfigs(self, optimizer, configs):
        sizes, keys, vals = [], [], []
        for m in configs:
            sizes.append(len(m))
            for k, v in m.items():
                keys.append(k.encode())
                vals.append(int(v))
        n = max(1, len(keys))
        rc = lib().kcg_set_configs(self._h, optimizer.encode(), len(configs), (C.c_int * max(1, len(sizes)))(*sizes),
                                   (C.c_char_p * n)(*keys), (C.c_int * n)(*vals))
        if rc != 0:
            raise GeneratorError(self._err())

    def getConfigs(self, optimizer):
        """The configuration candidates of one optimizer: a list of dicts."""
        text = lib().kcg_get_configs(self._h, optimizer.encode())
        if text is None:
            raise GeneratorError(self._err())
        return [{k: int(v) for k, v in (item.split("=") for item in line.split())} for line in text.decode().splitlines()]

    def optimize(self, graph=None):
        if lib().kcg_optimize(self._h) != 0:
            raise GeneratorError(self._err())
        return Module(self)

    def setLowering(self, mode):
        """"families": a recognised operator becomes a gfx950 kernel family sized by its schedule (default).
        "schedule": the scheduled function body itself is printed, one statement per operation, the way the
        reference's backend prints CUDA (src/Backend/CUDA.cc:61-1184)."""
        if lib().kcg_set_lowering(self._h, mode.encode()) != 0:
            raise GeneratorError(self._err())

    def codegen(self, module=None):
        src = lib().kcg_codegen(self._h)
        if src is None:
            raise GeneratorError(self._err())
        return src.decode()

    def adaptor(self, kernel_file):
        """C host program that compiles `kernel_file` (the saved result of codegen) and times its kernels."""
        text = lib().kcg_adaptor(self._h, str(kernel_file).encode())
        if text is None:
            raise GeneratorError(self._err())
        return text.decode()

    def launchInfos(self):
        out = []
        for i in range(lib().kcg_num_kernels(self._h)):
            info = LaunchInfo()
            lib().kcg_kernel_info(self._h, i, C.byref(info))
            d = info.as_dict()
            d["function"] = lib().kcg_kernel_function(self._h, i).decode()
            d["lowering"] = lib().kcg_kernel_lowering(self._h, i).decode()
            buf = (C.c_int64 * 16)()
            n = lib().kcg_kernel_arg_bytes(self._h, i, buf, 16)
            d["arg_bytes"] = list(buf[:n])
            types = (C.c_int * 16)()
            nt = lib().kcg_kernel_arg_types(self._h, i, types, 16)
            d["arg_types"] = list(types[:nt])
            out.append(d)
        return out

    def skippedFunctions(self):
        """Operators the graph calls but no optimizer scheduled: codegen() emitted no kernel for them."""
        return [lib().kcg_skipped_function(self._h, i).decode() for i in range(lib().kcg_num_skipped(self._h))]

    CONFIG_KEYS = ("BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "BLOCK_SIZE", "THREAD_SIZE_M", "THREAD_SIZE_N",
                   "THREAD_SIZE", "VECTORIZE_WIDTH", "DTYPE_BITS", "WARP_SIZE", "GROUP_SIZE_M", "TREE_REDUCE", "FUSE_GELU",
                   "ROW_BLOCK_SIZE", "CAUSAL", "Slice", "HdxBr", "BrxBc")

    def evaluations(self):
        """The candidates the last optimize() tried: optimizer, config (index and map), kernels emitted,
        latency in ms (inf when the candidate failed, 0 without a GPU), kept or not, note."""
        out = []
        for i in range(lib().kcg_num_evaluations(self._h)):
            name, note = C.c_char_p(), C.c_char_p()
            idx, kernels, kept, ms = C.c_int(), C.c_int(), C.c_int(), C.c_float()
            lib().kcg_evaluation(self._h, i, C.byref(name), C.byref(idx), C.byref(kernels), C.byref(ms), C.byref(kept),
                                 C.byref(note))
            config = {k: lib().kcg_evaluation_config(self._h, i, k.encode()) for k in self.CONFIG_KEYS}
            out.append({"optimizer": name.value.decode(), "config_index": idx.value, "kernels": kernels.value,
                        "latency_ms": float("inf") if ms.value > 1e38 else ms.value, "kept": bool(kept.value),
                        "note": note.value.decode(), "config": {k: v for k, v in config.items() if v >= 0}})
        return out

    def evaluate(self):
        """evaluate(optimized module): summed latency of its kernels in ms (0 without a GPU)."""
        ms = lib().kcg_evaluate(self._h)
        if ms < 0:
            raise GeneratorError(self._err())
        return ms

    def plan(self, which=1):
        """The calls of the module body in order with the buffers they read and write (kcg_module_plan)."""
        import json
        text = lib().kcg_module_plan(self._h, which)
        if text is None:
            raise GeneratorError(self._err())
        return json.loads(text.decode())

    def save(self, text, path):
        if path == "terminal":
            print(text, end="")
            return
        with open(path, "w") as f:
            f.write(text)

    def _dump(self, which):
        t = lib().kcg_dump(self._h, which)
        return t.decode() if t is not None else ""

    def verify(self, which=1):
        rc = lib().kcg_verify(self._h, which)
        return rc == 0, (self._err() if rc else "")

    def functionState(self, function, which=1):
        return lib().kcg_function_state(self._h, which, function.encode()).decode()

    def interpret(self, inputs, out_shape, which=1):
        """Runs the graph (which=0) or the optimized module (which=1) on the host
        interpreter; returns the result of the last call as an fp32 array."""
        arrs = [np.ascontiguousarray(a, dtype=np.float32) for a in inputs]
        ptrs = (C.POINTER(C.c_float) * max(1, len(arrs)))(*[a.ctypes.data_as(C.POINTER(C.c_float)) for a in arrs])
        sizes = (C.c_int64 * max(1, len(arrs)))(*[a.size for a in arrs])
        out = np.empty(out_shape, dtype=np.float32)
        n = lib().kcg_interpret(self._h, which, ptrs, sizes, len(arrs), out.ctypes.data_as(C.POINTER(C.c_float)), out.size)
        if n < 0:
            raise GeneratorError(self._err())
        if n != out.size:
            raise GeneratorError("result has %d elements, expected %d" % (n, out.size))
        return out


def fmha_map(name, *inputs):
    """FMHAOptimizer::getAffineMap(name) under the config the last optimize() with the FMHA optimizer left in force
    (reference: src/Optimizer/Optimizer.cc:2201-2437), evaluated at `inputs`: the list of results."""
    arr = (C.c_int64 * max(1, len(inputs)))(*inputs)
    out = (C.c_int64 * 8)()
    n = lib().kcg_fmha_map_evaluate(name.encode(), arr, len(inputs), out, 8)
    if n < 0:
        raise GeneratorError({-1: "unknown attention map %r", -2: "wrong number of inputs for map %r"}.get(n, "map %r failed") % name)
    return [int(out[i]) for i in range(n)]
