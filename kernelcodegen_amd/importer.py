"""Graph import: an operator graph written down as data (ONNX operator names and attributes, as JSON or as
Python dicts) becomes a ComputeDAG through the Frontend builders.  The reference plans this as "onnx -> affine"
(doc/Plan.md:4-8) and has no importer; ONNX protobufs are not read here (no onnx package in the build), only
their vocabulary is:

    {"name": "block",
     "inputs":  [{"name": "x", "shape": [16, 512], "dtype": "float32"}, ...],
     "nodes":   [{"op": "MatMul", "inputs": ["x", "w"], "output": "h"},
                 {"op": "Relu", "inputs": ["h"], "output": "h"},
                 {"op": "LayerNormalization", "inputs": ["h", "g", "b"], "output": "y", "axis": -1, "epsilon": 1e-5}]}

Supported: MatMul (2-d, or batched with equal leading dims; with four inputs the last two are per-tensor fp32 scales of
a quantised product, "dtype" names the result type), Relu, Gelu, Tanh, Sqrt, Log, Cast (to), Add, Sub,
Mul, Div, Pow, Softmax (last axis), LayerNormalization, Gather (indices of dtype "index").
"""
import json

from .generator import GeneratorError, KernelCodeGenerator, Layout, MemorySpace

_ELEMENTWISE = {"Gelu": "Gelu", "Tanh": "Tanh", "Sqrt": "Sqrt", "Log": "Log"}
_BINARY = {"Add", "Sub", "Mul", "Div", "Pow"}
_OPTIMIZER_OF = {"MatMul": "Matmul", "Relu": "ElementWise", "Gelu": "ElementWise", "Tanh": "ElementWise", "Sqrt": "ElementWise",
                 "Log": "ElementWise", "Cast": "ElementWise", "Add": "Binary", "Sub": "Binary", "Mul": "Binary", "Div": "Binary",
                 "Pow": "Binary", "Softmax": "Softmax", "LayerNormalization": "LayerNorm", "Gather": "Gather"}


def import_graph(description, platform="ROCm", optimizers="auto"):
    """Builds the graph.  Returns (generator, graph, values) where `values` maps every tensor name of the
    description to its graph value.  `optimizers="auto"` pushes the optimizer of every operator kind that occurs
    (attention fusion first when a MatMul -> Softmax -> MatMul chain is present); a list of names pushes those."""
    d = json.loads(description) if isinstance(description, (str, bytes)) else description
    gen = KernelCodeGenerator(platform)
    g = gen.createGraph(str(d.get("name", "graph")))
    values, shapes = {}, {}
    for t in d.get("inputs", []):
        values[t["name"]] = g.create("PlaceHolder", [int(x) for x in t["shape"]], t.get("dtype", "float32"))
        shapes[t["name"]] = [int(x) for x in t["shape"]]
    used = []

    def operand(node, i):
        name = node["inputs"][i]
        if name not in values:
            raise GeneratorError("node %s reads %r before it is produced" % (node.get("op"), name))
        return values[name]

    for node in d.get("nodes", []):
        op = node["op"]
        ins = node["inputs"]
        if op == "MatMul":
            a, b = operand(node, 0), operand(node, 1)
            sa, sb = shapes[ins[0]], shapes[ins[1]]
            trans_b = bool(node.get("transB", 0))
            # four inputs: a quantised product, inputs 2 and 3 are the per-tensor scales (one float32 element each);
            # "dtype" names the result's element type (fp8 operands have no result of their own type)
            scales = [operand(node, 2), operand(node, 3)] if len(ins) == 4 else []
            extra = scales + ([node["dtype"]] if "dtype" in node else [])
            if len(sa) == 2 and len(sb) == 2 and not trans_b:
                out = g.create("Matmul", a, b, *extra)
                shape = [sa[0], sb[1]]
                used.append("Matmul")
            else:
                out = g.create("BatchedMatmul", a, Layout.rowMajor, b, Layout.colMajor if trans_b else Layout.rowMajor, *extra)
                shape = sa[:-1] + [sb[-2] if trans_b else sb[-1]]
                used.append("BatchMatmul")
        elif op == "Relu":
            out, shape = g.create("Relu", operand(node, 0), MemorySpace.inplace), shapes[ins[0]]
        elif op in _ELEMENTWISE:
            out, shape = g.create("ElementWise", operand(node, 0), _ELEMENTWISE[op], MemorySpace.global_), shapes[ins[0]]
        elif op == "Cast":
            out = g.create("ElementWise", operand(node, 0), "Cast", MemorySpace.global_, node["to"])
            shape = shapes[ins[0]]
        elif op in _BINARY:
            import numpy as np
            out = g.create("Binary", operand(node, 0), operand(node, 1), op)
            shape = list(np.broadcast_shapes(tuple(shapes[ins[0]]), tuple(shapes[ins[1]])))
        elif op == "Softmax":
            out, shape = g.create("Softmax", operand(node, 0), int(node.get("axis", -1)), MemorySpace.inplace), shapes[ins[0]]
        elif op == "LayerNormalization":
            out = g.create("LayerNorm", operand(node, 0), operand(node, 1), operand(node, 2), int(node.get("axis", -1)),
                           float(node.get("epsilon", 1e-5)))
            shape = shapes[ins[0]]
        elif op == "Gather":
            axis = int(node.get("axis", 0))
            out = g.create("Gather", operand(node, 0), operand(node, 1), axis)
            sx, si = shapes[ins[0]], shapes[ins[1]]
            axis %= len(sx)
            shape = sx[:axis] + ([] if si == [1] else si) + sx[axis + 1:]
        else:
            raise GeneratorError("operator %r is not supported by the importer" % op)
        values[node["output"]] = out
        shapes[node["output"]] = shape
        if op in _OPTIMIZER_OF and op != "MatMul":
            used.append(_OPTIMIZER_OF[op])
    if optimizers == "auto":
        ops = [n["op"] for n in d.get("nodes", [])]
        chain = any(ops[i:i + 3] == ["MatMul", "Softmax", "MatMul"] for i in range(len(ops)))
        # fusing optimizers first: Matmul absorbs a following Relu, LayerNorm a following Gelu
        order = ["Matmul", "BatchMatmul", "LayerNorm", "Softmax", "Gather", "Binary", "ElementWise"]
        optimizers = (["FMHA"] if chain else []) + [n for n in order if n in used]
    for name in optimizers:
        gen.opts.append(name)
    gen.shapes = shapes
    return gen, g, values


_TORCH_DTYPE = {"float32": "float32", "float64": "float64", "float16": "float16", "bfloat16": "bfloat16",
                "float8_e4m3": "float8_e4m3fn", "int64": "int64", "int32": "int32", "int16": "int16", "index": "int64",
                "bool": "bool"}


def _prepare(gen, inputs):
    """codegen, compile (through the code-object cache), allocate per the module's plan; returns the module, the
    buffers by id and the launches [(kernel, arguments)] in call order."""
    import torch
    from . import runtime as R
    src = gen.codegen()
    infos = {i["function"]: i for i in gen.launchInfos()}
    mod = R.compile_source(src, list(infos.values()))
    plan = gen.plan(1)
    tensors, inputs = {}, list(inputs)
    for b in plan["buffers"]:
        if "alias" in b:
            continue
        dtype = getattr(torch, _TORCH_DTYPE[b["dtype"]])
        if b["input"] >= 0:
            if b["input"] >= len(inputs):
                raise GeneratorError("the graph has more placeholders than inputs were given")
            t = inputs[b["input"]]
            if not (t.is_cuda and t.is_contiguous()) or list(t.shape) != b["shape"] or t.dtype != dtype:
                raise GeneratorError("input for buffer %d must be a contiguous device tensor of shape %s and dtype %s"
                                     % (b["id"], b["shape"], b["dtype"]))
            tensors[b["id"]] = t
        else:
            tensors[b["id"]] = torch.empty(b["shape"], dtype=dtype, device="cuda")
    for b in plan["buffers"]:
        if "alias" in b:
            tensors[b["id"]] = tensors[b["alias"]]
    last, launches = None, []
    for call in plan["calls"]:
        info = infos.get(call["callee"])
        if info is None:
            raise GeneratorError("%s is called but has no kernel (no optimizer scheduled it)" % call["callee"])
        args = [tensors[i] for i in call["operands"]]
        if call["result"] >= 0 and call["result"] not in call["operands"]:
            args.append(tensors[call["result"]])
        if len(args) != info["num_args"] - info["num_scalars"] - (1 if info.get("workspace_bytes") else 0):
            raise GeneratorError("%s takes %d buffers, the plan gives %d" % (call["callee"], info["num_args"], len(args)))
        for t, nbytes in zip(args, info["arg_bytes"]):
            if t.numel() * t.element_size() != nbytes:
                raise GeneratorError("%s: operand of %d bytes where the kernel expects %d"
                                     % (call["callee"], t.numel() * t.element_size(), nbytes))
        launches.append((mod.kernel(info["name"]), args + [1.0] * info["num_scalars"]))
        last = call["result"] if call["result"] >= 0 else (call["operands"][-1] if call["operands"] else None)
    if last is not None:
        tensors["result"] = tensors[last]
    tensors["module"] = mod         # keeps the code object loaded while the launches run
    return mod, tensors, launches


def run_graph(gen, inputs, stream=None):
    """Runs the generator's optimized module on the device: codegen, compile (through the code-object cache),
    then every call of the module body in order, each on the buffers the module's plan names.  `inputs` are
    contiguous device tensors for the graph's placeholders in creation order; buffers a fusion allocated at
    module level and the results of the calls are allocated here.  Returns {buffer id: tensor}; the last call's
    result is under "result".  An operator that no optimizer scheduled has no kernel and raises."""
    _, tensors, launches = _prepare(gen, inputs)
    for kernel, args in launches:
        kernel.launch(*args, stream=stream)
    return tensors


class CapturedGraph:
    """The kernels of an optimized module recorded once as a HIP graph over fixed buffers: `replay()` runs all of
    them with one call, which is what a caller wants who runs the same small graph over and over (the launches of a
    chain of small kernels cost more on the host than the kernels take on the device).  `tensors` is what run_graph
    returns; write new inputs into the same input tensors before a replay."""

    def __init__(self, gen, inputs):
        import torch
        from . import runtime as R
        self.module, self.tensors, self.launches = _prepare(gen, inputs)
        for kernel, _ in self.launches:
            if (kernel.info or {}).get("workspace_bytes", 0):
                kernel.workspace()              # allocated and zeroed before the capture, never inside it
        torch.cuda.synchronize()
        self.graph = R.Graph()
        with self.graph:
            for kernel, args in self.launches:
                kernel.launch(*args, stream=self.graph.stream)

    def replay(self, stream=None):
        self.graph.launch(stream)

    def run_eagerly(self, stream=None):
        for kernel, args in self.launches:
            kernel.launch(*args, stream=stream)

    def destroy(self):
        self.graph.destroy()


def capture_graph(gen, inputs):
    """run_graph's launches recorded as one HIP graph; see CapturedGraph."""
    return CapturedGraph(gen, inputs)
