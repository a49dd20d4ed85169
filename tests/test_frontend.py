"""Frontend op builders: the naive affine nests they emit, executed on the host
interpreter, must equal the CPU oracle (bit for bit where the operation order
is the same), and the emitted IR must have the structure of the reference's
dumps (doc/pass.md:406-467 naive BatchMatmul / Softmax, :738-780 naive
LayerNorm)."""
import re

import numpy as np
import pytest

import oracle_lib as O
from kernelcodegen_amd.generator import GeneratorError, KernelCodeGenerator, Layout, MemorySpace


def new_graph(name="demo"):
    gen = KernelCodeGenerator("ROCm")
    return gen, gen.createGraph(name)


def test_matmul_nest_equals_oracle_bitwise():
    gen, g = new_graph()
    a, b = O.uniform((24, 40), 1), O.uniform((40, 16), 2)
    A = g.create("PlaceHolder", [24, 40], "float32")
    B = g.create("PlaceHolder", [40, 16], "float32")
    g.create("Matmul", A, B)
    assert np.array_equal(gen.interpret([a, b], (24, 16), which=0), O.matmul(a, b))
    text = g.dump()
    assert "func.func @Matmul_m24n16k40(" in text and 'func.state = "cpu"' in text
    assert "iter_args(" in text and "arith.mulf" in text and "arith.addf" in text
    ok, msg = gen.verify(0)
    assert ok, msg


@pytest.mark.parametrize("la,lb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_batched_matmul_layouts_equal_oracle(la, lb):
    gen, g = new_graph()
    m, n, k = 6, 10, 7
    a = O.uniform((2, 3) + ((k, m) if la else (m, k)), 3)
    b = O.uniform((2, 3) + ((n, k) if lb else (k, n)), 4)
    A = g.create("PlaceHolder", list(a.shape), "float32")
    B = g.create("PlaceHolder", list(b.shape), "float32")
    g.create("BatchedMatmul", A, la, B, lb)
    out = gen.interpret([a, b], (2, 3, m, n), which=0)
    assert np.array_equal(out, O.batched_matmul(a, b, bool(la), bool(lb)))
    assert "@BatchMatmul_2_3_m6_n10_k7_%s%s" % ("NT"[la], "NT"[lb]) in g.dump()


def test_softmax_in_place_equals_oracle():
    gen, g = new_graph()
    x = O.normal((3, 4, 9), 5)
    X = g.create("PlaceHolder", [3, 4, 9], "float32")
    g.create("Softmax", X, -1, MemorySpace.inplace)
    out = gen.interpret([x], (3, 4, 9), which=0)
    assert np.array_equal(out, O.softmax(x))
    assert "@Softmax_3_4_9_axis2" in g.dump()


@pytest.mark.parametrize("shape,axis,gshape", [((2, 6, 8), 1, (6, 8)), ((2, 6, 8), 2, (8,)), ((5, 12), 1, (12,)),
                                               ((2, 6, 8), 1, (8,)), ((2, 6, 8), -1, (1,))])
def test_layernorm_nest_equals_oracle_bitwise(shape, axis, gshape):
    gen, g = new_graph()
    x = O.normal(shape, 6)
    s = O.uniform(gshape, 7, 0.5, 1.5)
    b = O.uniform(gshape, 8, -0.1, 0.1)
    X = g.create("PlaceHolder", list(shape), "float32")
    S = g.create("PlaceHolder", list(gshape), "float32")
    Bv = g.create("PlaceHolder", list(gshape), "float32")
    g.create("LayerNorm", X, S, Bv, axis, 1e-5)
    out = gen.interpret([x, s, b], shape, which=0)
    ax = axis % len(shape)
    if gshape == (1,):
        ref = O.layernorm(x, np.full(shape[ax:], s[0], np.float32), np.full(shape[ax:], b[0], np.float32), ax)
    elif len(gshape) < len(shape) - ax:
        ref = O.layernorm(x, np.broadcast_to(s, shape[ax:]).copy(), np.broadcast_to(b, shape[ax:]).copy(), ax)
    else:
        ref = O.layernorm(x, s, b, ax)
    assert np.array_equal(out, ref)


def test_layernorm_ir_matches_reference_dump_structure():
    # doc/pass.md:738-780: LayerNorm_2_768_768_axis_1, N = 589824, eps as an f32 constant,
    # two iter_args nests, div / sub / mul / add / sqrt in that order, one alloc for the output
    gen, g = new_graph()
    X = g.create("PlaceHolder", [2, 768, 768], "float32")
    S = g.create("PlaceHolder", [768, 768], "float32")
    Bv = g.create("PlaceHolder", [768, 768], "float32")
    g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    text = g.dump()
    fn = text[text.index("func.func @LayerNorm_2_768_768_axis_1("):]
    fn = fn[:fn.index("return")]
    assert "(%arg0: memref<2x768x768xf32, 1>, %arg1: memref<768x768xf32, 1>, %arg2: memref<768x768xf32, 1>) -> memref<2x768x768xf32, 1>" in fn
    assert "arith.constant 5.898240e+05 : f32" in fn
    ops = re.findall(r"(affine\.for|arith\.\w+|math\.\w+|affine\.load|affine\.store|affine\.yield|memref\.alloc)", fn)
    assert ops.count("memref.alloc") == 1 and ops.count("math.sqrt") == 1
    assert fn.count("iter_args(") == 4          # two 2-deep reduction nests
    assert ops.count("arith.divf") == 3 and ops.count("arith.subf") == 1
    order = [o for o in ops if o in ("arith.divf", "arith.subf", "math.sqrt")]
    assert order == ["arith.divf", "arith.subf", "arith.divf", "math.sqrt", "arith.divf"]


@pytest.mark.parametrize("op", ["Tanh", "Sqrt", "Log", "Relu", "Gelu"])
def test_elementwise_nest_equals_oracle(op):
    gen, g = new_graph()
    x = O.uniform((3, 5, 4), 9, 0.1, 3.0) if op in ("Sqrt", "Log") else O.normal((3, 5, 4), 9)
    X = g.create("PlaceHolder", [3, 5, 4], "float32")
    g.create("ElementWise", X, op, MemorySpace.global_)
    out = gen.interpret([x], (3, 5, 4), which=0)
    assert np.array_equal(out, O.elementwise(x, op))
    assert "@%s_Elementwise_3_5_4" % op in g.dump()


def test_relu_and_cast_and_binary():
    gen, g = new_graph()
    x = O.normal((4, 6), 10, std=10.0)
    X = g.create("PlaceHolder", [4, 6], "float32")
    g.create("Relu", X, MemorySpace.inplace)
    assert np.array_equal(gen.interpret([x], (4, 6), which=0), np.maximum(x, 0))
    gen, g = new_graph()
    X = g.create("PlaceHolder", [4, 6], "float32")
    g.create("ElementWise", X, "Cast", MemorySpace.global_, "int32")
    assert np.array_equal(gen.interpret([x], (4, 6), which=0), np.trunc(x))
    gen, g = new_graph()
    y = O.normal((6,), 11)
    X = g.create("PlaceHolder", [4, 6], "float32")
    Y = g.create("PlaceHolder", [6], "float32")
    g.create("Binary", X, Y, "Add")
    assert np.array_equal(gen.interpret([x, y], (4, 6), which=0), x + y)


def test_attention_graph_equals_oracle_composition():
    gen, g = new_graph("attn")
    shp = (2, 2, 12, 8)
    q, k, v = O.normal(shp, 12), O.normal(shp, 13), O.normal(shp, 14)
    Q = g.create("PlaceHolder", list(shp), "float32")
    K = g.create("PlaceHolder", list(shp), "float32")
    V = g.create("PlaceHolder", list(shp), "float32")
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, K, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    out = gen.interpret([q, k, v], shp, which=0)
    assert np.array_equal(out, O.fmha(q, k, v))


def test_mixed_precision_operands_are_extended_to_the_accumulate_type():
    gen, g = new_graph()
    a = O.round_bf16(O.normal((8, 16), 15))
    b = O.round_bf16(O.normal((16, 8), 16))
    A = g.create("PlaceHolder", [8, 16], "bfloat16")
    B = g.create("PlaceHolder", [16, 8], "bfloat16")
    g.create("Matmul", A, B, "float32")
    text = g.dump()
    assert "memref<8x16xbf16, 1>" in text and "arith.extf" in text and "-> memref<8x8xf32, 1>" in text
    assert np.array_equal(gen.interpret([a, b], (8, 8), which=0), O.matmul(a, b))


def test_functions_are_shared_between_calls_of_the_same_shape():
    gen, g = new_graph()
    A = g.create("PlaceHolder", [8, 8], "float32")
    B = g.create("PlaceHolder", [8, 8], "float32")
    C1 = g.create("Matmul", A, B)
    g.create("Matmul", C1, B)
    text = g.dump()
    assert text.count("func.func @Matmul_m8n8k8(") == 1 and text.count("func.call @Matmul_m8n8k8(") == 2


def test_builder_errors_are_reported_not_fatal():
    gen, g = new_graph()
    A = g.create("PlaceHolder", [8, 4], "float32")
    with pytest.raises(GeneratorError, match="K-dim"):
        g.create("Matmul", A, A)
    with pytest.raises(GeneratorError, match="unknown dtype"):
        g.create("PlaceHolder", [4], "float128")
    with pytest.raises(GeneratorError, match="out of bounds"):
        g.create("LayerNorm", A, A, A, 5)
    with pytest.raises(GeneratorError, match="unknown operation"):
        g.create("ElementWise", A, "Sigmoid", MemorySpace.global_)
    with pytest.raises(GeneratorError, match="last dim"):
        g.create("Softmax", A, 0)
    # the graph is still usable
    B = g.create("PlaceHolder", [4, 8], "float32")
    g.create("Matmul", A, B)
    ok, msg = gen.verify(0)
    assert ok, msg


@pytest.mark.parametrize("shape,ishape,axis", [((2, 5, 8), (2, 3), 1), ((6, 4), (3,), 0), ((3, 7), (4,), 1), ((3, 7), (4,), -1),
                                                ((4, 5, 6), (1,), 1)])
def test_gather_nest_equals_oracle(shape, ishape, axis):
    """Gather (reference: Operators.cc:1253-1352): the axis is replaced by the index dimensions, a single
    index drops it; the index is read by affine.load and addresses a memref.load."""
    gen, g = new_graph()
    X = g.create("PlaceHolder", list(shape), "float32")
    I = g.create("PlaceHolder", list(ishape), "index")
    g.create("Gather", X, I, axis)
    ok, msg = gen.verify(0)
    assert ok, msg
    text = g.dump()
    a = axis % len(shape)
    name = "Gather_" + "_".join(map(str, shape)) + "_indices_" + "_".join(map(str, ishape)) + "_axis_%d" % a
    assert "func.func @%s(" % name in text and text.count("memref.load") == 1
    x = O.normal(shape, stream=61)
    rng = np.random.RandomState(7)
    idx = rng.randint(0, shape[a], size=ishape)
    ref = O.gather(x, idx, axis)
    assert np.array_equal(gen.interpret([x, idx.astype(np.float32)], ref.shape, which=0), ref)


def test_gather_errors():
    gen, g = new_graph()
    X = g.create("PlaceHolder", [4, 6], "float32")
    I = g.create("PlaceHolder", [3], "index")
    F = g.create("PlaceHolder", [3], "float32")
    with pytest.raises(GeneratorError, match="axis is greater"):
        g.create("Gather", X, I, 2)
    with pytest.raises(GeneratorError, match="index"):
        g.create("Gather", X, F, 0)
    # an index outside the axis traps in the interpreter instead of reading a neighbour
    g.create("Gather", X, I, 0)
    with pytest.raises(GeneratorError, match="outside dimension"):
        gen.interpret([O.normal((4, 6), stream=62), np.array([0, 4, 1], dtype=np.float32)], (3, 6), which=0)

