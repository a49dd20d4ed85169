"""GPU parity on shapes nobody chose: every GEMM family in every operand layout, and the attention kernel, on extents
drawn from a seeded generator (small integers as operands, so that every sum is exact and the comparison with the plain
nest is bit for bit whatever tile, edge guard and summation order the kernel picks)."""
import numpy as np
import pytest

import oracle_lib as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def ops():
    from kernelcodegen_amd import ops as _ops
    from kernelcodegen_amd._lib import lib, check
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    return _ops


def _shapes(seed, count, hi):
    rs = np.random.RandomState(seed)
    return [tuple(int(v) for v in rs.randint(1, hi, size=3)) for _ in range(count)]


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("family", ["f32", "f64", "bf16", "f16", "fp8"])
def test_gemm_random_extents_exact(ops, family, ta, tb):
    seed = {"f32": 1, "f64": 2, "bf16": 3, "f16": 4, "fp8": 5}[family] * 16 + ta * 2 + tb
    rs = np.random.RandomState(1000 + seed)
    for (m, n, k) in _shapes(seed, 3, 420):
        lim = 8 if family != "fp8" else 4           # |sum| < 420 * 64: exact in every accumulator type
        a = rs.randint(-lim, lim + 1, size=(k, m) if ta else (m, k)).astype(np.float32)
        b = rs.randint(-lim, lim + 1, size=(n, k) if tb else (k, n)).astype(np.float32)
        want = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        print("random gemm", family, (m, n, k), ta, tb, flush=True)
        if family == "fp8":
            c = ops.matmul_fp8(dev(O.to_fp8_bits(a)).view(torch.float8_e4m3fn), dev(O.to_fp8_bits(b)).view(torch.float8_e4m3fn),
                               1.0, 1.0, trans_a=bool(ta), trans_b=bool(tb))
        else:
            tdt = {"f32": torch.float32, "f64": torch.float64, "bf16": torch.bfloat16, "f16": torch.float16}[family]
            c = ops.matmul(dev(a).to(tdt), dev(b).to(tdt), trans_a=bool(ta), trans_b=bool(tb))
        assert tuple(c.shape) == (m, n)
        assert np.array_equal(c.double().cpu().numpy(), want), (family, m, n, k, ta, tb)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_random_extents(ops, dtype, causal):
    """Sequence lengths and head dims drawn at random (head dims from the multiples of 32), against fp64 attention on the
    same rounded operands: 1e-2 for the 16-bit result."""
    seed = 77 + int(causal) + 2 * int(dtype == torch.float16)
    rs = np.random.RandomState(seed)
    for _ in range(3):
        b, h = int(rs.randint(1, 4)), int(rs.randint(1, 5))
        s, d = int(rs.randint(1, 700)), int(rs.choice([32, 64, 96, 128, 160, 256]))
        shp = (b, h, s, d)
        rnd = O.round_bf16 if dtype == torch.bfloat16 else (lambda t: t.astype(np.float16).astype(np.float32))
        q, k, v = (rnd(O.normal(shp, stream=int(rs.randint(1, 1 << 20)))) for _ in range(3))
        print("random attention", shp, dtype, causal, flush=True)
        o = ops.fmha(dev(q).to(dtype), dev(k).to(dtype), dev(v).to(dtype), causal=causal)
        truth = O.fmha_f64(q, k, v, scale=d ** -0.5, causal=causal)
        got = o.float().cpu().numpy()
        assert got.shape == shp and np.isfinite(got).all()
        assert O.rel_frobenius(got, truth) <= 1e-2, shp


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_row_operators_random_extents(ops, seed):
    """LayerNorm (+GELU), softmax and an elementwise map on random row counts and row lengths (odd lengths take the
    scalar paths, long rows several wavefronts or the streamed kernel): 1e-5 against the naive nests."""
    rs = np.random.RandomState(seed)
    for _ in range(3):
        rows, n = int(rs.randint(1, 300)), int(rs.choice([int(rs.randint(1, 64)), int(rs.randint(64, 3000)), int(rs.randint(3000, 40000))]))
        x = O.normal((rows, n), stream=int(rs.randint(1, 1 << 20)))
        g = O.uniform((n,), stream=int(rs.randint(1, 1 << 20)), lo=0.5, hi=1.5)
        b = O.uniform((n,), stream=int(rs.randint(1, 1 << 20)), lo=-0.1, hi=0.1)
        gelu = bool(rs.randint(0, 2))
        print("random rows", (rows, n), gelu, flush=True)
        y = ops.layernorm(dev(x), dev(g), dev(b), 1, 1e-5, gelu=gelu).cpu().numpy()
        ref = O.layernorm(x, g, b, 1)
        ref = O.elementwise(ref, "Gelu") if gelu else ref
        assert O.rel_frobenius(y, ref) <= 1e-5, (rows, n, gelu)
        p = ops.softmax(dev(x)).cpu().numpy()
        assert O.rel_frobenius(p, O.softmax_f64(x)) <= 1e-5, (rows, n)
        t = ops.elementwise(dev(x), "Tanh").cpu().numpy()
        assert O.rel_frobenius(t, O.elementwise(x, "Tanh")) <= 1e-5


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_binary_and_gather_random_extents_exact(ops, seed):
    """Broadcast binary operators and Gather on random shapes, bit for bit against numpy (one IEEE operation per element;
    bytes moved)."""
    rs = np.random.RandomState(seed)
    for _ in range(4):
        rank = int(rs.randint(1, 5))
        full = [int(rs.randint(1, 40)) for _ in range(rank)]
        sa = [d if rs.randint(0, 3) else 1 for d in full]
        sb = [d if rs.randint(0, 3) else 1 for d in full][int(rs.randint(0, rank)):]        # fewer leading dims, some of them 1
        x, y = O.normal(tuple(sa), stream=int(rs.randint(1, 1 << 20))), O.normal(tuple(sb), stream=int(rs.randint(1, 1 << 20)))
        op = ["Add", "Sub", "Mul", "Div"][int(rs.randint(0, 4))]
        print("random binary", op, sa, sb, flush=True)
        z = ops.binary(dev(x), dev(y), op).cpu().numpy()
        want = {"Add": x + y, "Sub": x - y, "Mul": x * y, "Div": x / y}[op]
        assert z.shape == want.shape and np.array_equal(z, want), (op, sa, sb)
    for _ in range(3):
        shape = [int(rs.randint(1, 30)) for _ in range(int(rs.randint(1, 4)))]
        axis = int(rs.randint(0, len(shape)))
        idx = rs.randint(0, shape[axis], size=tuple(int(v) for v in rs.randint(1, 9, size=int(rs.randint(1, 3))))).astype(np.int64)
        x = O.normal(tuple(shape), stream=int(rs.randint(1, 1 << 20)))
        print("random gather", shape, axis, idx.shape, flush=True)
        got = ops.gather(dev(x), dev(idx), axis).cpu().numpy()
        want = np.take(x, idx, axis=axis)
        if idx.shape == (1,):
            want = np.squeeze(want, axis=axis)
        assert got.shape == want.shape and np.array_equal(got, want), (shape, axis, idx.shape)


@pytest.mark.parametrize("rows,n,dtype,inplace", [(4, 151936, torch.float32, False), (3, 33369, torch.float32, True),
                                                  (2, 200002, torch.float16, False), (5, 131076, torch.float16, True)])
def test_softmax_rows_too_long_for_registers(ops, rows, n, dtype, inplace):
    """Rows beyond 32 vectors per lane of a 1024-lane team (a vocabulary's worth of logits) take the streamed kernel:
    two passes, a running maximum with rescaled sums in the first.  Large and spread logits, so that the maximum moves
    often; against exp(x - max) / sum in fp64."""
    x = O.normal((rows, n), stream=31 + rows) * 6.0
    x[:, n // 2] += 40.0                     # the maximum sits in the middle of the row: sums are rescaled late
    if dtype == torch.float16:
        x = x.astype(np.float16).astype(np.float32)
    print("long softmax", rows, n, dtype, inplace, flush=True)
    got = ops.softmax(dev(x).to(dtype), inplace=inplace).float().cpu().numpy()
    want = O.softmax_f64(x)
    assert np.isfinite(got).all() and abs(got.sum(axis=1) - 1.0).max() <= (2e-3 if dtype == torch.float16 else 1e-4)
    assert O.rel_frobenius(got, want) <= (1e-3 if dtype == torch.float16 else 1e-5)


@pytest.mark.parametrize("rows,n,masked", [(3, 151936, 8192), (2, 140001, 3000), (2, 262144, 200000)])
def test_streamed_softmax_with_a_masked_prefix(ops, rows, n, masked):
    """A row whose first elements are -inf (left padding, a sliding window): those count as exp(-inf) = 0, as in the
    reference nest's exp(x) / sum exp(x) (`src/Frontend/Operators.cc:529-570`), also while a thread has seen nothing
    else yet (its running maximum is still -inf then).  Rows of 4-element vectors and a row length that forces
    single elements; one row masked entirely but for its last element; against fp64."""
    x = O.normal((rows, n), stream=77 + rows) * 3.0
    x[:, :masked] = -np.inf
    x[0, 5::7] = -np.inf                       # and scattered through the rest of one row
    x[rows - 1, :n - 1] = -np.inf              # a row with one finite element: the result is that element's 1.0
    print("masked softmax", rows, n, masked, flush=True)
    got = ops.softmax(dev(x), inplace=False).cpu().numpy()
    want = O.softmax_f64(x)
    assert np.isfinite(got).all()
    assert abs(got.sum(axis=1) - 1.0).max() <= 1e-4
    assert (got[:, :masked] == 0.0).all() and got[rows - 1, n - 1] == 1.0
    assert O.rel_frobenius(got, want) <= 1e-5


def _run_graph(desc, inputs, lowering=None):
    from kernelcodegen_amd.importer import import_graph, run_graph
    gen, g, _ = import_graph(desc)
    gen.optimize(g)
    if lowering:
        gen.setLowering(lowering)
    out = run_graph(gen, inputs)
    torch.cuda.synchronize()
    assert gen.skippedFunctions() == [], gen.skippedFunctions()
    return out["result"], gen


@pytest.mark.parametrize("lowering", [None, "schedule"])
@pytest.mark.parametrize("seed", [31, 32, 33])
def test_generator_path_random_graphs(ops, seed, lowering):
    """Graphs with random extents through the whole generator path (import, optimize, codegen with either lowering,
    hipRTC, launch on the plan's buffers): products of extents no tile divides, batched products, LayerNorm over a
    random axis followed by GELU, softmax, broadcast binary chains, gather.  Against numpy / the naive nests."""
    rs = np.random.RandomState(seed)
    st = lambda: int(rs.randint(1, 1 << 20))
    # product (+ Relu)
    m, n, k = (int(v) for v in rs.randint(1, 200, size=3))
    a, b = O.uniform((m, k), st()), O.uniform((k, n), st())
    desc = {"inputs": [{"name": "a", "shape": [m, k]}, {"name": "b", "shape": [k, n]}],
            "nodes": [{"op": "MatMul", "inputs": ["a", "b"], "output": "c"}, {"op": "Relu", "inputs": ["c"], "output": "c"}]}
    print("random graph: matmul+relu", (m, n, k), lowering, flush=True)
    got, _ = _run_graph(desc, [dev(a), dev(b)], lowering)
    assert O.rel_frobenius(got.cpu().numpy(), np.maximum(a.astype(np.float64) @ b.astype(np.float64), 0)) <= 1e-5
    # batched product, second operand transposed or not
    bt, m, n, k = int(rs.randint(1, 5)), *(int(v) for v in rs.randint(1, 100, size=3))
    tb = int(rs.randint(0, 2))
    a, b = O.uniform((bt, m, k), st()), O.uniform((bt, n, k) if tb else (bt, k, n), st())
    desc = {"inputs": [{"name": "a", "shape": list(a.shape)}, {"name": "b", "shape": list(b.shape)}],
            "nodes": [{"op": "MatMul", "inputs": ["a", "b"], "output": "c", "transB": tb}]}
    print("random graph: batched matmul", a.shape, b.shape, tb, lowering, flush=True)
    got, _ = _run_graph(desc, [dev(a), dev(b)], lowering)
    want = np.matmul(a.astype(np.float64), (np.swapaxes(b, 1, 2) if tb else b).astype(np.float64))
    assert O.rel_frobenius(got.cpu().numpy(), want) <= 1e-5
    # LayerNorm over the trailing axes from a random one, then GELU
    shape = [int(v) for v in rs.randint(1, 40, size=3)]
    axis = int(rs.randint(1, 3))
    x, g_, b_ = O.normal(tuple(shape), st()), O.uniform(tuple(shape[axis:]), st(), 0.5, 1.5), O.uniform(tuple(shape[axis:]), st(), -0.1, 0.1)
    desc = {"inputs": [{"name": "x", "shape": shape}, {"name": "g", "shape": shape[axis:]}, {"name": "b", "shape": shape[axis:]}],
            "nodes": [{"op": "LayerNormalization", "inputs": ["x", "g", "b"], "output": "y", "axis": axis, "epsilon": 1e-5},
                      {"op": "Gelu", "inputs": ["y"], "output": "z"}]}
    print("random graph: layernorm+gelu", shape, axis, lowering, flush=True)
    got, _ = _run_graph(desc, [dev(x), dev(g_), dev(b_)], lowering)
    assert O.rel_frobenius(got.cpu().numpy(), O.elementwise(O.layernorm(x, g_, b_, axis), "Gelu")) <= 1e-5
    # softmax after a broadcast binary chain
    rows, n = int(rs.randint(1, 70)), int(rs.randint(1, 900))
    x, bias, sc = O.normal((rows, n), st()), O.normal((n,), st()), O.uniform((rows, 1), st(), 0.5, 2.0)
    desc = {"inputs": [{"name": "x", "shape": [rows, n]}, {"name": "bias", "shape": [n]}, {"name": "sc", "shape": [rows, 1]}],
            "nodes": [{"op": "Add", "inputs": ["x", "bias"], "output": "t"}, {"op": "Mul", "inputs": ["t", "sc"], "output": "u"},
                      {"op": "Softmax", "inputs": ["u"], "output": "p"}]}
    print("random graph: add, mul, softmax", (rows, n), lowering, flush=True)
    got, _ = _run_graph(desc, [dev(x), dev(bias), dev(sc)], lowering)
    assert O.rel_frobenius(got.cpu().numpy(), O.softmax_f64((x + bias) * sc)) <= 1e-5
    # gather of random rows, then Tanh
    vocab, hidden, count = int(rs.randint(2, 500)), int(rs.randint(1, 300)), int(rs.randint(1, 200))
    table, idx = O.normal((vocab, hidden), st()), rs.randint(0, vocab, size=count).astype(np.int64)
    desc = {"inputs": [{"name": "table", "shape": [vocab, hidden]}, {"name": "idx", "shape": [count], "dtype": "index"}],
            "nodes": [{"op": "Gather", "inputs": ["table", "idx"], "output": "x", "axis": 0}, {"op": "Tanh", "inputs": ["x"], "output": "y"}]}
    print("random graph: gather, tanh", (vocab, hidden, count), lowering, flush=True)
    got, _ = _run_graph(desc, [dev(table), dev(idx)], lowering)
    assert O.rel_frobenius(got.cpu().numpy(), O.elementwise(table[idx], "Tanh")) <= 1e-5


@pytest.mark.parametrize("seed", [41, 42, 43])
def test_generator_path_random_attention(ops, seed):
    """The attention fusion on random extents through the generator: bf16 graphs get the attention family (any sequence
    length, head dims from the multiples of 32), fp32 graphs the fused schedule printed statement by statement (any
    head dim); masked or not, with or without the 1/sqrt(d) factor."""
    from kernelcodegen_amd.importer import import_graph, run_graph
    rs = np.random.RandomState(seed)
    for dtype in ("bfloat16", "float32"):
        b, h = int(rs.randint(1, 3)), int(rs.randint(1, 4))
        if dtype == "bfloat16":
            s, d = int(rs.randint(1, 600)), int(rs.choice([32, 64, 128]))
        else:
            s, d = int(rs.randint(1, 90)), int(rs.randint(1, 40))
        causal, scaled = int(rs.randint(0, 2)), int(rs.randint(0, 2))
        shp = [b, h, s, d]
        desc = {"name": "attn", "inputs": [{"name": n, "shape": shp, "dtype": dtype} for n in "qkv"],
                "nodes": [{"op": "MatMul", "inputs": ["q", "k"], "output": "s", "transB": 1},
                          {"op": "Softmax", "inputs": ["s"], "output": "p"},
                          {"op": "MatMul", "inputs": ["p", "v"], "output": "o"}]}
        gen, g, _ = import_graph(desc)
        gen.setConfigs("FMHA", [{"BLOCK_SIZE": int(rs.choice([32, 64, 128])), "CAUSAL": causal, "SCALE_RSQRT_D": scaled}])
        gen.optimize(g)
        rnd = O.round_bf16 if dtype == "bfloat16" else (lambda t: t)
        q, k, v = (rnd(O.normal(tuple(shp), stream=int(rs.randint(1, 1 << 20)), std=0.5)) for _ in range(3))
        tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        print("random attention graph", shp, dtype, causal, scaled, flush=True)
        out = run_graph(gen, [dev(t).to(tdt) for t in (q, k, v)])
        torch.cuda.synchronize()
        (info,) = gen.launchInfos()
        assert info["function"].startswith("Fused_Multi_Head_Attention")
        assert info["lowering"] == ("family fmha_bf16" if dtype == "bfloat16" else info["lowering"]) and (dtype == "bfloat16" or info["lowering"].startswith("schedule"))
        truth = O.fmha_f64(q, k, v, scale=d ** -0.5 if scaled else 1.0, causal=bool(causal))
        assert O.rel_frobenius(out["result"].float().cpu().numpy(), truth) <= (1e-2 if dtype == "bfloat16" else 1e-5), (shp, dtype)


@pytest.mark.parametrize("lowering", [None, "schedule"])
def test_generator_path_single_row_operators(ops, lowering):
    """Softmax of a vector, LayerNorm over the whole tensor and a Gather with one index along an inner axis through
    the generator path on the device (each found unscheduled or aborting by random graphs)."""
    x = O.normal((1000,), 51)
    got, _ = _run_graph({"inputs": [{"name": "x", "shape": [1000]}], "nodes": [{"op": "Softmax", "inputs": ["x"], "output": "p"}]},
                        [dev(x)], lowering)
    assert O.rel_frobenius(got.cpu().numpy(), O.softmax_f64(x)) <= 1e-5
    x, g_, b_ = O.normal((24, 40), 52), O.uniform((24, 40), 53, 0.5, 1.5), O.uniform((24, 40), 54, -0.1, 0.1)
    desc = {"inputs": [{"name": n, "shape": [24, 40]} for n in ("x", "g", "b")],
            "nodes": [{"op": "LayerNormalization", "inputs": ["x", "g", "b"], "output": "y", "axis": 0, "epsilon": 1e-5}]}
    got, _ = _run_graph(desc, [dev(x), dev(g_), dev(b_)], lowering)
    assert O.rel_frobenius(got.cpu().numpy(), O.layernorm(x, g_, b_, 0)) <= 1e-5
    table, idx = O.normal((30, 17), 55), np.array([11], dtype=np.int64)
    desc = {"inputs": [{"name": "t", "shape": [30, 17]}, {"name": "i", "shape": [1], "dtype": "index"}],
            "nodes": [{"op": "Gather", "inputs": ["t", "i"], "output": "x", "axis": 1}]}
    got, _ = _run_graph(desc, [dev(table), dev(idx)], lowering)
    assert np.array_equal(got.cpu().numpy(), table[:, 11])


@pytest.mark.parametrize("rows,n", [(7, 662), (33, 549), (64, 4096), (3, 140000)])
def test_row_operators_on_bfloat16_compute_in_fp32(ops, rows, n):
    """LayerNorm and softmax on bfloat16 tensors: bf16 in memory, fp32 arithmetic (the families' F16 = 2).  Through the
    schedule lowering these used to run the naive nest's bf16 additions, whose row sums lose most of their terms
    (relative error 4-17 % on rows of 500-700 elements); against fp64 on the same rounded operands the result is now
    within the rounding of its bf16 result."""
    x = O.round_bf16(O.normal((rows, n), stream=61))
    xd = dev(x).to(torch.bfloat16)
    p = ops.softmax(xd)
    assert p.dtype == torch.bfloat16
    assert O.rel_frobenius(p.float().cpu().numpy(), O.softmax_f64(x)) <= 4e-3
    if n <= 32768:
        g, b = O.round_bf16(O.uniform((n,), 62, 0.5, 1.5)), O.round_bf16(O.uniform((n,), 63, -0.1, 0.1))
        y = ops.layernorm(xd, dev(g).to(torch.bfloat16), dev(b).to(torch.bfloat16), 1, 1e-5)
        assert y.dtype == torch.bfloat16
        assert O.rel_frobenius(y.float().cpu().numpy(), O.layernorm_f64(x, g, b, 1)) <= 4e-3
        # the same through the generator path: the families take the bf16 graph
        desc = {"inputs": [{"name": "x", "shape": [rows, n], "dtype": "bfloat16"}, {"name": "g", "shape": [n], "dtype": "bfloat16"},
                           {"name": "b", "shape": [n], "dtype": "bfloat16"}],
                "nodes": [{"op": "LayerNormalization", "inputs": ["x", "g", "b"], "output": "y", "axis": 1, "epsilon": 1e-5},
                          {"op": "Softmax", "inputs": ["y"], "output": "p"}]}
        got, gen = _run_graph(desc, [xd, dev(g).to(torch.bfloat16), dev(b).to(torch.bfloat16)])
        assert sorted(i["lowering"] for i in gen.launchInfos()) == ["family layernorm", "family softmax"]
        want = O.softmax_f64(O.round_bf16(O.layernorm_f64(x, g, b, 1).astype(np.float32)))
        assert O.rel_frobenius(got.float().cpu().numpy(), want) <= 1e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_layernorm_rows_too_long_for_registers_in_16_bit_storage(ops, dtype):
    """The streamed three-pass LayerNorm (rows beyond 32 vectors per lane of 1024 lanes) on IEEE half and bfloat16
    tensors: 16 bits in memory, fp32 arithmetic; vector and scalar paths, with and without GELU."""
    for n, gelu in ((150000, True), (140001, False)):
        rnd = O.round_bf16 if dtype == torch.bfloat16 else (lambda t: t.astype(np.float16).astype(np.float32))
        x, g, b = rnd(O.normal((3, n), 71)), rnd(O.uniform((n,), 72, 0.5, 1.5)), rnd(O.uniform((n,), 73, -0.1, 0.1))
        y = ops.layernorm(dev(x).to(dtype), dev(g).to(dtype), dev(b).to(dtype), 1, 1e-5, gelu=gelu)
        want = O.layernorm_f64(x, g, b, 1)
        want = O.gelu_f64(want.astype(np.float32)) if gelu else want
        assert y.dtype == dtype
        assert O.rel_frobenius(y.float().cpu().numpy(), want) <= (4e-3 if dtype == torch.bfloat16 else 1e-3)


@pytest.mark.parametrize("op", ["Gelu", "Tanh", "Relu", "Sqrt", "Log"])
def test_elementwise_maps_on_bfloat16_compute_in_fp32(ops, op):
    """The elementwise family on bfloat16 tensors (bf16 in memory, the map in fp32, one rounding at the end), from ops
    and from a bf16 graph: within the rounding of the bf16 result of the fp64 map on the same operands."""
    from kernelcodegen_amd.importer import import_graph, run_graph
    x = O.round_bf16(np.abs(O.normal((37, 1001), 81)) + 0.1 if op in ("Sqrt", "Log") else O.normal((37, 1001), 81))
    want = {"Gelu": lambda t: O.gelu_f64(t), "Tanh": np.tanh, "Relu": lambda t: np.maximum(t, 0), "Sqrt": np.sqrt, "Log": np.log}[op](x.astype(np.float64))
    xd = dev(x).to(torch.bfloat16)
    y = ops.elementwise(xd, op)
    assert y.dtype == torch.bfloat16
    assert O.rel_frobenius(y.float().cpu().numpy(), want) <= 4e-3
    if op != "Relu":          # (Relu is a builder of its own in the graph vocabulary)
        gen, g, _ = import_graph({"inputs": [{"name": "x", "shape": [37, 1001], "dtype": "bfloat16"}],
                                  "nodes": [{"op": op, "inputs": ["x"], "output": "y"}]})
        gen.optimize(g)
        out = run_graph(gen, [xd])
        torch.cuda.synchronize()
        assert [i["lowering"] for i in gen.launchInfos()] == ["family elementwise"]
        assert O.rel_frobenius(out["result"].float().cpu().numpy(), want) <= 4e-3
