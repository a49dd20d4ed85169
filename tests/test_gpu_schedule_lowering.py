"""The schedules themselves on the device.  With lowering "schedule" the backend prints the scheduled function body
one statement per operation (the reference's own way, src/Backend/CUDA.cc:61-1184) instead of choosing a kernel family,
so every Rewriter primitive an optimizer used (split, reorder, parallel, cache_read/write, vectorize, pipeline with its
double buffers, barriers, bufferized loop-carried values) runs as emitted.  The kernel is compared with the host
interpreter running the same body and with the CPU oracle: bit for bit where the body holds only +, -, *, / and sqrt
(the kernel is compiled without floating-point contraction and HIP's division and square root are correctly rounded),
within the fp32 bar (1e-5 relative Frobenius, in fact tighter) where it calls exp, tanh or pow."""
import numpy as np
import pytest

import oracle_lib as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from kernelcodegen_amd.generator import KernelCodeGenerator, Layout, MemorySpace  # noqa: E402

# With a device present optimize() times its candidate configs and keeps the fastest, so every test names the one
# config it means.
BIG_GEMM = {"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 16, "THREAD_SIZE_M": 8, "THREAD_SIZE_N": 8,
            "VECTORIZE_WIDTH": 4, "WARP_SIZE": 64}
SMALL_GEMM = {"BLOCK_SIZE_M": 32, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 8, "THREAD_SIZE_M": 4, "THREAD_SIZE_N": 4,
              "VECTORIZE_WIDTH": 4, "WARP_SIZE": 64}


@pytest.fixture(scope="module")
def rt():
    from kernelcodegen_amd import runtime as R
    from kernelcodegen_amd._lib import lib, check
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    return R


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.to(dtype) if dtype is not None else t


def lower_and_run(rt, gen, graph, args):
    """optimize, print the schedule as a kernel, compile, launch the single kernel with `args`."""
    module = gen.optimize(graph)
    ok, msg = gen.verify(1)
    assert ok, msg
    gen.setLowering("schedule")
    src = gen.codegen(module)
    (info,) = gen.launchInfos()
    body = src[src.index("KCG_SCHEDULE_HELPERS"):]
    assert "mfma" not in body and "extern \"C\" __global__" in body       # the schedule, not a kernel family
    assert len(args) == info["num_args"]
    for t, nbytes in zip(args, info["arg_bytes"]):
        assert t.numel() * t.element_size() == nbytes
    mod = rt.compile_source(src, [info])
    mod.kernel(info["name"]).launch(*args)
    torch.cuda.synchronize()
    return body, info


@pytest.mark.parametrize("m,n,k,cfg", [(256, 256, 128, BIG_GEMM), (128, 384, 64, BIG_GEMM), (64, 96, 40, SMALL_GEMM),
                                       (96, 64, 24, dict(SMALL_GEMM, WARP_SIZE=32))])
def test_matmul_schedule_runs_bit_exact(rt, m, n, k, cfg):
    a, b = O.uniform((m, k), 301), O.uniform((k, n), 302)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("Matmul", [cfg])
    g = gen.createGraph("mm")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [m, k], "float32")
    B = g.create("PlaceHolder", [k, n], "float32")
    g.create("Matmul", A, B)
    c = torch.full((m, n), float("nan"), device="cuda")
    body, info = lower_and_run(rt, gen, g, [dev(a), dev(b), c])
    bm, tm = cfg["BLOCK_SIZE_M"], cfg["THREAD_SIZE_M"]
    assert info["grid"] == [n // bm, m // bm, 1] and info["block"] == [bm // tm, bm // tm, 1]
    assert body.count("__shared__") == 2 and "__syncthreads();" in body and "kcg_v4_float" in body
    got = c.cpu().numpy()
    assert np.array_equal(got, O.matmul(a, b))                      # the reference nest: sequential k, mul then add
    assert np.array_equal(got, gen.interpret([a, b], (m, n), which=1))


@pytest.mark.parametrize("la,lb", [(0, 0), (0, 1), (1, 0)])
def test_batched_matmul_schedule_runs_bit_exact(rt, la, lb):
    batch, m, n, k = (2, 3), 128, 128, 32
    a = O.uniform(batch + ((k, m) if la else (m, k)), 303)
    b = O.uniform(batch + ((n, k) if lb else (k, n)), 304)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("BatchMatmul", [BIG_GEMM])
    g = gen.createGraph("bmm")
    gen.opts.append("BatchMatmul")
    A = g.create("PlaceHolder", list(a.shape), "float32")
    B = g.create("PlaceHolder", list(b.shape), "float32")
    g.create("BatchedMatmul", A, Layout.colMajor if la else Layout.rowMajor, B, Layout.colMajor if lb else Layout.rowMajor)
    c = torch.full(batch + (m, n), float("nan"), device="cuda")
    lower_and_run(rt, gen, g, [dev(a), dev(b), c])
    got = c.cpu().numpy()
    am = np.swapaxes(a, -1, -2) if la else a
    bm_ = np.swapaxes(b, -1, -2) if lb else b
    assert np.array_equal(got, gen.interpret([a, b], got.shape, which=1))
    assert O.rel_frobenius(got, np.matmul(am.astype(np.float64), bm_.astype(np.float64))) <= 1e-6


@pytest.mark.parametrize("shape,axis,gshape,tpr", [((6, 256), 1, (256,), 64), ((3, 2, 16, 32), 2, (16, 32), 128),
                                                   ((64, 1024), 1, (1024,), 256)])
def test_layernorm_schedule_runs_bit_exact(rt, shape, axis, gshape, tpr):
    x, gamma, beta = O.normal(shape, 305), O.uniform(gshape, 306, 0.5, 1.5), O.uniform(gshape, 307, -0.1, 0.1)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("LayerNorm", [{"BLOCK_SIZE": tpr * 4, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4}])
    g = gen.createGraph("ln")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", list(shape), "float32")
    S = g.create("PlaceHolder", list(gshape), "float32")
    Bv = g.create("PlaceHolder", list(gshape), "float32")
    g.create("LayerNorm", X, S, Bv, axis, 1e-5)
    y = torch.full(shape, float("nan"), device="cuda")
    body, info = lower_and_run(rt, gen, g, [dev(x), dev(gamma), dev(beta), y])
    assert info["block"][0] == tpr and body.count("__syncthreads();") == 2 and " / " in body and "sqrtf(" in body
    got = y.cpu().numpy()
    # the schedule's order of additions (per-thread partial sums, then the partials in thread order) is the
    # interpreter's; the oracle adds along the row, so it agrees to rounding only
    assert np.array_equal(got, gen.interpret([x, gamma, beta], shape, which=1))
    assert O.rel_frobenius(got, O.layernorm_f64(x, gamma, beta, len(shape) - len(gshape), 1e-5)) <= 1e-6


@pytest.mark.parametrize("shape,op,ms", [((2, 48, 64), "Gelu", MemorySpace.global_), ((6, 10), "Relu", MemorySpace.inplace),
                                         ((3, 5, 7), "Tanh", MemorySpace.global_), ((256, 512), "Gelu", MemorySpace.inplace)])
def test_elementwise_schedule_runs(rt, shape, op, ms):
    x = O.normal(shape, 308)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ew")
    gen.opts.append("ElementWise")
    X = g.create("PlaceHolder", list(shape), "float32")
    g.create("ElementWise", X, op, ms)
    xin = dev(x)
    y = xin if ms == MemorySpace.inplace else torch.full(shape, float("nan"), device="cuda")
    lower_and_run(rt, gen, g, [xin] if ms == MemorySpace.inplace else [xin, y])
    got, ref = y.cpu().numpy(), O.elementwise(x, op)
    if op == "Relu":
        assert np.array_equal(got, ref)
    else:
        assert O.rel_frobenius(got, ref) <= 1e-6          # the device's tanhf against the host's


@pytest.mark.parametrize("shape", [(4, 6, 512), (3, 100), (5, 1001)])
def test_softmax_schedule_runs(rt, shape):
    x = O.normal(shape, stream=309, std=2.0)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("softmax")
    gen.opts.append("Softmax")
    X = g.create("PlaceHolder", list(shape), "float32")
    g.create("Softmax", X, -1, MemorySpace.inplace)
    y = dev(x)
    lower_and_run(rt, gen, g, [y])
    got = y.cpu().numpy()
    assert O.rel_frobenius(got, O.softmax_f64(x)) <= 1e-6
    assert np.allclose(got.sum(-1), 1.0, atol=1e-5)


@pytest.mark.parametrize("sa,sb,op", [((16, 1, 1, 64), (1, 8, 64), "Add"), ((4, 6), (6,), "Mul"), ((3, 5, 7), (3, 5, 7), "Sub"),
                                      ((8, 12), (8, 1), "Div"), ((64, 512), (512,), "Pow"), ((4, 8), (8,), "Equal"),
                                      ((4, 8), (8,), "Greater")])
def test_binary_schedule_runs(rt, sa, sb, op):
    compare = op in ("Equal", "Greater")
    if compare:
        x, y = np.round(O.normal(sa, 53)), np.round(O.normal(sb, 54))
    else:
        x, y = O.uniform(sa, 310, 0.5, 2.0), O.uniform(sb, 311, 0.5, 2.0)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("bin")
    gen.opts.append("Binary")
    X = g.create("PlaceHolder", list(sa), "float32")
    Y = g.create("PlaceHolder", list(sb), "float32")
    g.create("Binary", X, Y, op)
    ref = {"Add": lambda: x + y, "Mul": lambda: x * y, "Sub": lambda: x - y, "Div": lambda: x / y,
           "Pow": lambda: np.power(x.astype(np.float64), y.astype(np.float64)), "Equal": lambda: x == y, "Greater": lambda: x > y}[op]()
    out = torch.full(ref.shape, 77, device="cuda", dtype=torch.uint8) if compare else torch.full(ref.shape, float("nan"), device="cuda")
    lower_and_run(rt, gen, g, [dev(x), dev(y), out])
    got = out.cpu().numpy()
    if compare:
        assert ref.any() and not ref.all() and np.array_equal(got.astype(bool), ref) and set(np.unique(got)) <= {0, 1}
    elif op == "Pow":
        assert O.rel_frobenius(got, ref) <= 1e-6
    else:
        assert np.array_equal(got, ref.astype(np.float32))


@pytest.mark.parametrize("shape,ishape,axis,dtype", [((2, 5, 8), (2, 3), 1, "float32"), ((64, 32), (48,), 0, "float32"),
                                                      ((16, 24), (4, 2), 0, "bfloat16")])
def test_gather_schedule_runs(rt, shape, ishape, axis, dtype):
    x = O.normal(shape, stream=312)
    if dtype == "bfloat16":
        x = O.round_bf16(x)
    idx = np.random.RandomState(11).randint(0, shape[axis], size=ishape)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("gather")
    gen.opts.append("Gather")
    X = g.create("PlaceHolder", list(shape), dtype)
    I = g.create("PlaceHolder", list(ishape), "index")
    g.create("Gather", X, I, axis)
    ref = O.gather(x, idx, axis)
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    out = torch.full(ref.shape, float("nan"), device="cuda", dtype=tdt)
    lower_and_run(rt, gen, g, [dev(x, tdt), dev(idx.astype(np.int64)), out])
    assert np.array_equal(out.float().cpu().numpy(), ref)


@pytest.mark.parametrize("causal,scaled", [(0, 0), (1, 1)])
def test_fused_attention_schedule_runs(rt, causal, scaled):
    shp = (2, 2, 64, 16)
    q, k, v = O.normal(shp, 313), O.normal(shp, 314), O.normal(shp, 315)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [{"BLOCK_SIZE": 32, "CAUSAL": causal, "SCALE_RSQRT_D": scaled}])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    Q = g.create("PlaceHolder", list(shp), "float32")
    Kv = g.create("PlaceHolder", list(shp), "float32")
    V = g.create("PlaceHolder", list(shp), "float32")
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    o = torch.full(shp, float("nan"), device="cuda")
    body, _ = lower_and_run(rt, gen, g, [dev(q), dev(k), dev(v), o])
    assert body.count("__shared__") == 2 and body.count("__syncthreads();") == 2      # staged K and V tiles
    truth = O.fmha_f64(q, k, v, scale=1.0 / np.sqrt(16.0) if scaled else 1.0, causal=bool(causal))
    assert O.rel_frobenius(o.cpu().numpy(), truth) <= 2e-6


TILED_FMHA = {"BLOCK_SIZE": 128, "HdxBr": 128 * 64, "BrxBc": 128 * 64, "WarpX_O": 2, "Slice": 8, "BrTileS": 8, "BcTileS": 8,
              "BrTileO": 8, "HdTileO": 8, "Width": 4, "WARP_SIZE": 64}


@pytest.mark.parametrize("shp,warp,causal,scaled", [((2, 3, 512, 64), 32, 0, 0), ((2, 3, 512, 64), 64, 1, 1),
                                                    ((1, 4, 384, 128), 64, 0, 1), ((2, 2, 256, 128), 32, 1, 0)])
def test_tiled_attention_schedule_runs(rt, shp, warp, causal, scaled):
    """The reference's tiled attention schedule (src/Optimizer/Optimizer.cc:2606-2860; Q, K, V slices and the
    probabilities in shared memory, 8 x 8 register tiles from outer products, online softmax with shuffles between the
    threads that share a query), printed statement by statement and run: against fp64 attention, in the reference's
    semantics (no scale, no mask) and with both, head dims 64 and 128, 32- and 64-thread layout units."""
    q, k, v = O.normal(shp, 333), O.normal(shp, 334), O.normal(shp, 335)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [dict(TILED_FMHA, WARP_SIZE=warp, CAUSAL=causal, SCALE_RSQRT_D=scaled)])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    Q, Kv, V = (g.create("PlaceHolder", list(shp), "float32") for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    o = torch.full(shp, float("nan"), device="cuda")
    print("tiled attention schedule", shp, warp, causal, scaled, flush=True)
    body, info = lower_and_run(rt, gen, g, [dev(q), dev(k), dev(v), o])
    br = 8192 // shp[3]
    assert info["grid"] == [shp[2] // br, shp[1], shp[0]] and info["block"] == [128, 1, 1]
    assert body.count("__shared__") == 7 and body.count("__syncthreads();") == 5 and "__shfl_down" in body
    truth = O.fmha_f64(q, k, v, scale=shp[3] ** -0.5 if scaled else 1.0, causal=bool(causal))
    assert O.rel_frobenius(o.cpu().numpy(), truth) <= 2e-6


@pytest.mark.parametrize("causal", [0, 1])
def test_fused_attention_with_a_partly_filled_last_workgroup_runs(rt, causal):
    """A sequence length that the fusion's block does not divide (77 queries in workgroups of 32): the body of the
    surplus threads is under a condition, the result's guard rows stay as they were."""
    shp = (2, 2, 77, 16)
    q, k, v = O.normal(shp, 323), O.normal(shp, 324), O.normal(shp, 325)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("FMHA", [{"BLOCK_SIZE": 32, "CAUSAL": causal, "SCALE_RSQRT_D": 1}])
    g = gen.createGraph("attn")
    gen.opts.append("FMHA")
    Q, Kv, V = (g.create("PlaceHolder", list(shp), "float32") for _ in range(3))
    S = g.create("BatchedMatmul", Q, Layout.rowMajor, Kv, Layout.colMajor)
    P = g.create("Softmax", S, -1, MemorySpace.inplace)
    g.create("BatchedMatmul", P, Layout.rowMajor, V, Layout.rowMajor)
    n = int(np.prod(shp))
    buf = torch.full((n + 4096,), 7.0, device="cuda")
    body, info = lower_and_run(rt, gen, g, [dev(q), dev(k), dev(v), buf[:n]])
    assert info["grid"] == [3, 2, 2] and "__syncthreads" not in body
    assert bool((buf[n:] == 7.0).all())
    truth = O.fmha_f64(q, k, v, scale=0.25, causal=bool(causal))
    assert O.rel_frobenius(buf[:n].cpu().numpy().reshape(shp), truth) <= 2e-6


def test_layernorm_with_absorbed_gelu_and_matmul_with_absorbed_relu_run(rt):
    shape = (32, 512)
    x, gamma, beta = O.normal(shape, 316), O.uniform((512,), 317, 0.5, 1.5), O.uniform((512,), 318, -0.1, 0.1)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ln_gelu")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", list(shape), "float32")
    S = g.create("PlaceHolder", [512], "float32")
    Bv = g.create("PlaceHolder", [512], "float32")
    Y = g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    g.create("ElementWise", Y, "Gelu", MemorySpace.inplace)
    y = torch.full(shape, float("nan"), device="cuda")
    body, _ = lower_and_run(rt, gen, g, [dev(x), dev(gamma), dev(beta), y])
    assert "tanhf(" in body
    assert O.rel_frobenius(y.cpu().numpy(), O.elementwise(O.layernorm(x, gamma, beta, 1, 1e-5), "Gelu")) <= 1e-6

    a, b = O.uniform((128, 64), 319), O.uniform((64, 128), 320)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("Matmul", [BIG_GEMM])
    g = gen.createGraph("mm_relu")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [128, 64], "float32")
    B = g.create("PlaceHolder", [64, 128], "float32")
    C = g.create("Matmul", A, B)
    g.create("Relu", C, MemorySpace.inplace)
    c = torch.full((128, 128), float("nan"), device="cuda")
    lower_and_run(rt, gen, g, [dev(a), dev(b), c])
    assert np.array_equal(c.cpu().numpy(), np.maximum(O.matmul(a, b), 0.0))


def test_float64_operators_run_as_their_schedules(rt):
    """LayerNorm, elementwise, softmax and binary kernel families have no f64 form; codegen falls back to the schedule by
    itself (no setLowering needed)."""
    def run(gen, graph, args, lowering=None):
        module = gen.optimize(graph)
        assert gen.skippedFunctions() == []
        if lowering:
            gen.setLowering(lowering)
        src = gen.codegen(module)
        (info,) = gen.launchInfos()
        assert "KCG_SCHEDULE_HELPERS" in src and "double* __restrict__ arg0" in src
        rt.compile_source(src, [info]).kernel(info["name"]).launch(*args)
        torch.cuda.synchronize()

    f64 = torch.float64
    # GEMM: sequential k in double, no contraction -> the numpy loop below bit for bit
    m, n, k = 128, 192, 48
    a, b = O.uniform((m, k), 331).astype(np.float64), O.uniform((k, n), 332).astype(np.float64)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mm64")
    gen.opts.append("Matmul")
    A = g.create("PlaceHolder", [m, k], "float64")
    B = g.create("PlaceHolder", [k, n], "float64")
    g.create("Matmul", A, B)
    c = torch.full((m, n), float("nan"), device="cuda", dtype=f64)
    run(gen, g, [dev(a), dev(b), c], "schedule")          # (by default an f64 product gets the f64 MFMA family)
    want = np.zeros((m, n))
    for kk in range(k):
        want = a[:, kk:kk + 1] * b[kk:kk + 1, :] + want
    assert np.array_equal(c.cpu().numpy(), want)

    # LayerNorm, then GELU
    shape = (48, 512)
    x = O.normal(shape, 333).astype(np.float64)
    gamma, beta = O.uniform((512,), 334, 0.5, 1.5).astype(np.float64), O.uniform((512,), 335, -0.1, 0.1).astype(np.float64)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("ln64")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", list(shape), "float64")
    S = g.create("PlaceHolder", [512], "float64")
    Bv = g.create("PlaceHolder", [512], "float64")
    Y = g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    g.create("ElementWise", Y, "Gelu", MemorySpace.inplace)
    y = torch.full(shape, float("nan"), device="cuda", dtype=f64)
    run(gen, g, [dev(x), dev(gamma), dev(beta), y])
    ln = O.layernorm_f64(x, gamma, beta, 1, float(np.float32(1e-5)))
    ref = 0.5 * ln * (1.0 + np.tanh(0.797884 * (ln + 0.044715 * ln ** 3)))      # the reference's truncated constants
    assert O.rel_frobenius(y.cpu().numpy(), ref) <= 1e-7       # the constants are fp32 values widened

    # Softmax and a broadcast Binary
    xs = O.normal((6, 300), 336, std=2.0).astype(np.float64)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("sm64")
    gen.opts.append("Softmax")
    X = g.create("PlaceHolder", [6, 300], "float64")
    g.create("Softmax", X, -1, MemorySpace.inplace)
    ys = dev(xs)
    run(gen, g, [ys])
    assert O.rel_frobenius(ys.cpu().numpy(), O.softmax_f64(xs)) <= 1e-13

    p, q = O.uniform((16, 8, 64), 337, 0.5, 2.0).astype(np.float64), O.uniform((8, 1), 338, 0.5, 2.0).astype(np.float64)
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("div64")
    gen.opts.append("Binary")
    P = g.create("PlaceHolder", [16, 8, 64], "float64")
    Q = g.create("PlaceHolder", [8, 1], "float64")
    g.create("Binary", P, Q, "Div")
    r = torch.full((16, 8, 64), float("nan"), device="cuda", dtype=f64)
    run(gen, g, [dev(p), dev(q), r])
    assert np.array_equal(r.cpu().numpy(), p / q)


def test_bfloat16_binary_runs_as_its_schedule(rt):
    x, y = O.round_bf16(O.uniform((32, 256), 339, 0.5, 2.0)), O.round_bf16(O.uniform((256,), 340, 0.5, 2.0))
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("mul16")
    gen.opts.append("Binary")
    X = g.create("PlaceHolder", [32, 256], "bfloat16")
    Y = g.create("PlaceHolder", [256], "bfloat16")
    g.create("Binary", X, Y, "Mul")
    module = gen.optimize(g)
    src = gen.codegen(module)
    (info,) = gen.launchInfos()
    assert "KCG_SCHEDULE_HELPERS" in src and "__bf16* __restrict__ arg0" in src
    out = torch.zeros((32, 256), device="cuda", dtype=torch.bfloat16)
    rt.compile_source(src, [info]).kernel(info["name"]).launch(dev(x, torch.bfloat16), dev(y, torch.bfloat16), out)
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), O.round_bf16(x * y))      # one rounding of the exact product


@pytest.mark.parametrize("tpr", [256, 64])
def test_tree_reductions_with_wavefront_shuffles_run_bit_exact(rt, tpr):
    """TREE_REDUCE: the reference's reduction of the per-thread partials (src/Optimizer/Optimizer.cc:1623-1749): halving
    steps in shared memory under `if (tid < h)`, gpu.shuffle down inside the last wavefront, lane 0 adds into a shared
    cell.  The interpreter executes the same tree in the same order, so the device result equals its result."""
    shape = (12, 1024)
    x, gamma, beta = O.normal(shape, 341), O.uniform((1024,), 342, 0.5, 1.5), O.uniform((1024,), 343, -0.1, 0.1)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("LayerNorm", [{"BLOCK_SIZE": tpr * 4, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4, "TREE_REDUCE": 1}])
    g = gen.createGraph("ln_tree")
    gen.opts.append("LayerNorm")
    X = g.create("PlaceHolder", list(shape), "float32")
    S = g.create("PlaceHolder", [1024], "float32")
    Bv = g.create("PlaceHolder", [1024], "float32")
    g.create("LayerNorm", X, S, Bv, 1, 1e-5)
    y = torch.full(shape, float("nan"), device="cuda")
    body, info = lower_and_run(rt, gen, g, [dev(x), dev(gamma), dev(beta), y])
    assert info["block"][0] == tpr and body.count("__shfl_down(") == 12          # two reductions, offsets 32 ... 1
    got = y.cpu().numpy()
    assert np.array_equal(got, gen.interpret([x, gamma, beta], shape, which=1))
    assert O.rel_frobenius(got, O.layernorm_f64(x, gamma, beta, 1, 1e-5)) <= 1e-6

    xs = O.normal((5, 2048), 344, std=2.0)
    gen = KernelCodeGenerator("ROCm")
    gen.setConfigs("Softmax", [{"BLOCK_SIZE": tpr * 4, "THREAD_SIZE": 4, "VECTORIZE_WIDTH": 4, "TREE_REDUCE": 1}])
    g = gen.createGraph("sm_tree")
    gen.opts.append("Softmax")
    X = g.create("PlaceHolder", [5, 2048], "float32")
    g.create("Softmax", X, -1, MemorySpace.inplace)
    ys = dev(xs)
    body, _ = lower_and_run(rt, gen, g, [ys])
    assert body.count("__shfl_down(") == 6
    assert O.rel_frobenius(ys.cpu().numpy(), O.softmax_f64(xs)) <= 1e-6


def test_more_than_two_to_the_31_elements_are_indexed_in_64_bits(rt):
    """Index values are 32-bit like the reference's, but a buffer with more elements than that counts switches the
    whole kernel to 64-bit index arithmetic (the flattened position is an intermediate value of its index maps)."""
    rows, cols = 32769, 65536                         # 2^31 + 65536 half elements, 4.3 GB each way
    gen = KernelCodeGenerator("ROCm")
    g = gen.createGraph("big")
    gen.opts.append("ElementWise")
    X = g.create("PlaceHolder", [rows, cols], "float16")
    g.create("ElementWise", X, "Relu", MemorySpace.global_)
    x = torch.randn(rows, cols, device="cuda", dtype=torch.float16)
    y = torch.full((rows, cols), float("nan"), device="cuda", dtype=torch.float16)
    body, info = lower_and_run(rt, gen, g, [x, y])
    assert "const long i0 = (long)blockIdx.y;" in body and "for (long " in body
    assert torch.equal(y, torch.relu(x))
    assert bool((y[-1] == torch.relu(x[-1])).all()) and not bool(torch.isnan(y[-1]).any())      # past element 2^31


@pytest.mark.parametrize("m,n,k,cfg", [(100, 77, 33, BIG_GEMM), (45, 70, 9, SMALL_GEMM), (300, 520, 130, BIG_GEMM)])
def test_ragged_matmul_through_optimize_runs_both_ways(rt, m, n, k, cfg):
    """Extents that are no multiples of the tile go through optimize() (the guarded schedule): the kernel family guards
    its own edges, the statement-by-statement lowering runs the `if (m < M && n < N)` of the schedule."""
    a, b = O.uniform((m, k), 351), O.uniform((k, n), 352)
    want = O.matmul(a, b)
    for lowering in ("families", "schedule"):
        gen = KernelCodeGenerator("ROCm")
        gen.setConfigs("Matmul", [cfg])
        g = gen.createGraph("mm")
        gen.opts.append("Matmul")
        A = g.create("PlaceHolder", [m, k], "float32")
        B = g.create("PlaceHolder", [k, n], "float32")
        g.create("Matmul", A, B)
        module = gen.optimize(g)
        gen.setLowering(lowering)
        src = gen.codegen(module)
        (info,) = gen.launchInfos()
        assert info["lowering"] == ("family gemm_f32" if lowering == "families" else "schedule")
        c = torch.full((m + 1, n), float("nan"), device="cuda")          # one row more: nothing may be written there
        rt.compile_source(src, [info]).kernel(info["name"]).launch(dev(a), dev(b), c[:m])
        torch.cuda.synchronize()
        got = c.cpu().numpy()
        assert np.isnan(got[m]).all()
        if lowering == "schedule":
            assert np.array_equal(got[:m], want)                          # sequential k, mul then add, no contraction
        else:
            assert O.rel_frobenius(got[:m], O.matmul_f64(a, b)) <= 1e-5


@pytest.mark.parametrize("batch,m,n,k,la,lb", [((3,), 45, 70, 9, 0, 0), ((2, 2), 33, 40, 12, 1, 1), ((2,), 50, 31, 8, 0, 1)])
def test_ragged_batched_matmul_through_optimize_runs_both_ways(rt, batch, m, n, k, la, lb):
    a = O.uniform(batch + ((k, m) if la else (m, k)), 353)
    b = O.uniform(batch + ((n, k) if lb else (k, n)), 354)
    am = np.swapaxes(a, -1, -2) if la else a
    bm_ = np.swapaxes(b, -1, -2) if lb else b
    want = np.matmul(am.astype(np.float64), bm_.astype(np.float64))
    for lowering in ("families", "schedule"):
        gen = KernelCodeGenerator("ROCm")
        gen.setConfigs("BatchMatmul", [SMALL_GEMM])
        g = gen.createGraph("bmm")
        gen.opts.append("BatchMatmul")
        A = g.create("PlaceHolder", list(a.shape), "float32")
        B = g.create("PlaceHolder", list(b.shape), "float32")
        g.create("BatchedMatmul", A, Layout.colMajor if la else Layout.rowMajor, B, Layout.colMajor if lb else Layout.rowMajor)
        module = gen.optimize(g)
        assert "kcg.ragged = 1" in gen._dump(1)
        gen.setLowering(lowering)
        src = gen.codegen(module)
        (info,) = gen.launchInfos()
        assert gen.skippedFunctions() == []
        c = torch.full(batch + (m, n), float("nan"), device="cuda")
        rt.compile_source(src, [info]).kernel(info["name"]).launch(dev(a), dev(b), c)
        torch.cuda.synchronize()
        got = c.cpu().numpy()
        assert O.rel_frobenius(got, want) <= 1e-6
        if lowering == "schedule":
            assert np.array_equal(got, gen.interpret([a, b], got.shape, which=1))
