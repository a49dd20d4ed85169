"""GPU parity: every emitted kernel family against the CPU oracle on the same
seeded inputs, through the C ABI (emit -> hipRTC -> hipModule launch)."""
import numpy as np
import pytest

import oracle_lib as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5   # relative Frobenius error, fp32 operators
LOWP_TOL = 1e-2   # bf16 / fp8 operands against fp64 on the same rounded inputs


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    import kernelcodegen_amd as K  # noqa: F401
    from kernelcodegen_amd import ops as _ops
    from kernelcodegen_amd._lib import lib, check
    check(lib().kcg_hip_init(0), "kcg_hip_init")
    return _ops


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape,axis,gshape", [
    ((64, 4096), 1, (4096,)),       # C3 row length, vector path, one wave per row
    ((7, 1000), 1, (1000,)),        # ragged last vector
    ((5, 1001), 1, (1001,)),        # scalar path
    ((3, 24, 40), 1, (24, 40)),     # group spans two dims, gamma [24,40]
    ((3, 24, 40), 1, (40,)),        # gamma broadcast over the group
    ((2, 16384), 1, (16384,)),      # several waves per row (cross-wave reduction)
    ((4, 3, 8), 2, (8,)),           # tiny rows
])
@pytest.mark.parametrize("gelu", [False, True])
def test_layernorm_matches_oracle(ops, shape, axis, gshape, gelu):
    x = O.normal(shape, stream=101)
    g = O.uniform(gshape, stream=102, lo=0.5, hi=1.5)
    b = O.uniform(gshape, stream=103, lo=-0.1, hi=0.1)
    print("layernorm", shape, axis, gshape, gelu, flush=True)
    y = host(ops.layernorm(dev(x), dev(g), dev(b), axis, 1e-5, gelu=gelu))
    ref32 = O.layernorm(x, g, b, axis)
    ref64 = O.layernorm_f64(x, g, b, axis)
    if gelu:
        ref32 = O.elementwise(ref32, "Gelu")
        ref64 = O.gelu_f64(O.layernorm_f64(x, g, b, axis).astype(np.float32))
    assert y.shape == x.shape
    assert O.rel_frobenius(y, ref64) <= FP32_TOL
    assert O.rel_frobenius(y, ref32) <= FP32_TOL
    assert np.allclose(y, ref32, rtol=0, atol=2e-5)


def test_layernorm_known_answer(ops):
    x = np.array([[1, 2, 3, 4]], dtype=np.float32)
    g = np.array([0.5, 1.0, 1.5, 2.0], dtype=np.float32)
    b = np.array([0.1, -0.1, 0.0, 0.05], dtype=np.float32)
    y = host(ops.layernorm(dev(x), dev(g), dev(b), 1, 1e-5))
    assert np.allclose(y, [[-0.5708177090, -0.5472118258, 0.6708177328, 2.7332708836]], rtol=0, atol=5e-7)


@pytest.mark.parametrize("op", ["Tanh", "Sqrt", "Log", "Relu", "Gelu"])
@pytest.mark.parametrize("shape", [(2, 768, 768), (1001,), (3, 5, 7)])
def test_elementwise_matches_oracle(ops, op, shape):
    if op in ("Sqrt", "Log"):
        x = O.uniform(shape, stream=111, lo=0.05, hi=9.0)
    else:
        x = O.normal(shape, stream=112, std=2.0)
    print("elementwise", op, shape, flush=True)
    y = host(ops.elementwise(dev(x), op))
    ref = O.elementwise(x, op)
    assert y.shape == x.shape
    assert O.rel_frobenius(y, ref) <= FP32_TOL
    xi = dev(x)
    yi = host(ops.elementwise(xi, op, inplace=True))
    assert np.array_equal(yi, y)


def test_elementwise_cast_to_int32(ops):
    x = O.normal((2, 768, 768), stream=113, std=100.0)
    y = host(ops.elementwise(dev(x), "Cast", out_dtype=torch.int32))
    assert y.dtype == np.int32 and np.array_equal(y, np.trunc(x).astype(np.int32))


def test_gelu_known_answers(ops):
    kat = {-3.0: -0.0036373436, -1.0: -0.1588081419, -0.5: -0.1542860568, 0.0: 0.0,
           0.5: 0.3457139432, 1.0: 0.8411918879, 2.0: 1.9545974731, 3.0: 2.9963626862}
    xs = np.array(sorted(kat), dtype=np.float32)
    y = host(ops.elementwise(dev(xs), "Gelu"))
    assert np.allclose(y, [kat[float(v)] for v in xs], rtol=0, atol=1e-6)


# ---------------------------------------------------------------------------
GEMM_SHAPES = [
    (128, 128, 64), (256, 384, 128), (1024, 1024, 1024),
    (100, 77, 33), (129, 255, 17), (64, 64, 8), (33, 1, 5),
]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_matmul_f32_matches_oracle(ops, m, n, k):
    a = O.uniform((m, k), stream=121)
    b = O.uniform((k, n), stream=122)
    print("matmul f32", m, n, k, flush=True)
    c = host(ops.matmul(dev(a), dev(b)))
    truth = O.matmul_f64(a, b)
    assert c.shape == (m, n)
    assert O.rel_frobenius(c, truth) <= FP32_TOL
    assert O.rel_frobenius(c, O.matmul(a, b)) <= FP32_TOL


def test_matmul_f32_structured_operands_exact(ops):
    # A = I: C must equal B bit for bit; small integers: every partial sum is exact in fp32.
    n = 256
    b = O.uniform((n, n), stream=123)
    assert np.array_equal(host(ops.matmul(dev(np.eye(n, dtype=np.float32)), dev(b))), b)
    rng = np.random.RandomState(5)
    a = rng.randint(-3, 4, size=(192, 160)).astype(np.float32)
    bb = rng.randint(-3, 4, size=(160, 224)).astype(np.float32)
    assert np.array_equal(host(ops.matmul(dev(a), dev(bb))), O.matmul(a, bb))


T256 = dict(BM=256, BN=256)


@pytest.mark.parametrize("batch,m,n,k,cfg", [((), 256, 256, 16, T256), ((), 512, 768, 48, T256), ((2,), 256, 512, 1040, dict(T256, RELU=1)),
                                             ((), 768, 256, 4096, T256), ((), 256, 512, 96, dict(T256, BK=32)),
                                             ((), 128, 192, 64, dict(BM=64, BN=64, BK=32, WM=2, WN=2)), ((3,), 128, 64, 80, dict(BM=64, BN=64, BK=16, WM=2, WN=2)),
                                             ((), 256, 384, 160, dict(BM=128, BN=128, BK=32, WM=4, WN=4)), ((), 384, 256, 48, dict(BM=128, BN=128, BK=16, WM=4, WN=2)),
                                             ((), 256, 192, 64, dict(BM=128, BN=64, BK=32, WM=2, WN=2, RELU=1)), ((), 128, 256, 32, dict(BM=64, BN=128, BK=16, WM=2, WN=4)),
                                             ((), 384, 384, 128, dict(BM=192, BN=128, BK=32, WM=2, WN=2)),
                                             # two groups of wavefronts that split every k-tile's steps (WK), three and four LDS buffers (NBUF)
                                             ((), 128, 192, 256, dict(BM=64, BN=64, BK=32, WM=2, WN=2, WK=2, NBUF=3)),
                                             ((2,), 64, 64, 32, dict(BM=64, BN=64, BK=32, WM=2, WN=2, WK=2, NBUF=4)),
                                             ((), 128, 128, 96, dict(BM=64, BN=64, BK=32, WM=2, WN=2, WK=1, NBUF=4)),
                                             ((), 256, 256, 160, dict(BM=128, BN=128, BK=32, WM=2, WN=4, WK=2, NBUF=2, RELU=1)),
                                             ((), 256, 128, 64, dict(BM=128, BN=64, BK=32, WM=2, WN=2, WK=2, NBUF=3)),
                                             ((), 512, 256, 48, dict(T256, NBUF=3))])
def test_matmul_f32_tiles_loaded_straight_into_lds(ops, batch, m, n, k, cfg):
    """The fp32 GEMM for whole tiles of two row-major operands (tiles straight from global memory into LDS, A's rows
    swizzled on the source side and read four k at a time): 256 x 256 tiles with sixteen wavefronts, the smaller tiles
    and other wavefront grids, k-tiles of 16 and 32, one to many k-tiles, batches, the fused Relu.  Small integers make
    every partial sum exact whatever the order (the k order inside an MFMA is not the other kernel's); U(-1,1) operands
    check against fp64 within the fp32 bound and against the other kernel's result."""
    from kernelcodegen_amd import runtime as R
    nb = max(1, int(np.prod(batch)))
    text, info = R.emit_kernel("gemm_f32", "kernel0", M=m, N=n, K=k, BATCH=nb, **cfg)
    groups = cfg.get("WK", 2 if (cfg.get("BM"), cfg.get("BN"), cfg.get("BK")) == (64, 64, 32) else 1)    # small launches of 64 x 64 x 32 tiles default to two
    assert "global_load_lds_dwordx4" in text and info["block"] == [64 * cfg.get("WM", 4) * cfg.get("WN", 4) * groups, 1, 1]
    plain = {key: v for key, v in cfg.items() if key not in ("WK", "NBUF")}
    assert "global_load_lds_dwordx4" not in R.emit_kernel("gemm_f32", "kernel0", M=m, N=n, K=k, **dict(plain, D2L=0))[0]
    for kw in (dict(M=m + 8), dict(K=k + 4), dict(TA=1), dict(TB=1), dict(BK=8)):
        p = dict(M=m, N=n, K=k); p.update(plain); p.update(kw)
        assert "global_load_lds_dwordx4" not in R.emit_kernel("gemm_f32", "kernel0", **p)[0], kw
    rng = np.random.RandomState(m + n + k)
    a = rng.randint(-3, 4, size=batch + (m, k)).astype(np.float32)
    b = rng.randint(-3, 4, size=batch + (k, n)).astype(np.float32)
    print("matmul f32 direct loads", batch, m, n, k, cfg, flush=True)
    truth = np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)
    if cfg.get("RELU"):
        truth = np.maximum(truth, 0.0)
    c = host(ops.batched_matmul(dev(a), dev(b), **cfg))
    assert np.array_equal(c, truth)
    a = O.uniform(batch + (m, k), stream=127)
    b = O.uniform(batch + (k, n), stream=128)
    c = host(ops.batched_matmul(dev(a), dev(b), **cfg))
    truth = np.matmul(a.astype(np.float64), b.astype(np.float64))
    if cfg.get("RELU"):
        truth = np.maximum(truth, 0.0)
    assert O.rel_frobenius(c, truth) <= FP32_TOL
    other = host(ops.batched_matmul(dev(a), dev(b), **dict(plain, D2L=0)))
    assert O.rel_frobenius(c, other) <= FP32_TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("batch,m,n,k", [((3,), 128, 128, 64), ((2, 3), 100, 77, 33)])
def test_batched_matmul_f32_layouts(ops, ta, tb, batch, m, n, k):
    a = O.uniform(batch + ((k, m) if ta else (m, k)), stream=124)
    b = O.uniform(batch + ((n, k) if tb else (k, n)), stream=125)
    print("bmm f32", batch, m, n, k, ta, tb, flush=True)
    c = host(ops.batched_matmul(dev(a), dev(b), trans_a=ta, trans_b=tb))
    truth = O.batched_matmul_f64(a, b, ta, tb)
    assert c.shape == batch + (m, n)
    assert O.rel_frobenius(c, truth) <= FP32_TOL


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES + [(512, 512, 256)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_matmul_bf16_matches_oracle(ops, m, n, k, ta, tb):
    a = O.round_bf16(O.normal((k, m) if ta else (m, k), stream=131))
    b = O.round_bf16(O.normal((n, k) if tb else (k, n), stream=132, std=0.02))
    print("matmul bf16", m, n, k, ta, tb, flush=True)
    ad, bd = dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16)
    c = host(ops.batched_matmul(ad, bd, trans_a=ta, trans_b=tb))
    truth = O.batched_matmul_f64(a, b, ta, tb)
    assert c.shape == (m, n)
    assert O.rel_frobenius(c, truth) <= 1e-5      # fp32 accumulate of exact bf16 products
    cb = host(ops.batched_matmul(ad, bd, trans_a=ta, trans_b=tb, out_dtype=torch.bfloat16).float())
    assert O.rel_frobenius(cb, truth) <= LOWP_TOL


def test_matmul_bf16_exact_small_integers(ops):
    rng = np.random.RandomState(7)
    a = rng.randint(-4, 5, size=(256, 192)).astype(np.float32)
    b = rng.randint(-4, 5, size=(192, 320)).astype(np.float32)
    c = host(ops.matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16)))
    assert np.array_equal(c, O.matmul(a, b))


@pytest.mark.parametrize("m,n,k,cfg", [(1024, 1024, 1024, {}), (512, 768, 2048, dict(BM=256, BN=256)),
                                       (768, 512, 1536, dict(BM=128, BN=128)), (1024, 1024, 1024, dict(KROT=0))])
def test_matmul_bf16_k_walk_staggered_between_xcds(ops, m, n, k, cfg):
    """Two k-contiguous operands ([N][K] weights): the workgroups of XCD x start their walk along k at x/8 of K and
    wrap around.  Small integers make every partial sum exact, so the result must not depend on where a workgroup
    starts; N(0,1) operands check the same against fp64 within the fp32 bound."""
    from kernelcodegen_amd import runtime as R
    text, _ = R.emit_kernel("gemm_bf16", "kernel0", M=m, N=n, K=k, TB=1, **cfg)
    assert ("rot_k" in text.split("#if GB_KROT")[1]) and ("#define GB_KROT_ON 0" in text) == (cfg.get("KROT", 1) == 0)
    rng = np.random.RandomState(17)
    a = rng.randint(-4, 5, size=(m, k)).astype(np.float32)
    bt = rng.randint(-4, 5, size=(n, k)).astype(np.float32)
    print("matmul bf16 staggered k", m, n, k, cfg, flush=True)
    c = host(ops.batched_matmul(dev(a).to(torch.bfloat16), dev(bt).to(torch.bfloat16), trans_b=True, **cfg))
    assert np.array_equal(c, O.matmul(a, np.ascontiguousarray(bt.T)))
    a = O.round_bf16(O.normal((m, k), stream=133))
    bt = O.round_bf16(O.normal((n, k), stream=134, std=0.02))
    c = host(ops.batched_matmul(dev(a).to(torch.bfloat16), dev(bt).to(torch.bfloat16), trans_b=True, **cfg))
    assert O.rel_frobenius(c, O.batched_matmul_f64(a, bt, False, True)) <= 1e-5


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("m,n,k,cfg", [(512, 768, 512, dict(BM=256, BN=256)), (512, 512, 1024, dict(BM=256, BN=256, D2L=0)),
                                       (512, 768, 192, dict(BM=256, BN=256, STAGE_C=1)), (256, 512, 320, dict(BM=256, BN=256, D2L=0, STAGE_C=2)),
                                       (512, 512, 128, dict(BM=256, BN=256, STAGE_C=0)),
                                       (512, 768, 64, dict(BM=256, BN=256)), (256, 512, 128, dict(BM=256, BN=256)),
                                       (256, 512, 256, dict(BM=128, BN=128, WM=2, WN=2)), (512, 256, 320, dict(BM=256, BN=128, WM=4, WN=2, M16_DEAL=0, D2L=0)),
                                       (512, 256, 320, dict(BM=256, BN=128, WM=4, WN=2)), (256, 256, 128, dict(BM=128, BN=256, WM=2, WN=4, D2L=0))])
def test_matmul_bf16_on_16x16x32_mfma(ops, m, n, k, cfg, tb):
    """The GEMM family on v_mfma_f32_16x16x32 (M16): swizzled 128-byte LDS rows, rotating B fragments; operand tiles
    either straight from global memory into LDS (D2L, the default where every wavefront moves whole 1 KiB blocks) or
    through registers, where row-major weights get the regrouped k order that lets two lane groups' transposing reads
    take eight consecutive rows.  One, two, five and more k-tiles per product.  Small integers make every partial sum
    exact in any order; N(0,1) operands check against fp64 within the fp32 bound; the half-precision variant and the
    fused Relu go through the same code; so do the results that leave through LDS as whole rows of the tile (STAGE_C:
    the default for 16-bit results of 256 x 256 tiles, on request for fp32 results, off on request)."""
    from kernelcodegen_amd import runtime as R
    text, _ = R.emit_kernel("gemm_bf16", "kernel0", M=m, N=n, K=k, TB=int(tb), M16=1, **cfg)
    assert "#define GB_M16 1" in text
    assert [v for v in (1, 2) if "#define GB_STAGE_C %d" % v in text] == ([cfg["STAGE_C"]] if cfg.get("STAGE_C") else [])
    text16, _ = R.emit_kernel("gemm_bf16", "kernel0", M=m, N=n, K=k, TB=int(tb), M16=1, OUT_BF16=1, **cfg)
    expect = cfg.get("STAGE_C", 2) if cfg.get("BM") == 256 and cfg.get("BN") == 256 else 0
    assert [v for v in (1, 2) if "#define GB_STAGE_C %d" % v in text16] == ([expect] if expect else []), cfg
    direct = cfg.get("D2L", 1) and (tb or (cfg.get("BN") == 256 and cfg.get("WM", 4) * cfg.get("WN", 2) == 8))
    assert ("#define GB_D2L 1" in text) == bool(direct), (cfg, tb)
    rng = np.random.RandomState(m + n + k)
    a = rng.randint(-4, 5, size=(m, k)).astype(np.float32)
    b = rng.randint(-4, 5, size=(n, k) if tb else (k, n)).astype(np.float32)
    print("matmul bf16 16x16x32", m, n, k, cfg, tb, flush=True)
    truth = O.matmul(a, np.ascontiguousarray(b.T) if tb else b)
    for dt in (torch.bfloat16, torch.float16):
        c = host(ops.batched_matmul(dev(a).to(dt), dev(b).to(dt), trans_b=tb, M16=1, **cfg))
        assert np.array_equal(c, truth), dt
    c = host(ops.batched_matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16), trans_b=tb, M16=1, RELU=1, out_dtype=torch.bfloat16, **cfg).float())
    assert np.array_equal(c, O.round_bf16(np.maximum(truth, 0.0)))
    a = O.round_bf16(O.normal((2, m, k), stream=135))
    b = O.round_bf16(O.normal((2, n, k) if tb else (2, k, n), stream=136, std=0.02))
    c = host(ops.batched_matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16), trans_b=tb, M16=1, **cfg))
    assert O.rel_frobenius(c, O.batched_matmul_f64(a, b, False, tb)) <= 1e-5


def test_matmul_bf16_large_tiles_default_to_16x16x32_with_direct_loads(ops):
    from kernelcodegen_amd import runtime as R
    for tb in (0, 1):
        text, _ = R.emit_kernel("gemm_bf16", "kernel0", M=4096, N=11008, K=4096, TB=tb)
        assert "#define GB_M16 1" in text and "#define GB_D2L 1" in text
    for kw in (dict(TA=1), dict(M=4000), dict(K=4100), dict(BM=128, BN=128), dict(M16=0), dict(D2L=0, TB=1)):
        p = dict(M=4096, N=11008, K=4096); p.update(kw)
        assert "#define GB_M16 1" not in R.emit_kernel("gemm_bf16", "kernel0", **p)[0], kw
    text, _ = R.emit_kernel("gemm_bf16", "kernel0", M=4096, N=11008, K=4096, M16=1, D2L=0)
    assert "#define GB_M16 1" in text and "#define GB_D2L 1" not in text and "#define GB_BPAD 32" in text


# ---------------------------------------------------------------------------
FMHA_SHAPES = [
    (1, 1, 128, 128, 128, 64),    # one query tile, two key tiles
    (2, 3, 256, 64, 128, 64),     # head dim 64
    (1, 2, 96, 32, 32, 32),       # smallest tiles, one wavefront
    (2, 2, 512, 128, 128, 64),    # several query tiles: causal tile skipping
    (1, 1, 256, 96, 64, 32),      # head dim 96: three 32-wide output tiles
]


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,s,d,br,bc", FMHA_SHAPES)
def test_fmha_bf16_matches_oracle(ops, b, h, s, d, br, bc, causal):
    shp = (b, h, s, d)
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (141, 142, 143))
    scale = d ** -0.5
    print("fmha bf16", shp, br, bc, causal, flush=True)
    qd, kd, vd = (dev(t).to(torch.bfloat16) for t in (q, k, v))
    truth = O.fmha_f64(q, k, v, scale=scale, causal=causal)
    o32 = host(ops.fmha(qd, kd, vd, scale=scale, causal=causal, out_dtype=torch.float32, BR=br, BC=bc))
    assert o32.shape == shp and np.isfinite(o32).all()
    # probabilities are rounded to bf16 before the second product: 2^-9 relative per term
    assert O.rel_frobenius(o32, truth) <= LOWP_TOL
    assert O.rel_frobenius(o32, truth) <= 4e-3
    ob = host(ops.fmha(qd, kd, vd, scale=scale, causal=causal, BR=br, BC=bc).float())
    assert O.rel_frobenius(ob, truth) <= LOWP_TOL


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,s,cfg", [(1, 2, 512, dict(PERSIST=0)), (2, 3, 256, dict(PERSIST=0)), (3, 96, 1024, {}), (2, 130, 512, dict(PAIR=1))])
def test_fmha_bf16_tiles_loaded_straight_into_lds(ops, b, h, s, cfg, causal):
    """D2L: the K and V tiles go from global memory into swizzled, unpadded LDS rows without passing through registers.
    The arithmetic and its order are those of the register form, so the results must agree with it bit for bit (and
    with the oracle within the kernel's bound): one job per workgroup and persistent workgroups with the job stream
    (more than 256 items), with and without the mask, both pairings of query tiles, bf16 and IEEE half."""
    d = 128
    shp = (b, h, s, d)
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (144, 145, 146))
    print("fmha bf16 direct loads", shp, cfg, causal, flush=True)
    for dt in (torch.bfloat16, torch.float16):
        qd, kd, vd = (dev(t).to(dt) for t in (q, k, v))
        plain = ops.fmha(qd, kd, vd, causal=causal, **cfg)
        direct = ops.fmha(qd, kd, vd, causal=causal, D2L=1, **cfg)
        assert torch.equal(plain.view(torch.int16), direct.view(torch.int16)), dt
    sample = (slice(0, b, max(1, b - 1)), slice(0, h, max(1, h // 3)))
    truth = O.fmha_f64(q[sample], k[sample], v[sample], scale=d ** -0.5, causal=causal)
    assert O.rel_frobenius(host(direct.float())[sample], truth) <= 4e-3
    from kernelcodegen_amd._lib import KcgError
    with pytest.raises(KcgError):
        ops.fmha(qd[:, :, :200].contiguous(), kd[:, :, :200].contiguous(), vd[:, :, :200].contiguous(), D2L=1)


@pytest.mark.parametrize("m,n,k,ta,tb,cfg", [(256, 256, 128, 0, 0, {}), (512, 384, 200, 0, 1, {}), (100, 77, 33, 0, 0, {}),
                                             (130, 64, 48, 1, 0, {}), (96, 160, 72, 1, 1, {}), (256, 256, 64, 0, 0, {"BM": 128, "BN": 128}),
                                             (192, 320, 36, 0, 0, {"BK": 8}), (300, 260, 50, 0, 1, {"BM": 128, "BN": 128, "WM": 2, "WN": 4})])
def test_matmul_f64_matches_numpy(ops, m, n, k, ta, tb, cfg):
    """The fp64 family (v_mfma_f64_16x16x4_f64) against numpy's fp64 product: every layout, ragged extents, both tile
    sizes.  fp64 products summed in another order: 1e-13 relative."""
    rs = np.random.RandomState(m * 7 + n * 3 + k)
    a = rs.standard_normal((k, m) if ta else (m, k))
    b = rs.standard_normal((n, k) if tb else (k, n))
    print("gemm f64", m, n, k, ta, tb, cfg, flush=True)
    c = ops.matmul(dev(a), dev(b), trans_a=bool(ta), trans_b=bool(tb), **cfg)
    assert c.dtype == torch.float64 and tuple(c.shape) == (m, n)
    want = (a.T if ta else a) @ (b.T if tb else b)
    assert O.rel_frobenius(host(c), want) <= 1e-13


@pytest.mark.parametrize("batch,m,n,k,cfg", [((), 128, 256, 16, {}), ((), 256, 512, 48, {}), ((2,), 128, 512, 208, dict(RELU=1)),
                                             ((), 384, 256, 1024, {}), ((), 256, 256, 80, dict(BM=128, BN=128)),
                                             ((), 128, 256, 64, dict(BM=64, BN=128, WM=2, WN=2)), ((), 128, 512, 32, dict(WM=2, WN=4))])
def test_matmul_f64_tiles_loaded_straight_into_lds(ops, batch, m, n, k, cfg):
    """The fp64 GEMM for whole tiles of two row-major operands (tiles straight from global memory into LDS, A's rows
    swizzled on the source side and read two k at a time, B's odd rows with their 128-byte halves exchanged): the
    128 x 256 tile with sixteen wavefronts and smaller ones, one to many k-tiles, batches, the fused Relu.  Small
    integers are exact in any order; N(0,1) operands against numpy's product at 1e-13, and against the other kernel."""
    from kernelcodegen_amd import runtime as R
    cfg = dict(dict(BM=128, BN=256), **cfg)
    nb = max(1, int(np.prod(batch)))
    text, info = R.emit_kernel("gemm_f64", "kernel0", M=m, N=n, K=k, BATCH=nb, **cfg)
    assert "global_load_lds_dwordx4" in text
    assert "global_load_lds_dwordx4" not in R.emit_kernel("gemm_f64", "kernel0", M=m, N=n, K=k, **dict(cfg, D2L=0))[0]
    for kw in (dict(M=m + 8), dict(K=k + 4), dict(TA=1), dict(TB=1), dict(BK=8)):
        p = dict(M=m, N=n, K=k); p.update(cfg); p.update(kw)
        assert "global_load_lds_dwordx4" not in R.emit_kernel("gemm_f64", "kernel0", **p)[0], kw
    rs = np.random.RandomState(m + n + k)
    a = rs.randint(-9, 10, size=batch + (m, k)).astype(np.float64)
    b = rs.randint(-9, 10, size=batch + (k, n)).astype(np.float64)
    print("gemm f64 direct loads", batch, m, n, k, cfg, flush=True)
    relu = (lambda x: np.maximum(x, 0.0)) if cfg.get("RELU") else (lambda x: x)
    assert np.array_equal(host(ops.batched_matmul(dev(a), dev(b), **cfg)), relu(a @ b))
    a, b = rs.standard_normal(batch + (m, k)), rs.standard_normal(batch + (k, n))
    c = host(ops.batched_matmul(dev(a), dev(b), **cfg))
    assert O.rel_frobenius(c, relu(a @ b)) <= 1e-13
    assert O.rel_frobenius(c, host(ops.batched_matmul(dev(a), dev(b), **dict(cfg, D2L=0)))) <= 1e-13


def test_batched_matmul_f64_and_exact_integers(ops):
    rs = np.random.RandomState(5)
    a, b = rs.randint(-9, 10, size=(3, 2, 144, 80)).astype(np.float64), rs.randint(-9, 10, size=(3, 2, 80, 96)).astype(np.float64)
    c = ops.batched_matmul(dev(a), dev(b))
    assert c.dtype == torch.float64 and np.array_equal(host(c), a @ b)          # small integers: every sum is exact


@pytest.mark.parametrize("b,h,s,d,causal", [(2, 2, 512, 128, False), (2, 2, 512, 128, True), (1, 3, 256, 64, True),
                                            (8, 8, 2048, 128, False), (8, 8, 2048, 128, True)])
def test_fmha_f16_matches_oracle(ops, b, h, s, d, causal):
    """IEEE half operands through the same kernel (FA_F16: the f16 MFMA, probabilities packed to half; the last two
    shapes run the persistent workgroups).  Half has three more mantissa bits than bf16, so the result is closer to the
    fp64 truth than the bf16 kernel's: 1e-3 on the fp32 result where bf16 needs 4e-3; the bar is 1e-2."""
    shp = (b, h, s, d)
    q, k, v = (O.normal(shp, stream=st).astype(np.float16).astype(np.float32) for st in (151, 152, 153))
    scale = d ** -0.5
    print("fmha f16", shp, causal, flush=True)
    qd, kd, vd = (dev(t).to(torch.float16) for t in (q, k, v))
    rows = slice(None) if s <= 512 else slice(0, s, 61)                 # sampled query rows at the long sequence
    if s <= 512:
        truth = O.fmha_f64(q, k, v, scale=scale, causal=causal)
    else:
        truth = np.stack([np.stack([np.concatenate([O.fmha_rows_f64(q[bi, hi], k[bi, hi], v[bi, hi], r, 1, scale=scale, causal=causal)
                                                    for r in range(0, s, 61)]) for hi in range(0, h, 3)]) for bi in range(0, b, 3)])
    o32 = host(ops.fmha(qd, kd, vd, scale=scale, causal=causal, out_dtype=torch.float32))
    got = o32 if s <= 512 else o32[::3, ::3][:, :, rows]
    assert np.isfinite(o32).all()
    assert O.rel_frobenius(got, truth) <= 1e-3
    oh = ops.fmha(qd, kd, vd, scale=scale, causal=causal)
    assert oh.dtype == torch.float16
    got16 = host(oh.float())
    got16 = got16 if s <= 512 else got16[::3, ::3][:, :, rows]
    assert O.rel_frobenius(got16, truth) <= LOWP_TOL
    with pytest.raises(ValueError):
        ops.fmha(qd, kd.to(torch.bfloat16), vd)


RAGGED_FMHA = [
    (2, 3, 1000, 128, {}, torch.bfloat16),                 # 256-query and 64-key tiles, the last of each partly filled
    (1, 2, 700, 128, {}, torch.bfloat16),                  # an odd number of query tiles: no pairs under the mask
    (1, 2, 900, 128, {}, torch.bfloat16),                  # 15 key tiles: under the mask a sixteenth, fully masked one is run
    (1, 2, 4000, 128, {}, torch.bfloat16),                 # 32 divides it: 256-query tiles with a guarded edge all the same
    (1, 2, 77, 64, {}, torch.bfloat16),                    # one query tile of 128, two key tiles
    (2, 2, 197, 64, {}, torch.float16),                    # IEEE half
    (1, 1, 33, 32, {}, torch.bfloat16),                    # one row into the second tile
    (1, 1, 7, 32, {}, torch.bfloat16),                     # shorter than any tile
    (1, 2, 300, 256, {}, torch.bfloat16),                  # head dim 256 (32-key tiles)
    (1, 2, 130, 96, {}, torch.bfloat16),                   # head dim 96
    (2, 1, 200, 64, {"BR": 64, "BC": 32}, torch.bfloat16),   # four query tiles, the last with 8 rows; keys divide
    (1, 2, 224, 64, {"BR": 64, "BC": 64}, torch.bfloat16),   # queries ragged (3.5 tiles), keys ragged
]


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,s,d,cfg,dtype", RAGGED_FMHA)
def test_fmha_sequence_length_no_multiple_of_the_tiles(ops, b, h, s, d, cfg, dtype, causal):
    """A sequence length that the query or key tiles do not divide: the kernel's last tiles read no row past the end
    (they repeat the last one), mask the keys past the end and write no result row past the end.  Against the fp64
    attention on the same rounded operands; the result buffer is followed by a guard area that must stay untouched."""
    from kernelcodegen_amd import runtime as R
    shp = (b, h, s, d)
    rnd = O.round_bf16 if dtype == torch.bfloat16 else (lambda t: t.astype(np.float16).astype(np.float32))
    q, k, v = (rnd(O.normal(shp, stream=st)) for st in (161, 162, 163))
    scale = d ** -0.5
    print("fmha ragged", shp, cfg, dtype, causal, flush=True)
    qd, kd, vd = (dev(t).to(dtype) for t in (q, k, v))
    truth = O.fmha_f64(q, k, v, scale=scale, causal=causal)
    o32 = host(ops.fmha(qd, kd, vd, scale=scale, causal=causal, out_dtype=torch.float32, **cfg))
    assert o32.shape == shp and np.isfinite(o32).all()
    assert O.rel_frobenius(o32, truth) <= (4e-3 if dtype == torch.bfloat16 else 1e-3)
    # the 16-bit result inside a larger buffer whose tail holds a pattern
    n = b * h * s * d
    guard = 512 * d
    buf = torch.full((n + guard,), 7.0, dtype=dtype, device="cuda")
    kern = R.get_kernel("fmha_bf16", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale, OUT_BF16=1,
                        F16=int(dtype == torch.float16), **cfg)
    kern.launch(qd, kd, vd, buf)
    torch.cuda.synchronize()
    assert bool((buf[n:] == 7.0).all()), "the kernel wrote past the end of its result"
    assert O.rel_frobenius(host(buf[:n].float()).reshape(shp), truth) <= LOWP_TOL


FMHA_F32 = [
    # b, h, s, d, causal, scale (None: 1 / sqrt(d)), config
    (2, 2, 256, 64, False, 1.0, {}),                  # the reference graph's semantics: no scale, no mask
    (1, 3, 320, 128, True, None, {}),
    (2, 1, 128, 32, True, None, {"BR": 64}),
    (1, 2, 256, 256, False, None, {}),                # the widest head: one workgroup per CU
    (1, 2, 77, 64, True, None, {}),                   # no tile divides the sequence length
    (2, 2, 200, 96, False, 0.2, {"BC": 32}),
    (1, 1, 33, 32, True, None, {"BR": 32}),
    (3, 5, 1000, 64, True, None, {"BR": 256}),        # a head count no multiple of eight: plain workgroup numbering
    # K and V tiles straight from global memory into two LDS buffers each (the default for whole tiles of head dim 128)
    (2, 8, 512, 128, True, None, {}),
    (1, 8, 384, 128, False, None, {"D2L": 0}),
    (2, 3, 256, 64, True, None, {"D2L": 1}),
    (1, 2, 512, 64, False, None, {"D2L": 1, "BC": 64}),
    (1, 2, 512, 128, True, None, {"D2L": 1, "BC": 64, "BR": 256}),
    # under the mask a workgroup takes two query tiles, the longest with the shortest (the default on grids that fill the part)
    (2, 8, 512, 128, True, None, {"PAIR": 1}),
    (2, 3, 256, 64, True, None, {"PAIR": 1}),          # one pair per head, plain workgroup numbering
    (1, 2, 512, 64, True, None, {"PAIR": 1, "D2L": 1, "BC": 64}),
    (1, 8, 1024, 96, True, None, {"PAIR": 1, "BR": 64}),
    (3, 5, 1000, 64, True, None, {"PAIR": 1, "BR": 256}),      # the last of four query tiles partly filled
    (1, 2, 77, 64, True, None, {"PAIR": 1, "BR": 64}),         # two tiles, the second with 13 queries
]


@pytest.mark.parametrize("b,h,s,d,causal,scale,cfg", FMHA_F32)
def test_fmha_f32_matches_oracle(ops, b, h, s, d, causal, scale, cfg):
    """fp32 attention with both products on the fp32 MFMA (fmha_f32): the fp32 bar, 1e-5 relative Frobenius against
    fp64 attention on the same operands (the unfused nests of the reference graph, test/test.cc:107-147, compute the
    same function); sequence lengths that no tile divides leave the guard area behind the result untouched."""
    from kernelcodegen_amd import runtime as R
    shp = (b, h, s, d)
    scale = d ** -0.5 if scale is None else scale
    std = 1.0 if scale < 1.0 else d ** -0.25          # unscaled scores of N(0, 1) operands would saturate the softmax
    q, k, v = (O.normal(shp, stream=st, std=std) for st in (341, 342, 343))
    print("fmha f32", shp, causal, scale, cfg, flush=True)
    n = b * h * s * d
    buf = torch.full((n + 512 * d,), 7.0, device="cuda")
    kern = R.get_kernel("fmha_f32", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale, **cfg)
    direct = "#define FF_D2L 1" in R.emit_kernel("fmha_f32", "kernel0", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale, **cfg)[0]
    whole = s % cfg.get("BR", 128) == 0 and s % cfg.get("BC", 32) == 0 and d in (64, 128)
    assert direct == bool(whole and cfg.get("D2L", d == 128)), cfg
    kern.launch(dev(q), dev(k), dev(v), buf)
    torch.cuda.synchronize()
    assert bool((buf[n:] == 7.0).all()), "the kernel wrote past the end of its result"
    got = host(buf[:n]).reshape(shp)
    truth = O.fmha_f64(q, k, v, scale=scale, causal=causal)
    assert np.isfinite(got).all() and O.rel_frobenius(got, truth) <= 1e-5
    if not cfg:
        assert np.array_equal(host(ops.fmha(dev(q), dev(k), dev(v), scale=scale, causal=causal)), got)
    if direct:                                        # the same sums in the same order as with the tiles through registers
        plain = torch.empty(n, device="cuda")
        R.get_kernel("fmha_f32", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale, **dict(cfg, D2L=0)).launch(dev(q), dev(k), dev(v), plain)
        torch.cuda.synchronize()
        assert np.array_equal(host(plain).reshape(shp), got)
    if cfg.get("PAIR"):                               # a query tile's arithmetic does not depend on which workgroup runs it
        single = torch.empty(n, device="cuda")
        R.get_kernel("fmha_f32", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=scale, **dict(cfg, PAIR=0)).launch(dev(q), dev(k), dev(v), single)
        torch.cuda.synchronize()
        assert np.array_equal(host(single).reshape(shp), got)


def test_fmha_f32_invariants(ops):
    """A constant V comes back unchanged up to rounding (probabilities sum to one), the first causal row is V's first
    row exactly (one probability, 1.0), and the result does not depend on the tile sizes beyond rounding."""
    shp = (1, 2, 256, 64)
    q, k, v = (O.normal(shp, stream=st) for st in (351, 352, 353))
    vconst = np.broadcast_to(O.normal((1, 2, 1, 64), stream=354), shp).copy()
    o = host(ops.fmha(dev(q), dev(k), dev(vconst), causal=True))
    assert np.abs(o - vconst).max() <= 1e-6 * np.abs(vconst).max() + 1e-6
    o = host(ops.fmha(dev(q), dev(k), dev(v), causal=True))
    assert np.array_equal(o[:, :, 0, :], v[:, :, 0, :])
    o2 = host(ops.fmha(dev(q), dev(k), dev(v), causal=True, BR=64, BC=32))
    assert O.rel_frobenius(o2, o) <= 2e-6
    with pytest.raises(ValueError):
        ops.fmha(dev(q), dev(k), dev(v).to(torch.bfloat16))


def test_fmha_bf16_default_tiles_and_unit_scale(ops):
    shp = (2, 2, 384, 128)
    q, k, v = (O.round_bf16(O.normal(shp, stream=st, std=0.3)) for st in (144, 145, 146))
    qd, kd, vd = (dev(t).to(torch.bfloat16) for t in (q, k, v))
    o = host(ops.fmha(qd, kd, vd, scale=1.0, causal=False, out_dtype=torch.float32))
    assert O.rel_frobenius(o, O.fmha_f64(q, k, v, scale=1.0, causal=False)) <= 4e-3


@pytest.mark.parametrize("causal", [False, True])
def test_fmha_bf16_head_dim_256_default_tiles(ops, causal):
    """The largest head dimension: 64-key tiles do not fit the LDS, the default falls back to 32-key tiles."""
    shp = (1, 2, 256, 256)
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (147, 148, 149))
    print("fmha bf16 head dim 256", shp, causal, flush=True)
    qd, kd, vd = (dev(t).to(torch.bfloat16) for t in (q, k, v))
    o = host(ops.fmha(qd, kd, vd, scale=256 ** -0.5, causal=causal, out_dtype=torch.float32))
    assert O.rel_frobenius(o, O.fmha_f64(q, k, v, scale=256 ** -0.5, causal=causal)) <= 4e-3


def test_fmha_bf16_invariants(ops):
    """Properties that hold whatever the tile sizes: a constant V is returned
    unchanged (softmax rows sum to one); the first causal row is V's first row;
    equal keys give the plain mean of V."""
    b, h, s, d = 1, 2, 256, 128
    q = O.round_bf16(O.normal((b, h, s, d), stream=147))
    k = O.round_bf16(O.normal((b, h, s, d), stream=148))
    v = O.round_bf16(O.normal((b, h, s, d), stream=149))
    qd, kd, vd = (dev(t).to(torch.bfloat16) for t in (q, k, v))
    vconst = np.broadcast_to(O.round_bf16(O.normal((b, h, 1, d), stream=150)), (b, h, s, d)).copy()
    o = host(ops.fmha(qd, kd, dev(vconst).to(torch.bfloat16), causal=True, out_dtype=torch.float32))
    assert np.abs(o - vconst).max() <= 2e-2 * np.abs(vconst).max()
    o = host(ops.fmha(qd, kd, vd, causal=True, out_dtype=torch.float32))
    assert np.array_equal(o[:, :, 0, :], v[:, :, 0, :])
    kconst = np.broadcast_to(k[:, :, :1, :], (b, h, s, d)).copy()
    o = host(ops.fmha(qd, dev(kconst).to(torch.bfloat16), vd, causal=False, out_dtype=torch.float32))
    mean = v.astype(np.float64).mean(axis=2, keepdims=True)
    assert np.abs(o - mean).max() <= 1e-2


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("d", [64, 128])
def test_fmha_bf16_two_query_blocks_per_wavefront(ops, d, causal):
    """QW=2: a wavefront owns 64 queries and every LDS fragment feeds two MFMAs."""
    shp = (1, 2, 512, d)
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (161, 162, 163))
    qd, kd, vd = (dev(t).to(torch.bfloat16) for t in (q, k, v))
    print("fmha bf16 QW=2", shp, causal, flush=True)
    truth = O.fmha_f64(q, k, v, scale=d ** -0.5, causal=causal)
    o = host(ops.fmha(qd, kd, vd, scale=d ** -0.5, causal=causal, out_dtype=torch.float32, BR=256, BC=64, QW=2))
    assert O.rel_frobenius(o, truth) <= 4e-3


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("trend", ["rising", "falling", "far_below_zero"])
def test_fmha_bf16_moving_reference_point(ops, trend, causal):
    """Scores that keep growing along the keys move the softmax reference point in every tile, also inside
    the steady-state loop; falling scores never move it after the first tile; scores far below zero must
    not underflow the first tile's probabilities (the reference point starts at the first tile's maximum)."""
    b, h, s, d = 1, 2, 512, 128
    base = O.round_bf16(O.normal((b, h, 1, d), stream=171))
    base /= np.sqrt((base.astype(np.float64) ** 2).sum(-1, keepdims=True)).astype(np.float32)
    ramp = np.linspace(0.0, 1.0, s, dtype=np.float32).reshape(1, 1, s, 1)
    noise = 0.05 * O.normal((b, h, s, d), stream=172)
    if trend == "rising":
        k = 60.0 * ramp * base + noise
    elif trend == "falling":
        k = 60.0 * (1.0 - ramp) * base + noise
    else:
        k = -(200.0 + 20.0 * ramp) * base + noise
    q = np.broadcast_to(4.0 * base, (b, h, s, d)) + 0.05 * O.normal((b, h, s, d), stream=173)
    q, k = O.round_bf16(q.astype(np.float32)), O.round_bf16(k.astype(np.float32))
    v = O.round_bf16(O.normal((b, h, s, d), stream=174))
    qd, kd, vd = (dev(t).to(torch.bfloat16) for t in (q, k, v))
    print("fmha bf16 reference point", trend, causal, flush=True)
    # scale = ln 2 makes scale * log2(e) = 1: the kernel's pre-scaled queries are then exact, and exponents of
    # several hundred test the reference point alone rather than one more bf16 rounding of the queries
    scale = float(np.log(2.0))
    truth = O.fmha_f64(q, k, v, scale=scale, causal=causal)
    o = host(ops.fmha(qd, kd, vd, scale=scale, causal=causal, out_dtype=torch.float32, BR=128, BC=64))
    assert np.isfinite(o).all()
    assert O.rel_frobenius(o, truth) <= LOWP_TOL


@pytest.mark.parametrize("causal", [False, True])
def test_fmha_bf16_full_size_sampled_rows(ops, causal):
    """B8 H32 S2048 D128: generated on the device, rows sampled against the fp64 oracle."""
    b, h, s, d = 8, 32, 2048, 128
    g = torch.Generator(device="cuda")
    g.manual_seed(1234)
    q, k, v = (torch.randn((b, h, s, d), device="cuda", generator=g).bfloat16() for _ in range(3))
    scale = d ** -0.5
    print("fmha full size causal=%s" % causal, flush=True)
    o = ops.fmha(q, k, v, scale=scale, causal=causal, out_dtype=torch.float32)
    for (bi, hi, row0) in [(0, 0, 0), (3, 17, 1000), (7, 31, 2040)]:
        qs, ks, vs = (host(t[bi, hi].float()) for t in (q, k, v))
        truth = O.fmha_rows_f64(qs, ks, vs, row0, 8, scale=scale, causal=causal)
        assert O.rel_frobenius(host(o[bi, hi, row0:row0 + 8]), truth) <= 4e-3


# ---------------------------------------------------------------------------
def _fp8_operands(m, n, k, batch=()):
    """Oracle-quantised e4m3 operands: bits for the device, decoded values for the truth."""
    a = O.normal(batch + (m, k), stream=151)
    bt = O.normal(batch + (n, k), stream=152, std=0.02)
    sa, sb = float(np.abs(a).max()) / 448.0, float(np.abs(bt).max()) / 448.0
    abits, bbits = O.to_fp8_bits(a, 1.0 / sa), O.to_fp8_bits(bt, 1.0 / sb)
    return abits, bbits, O.from_fp8_bits(abits), O.from_fp8_bits(bbits), sa, sb


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (128, 192, 512), (100, 77, 200), (512, 512, 1024), (64, 64, 64)])
def test_matmul_fp8_matches_oracle(ops, m, n, k):
    abits, bbits, adec, bdec, sa, sb = _fp8_operands(m, n, k)
    print("matmul fp8", m, n, k, flush=True)
    ad = dev(abits).view(torch.float8_e4m3fn)
    bd = dev(bbits).view(torch.float8_e4m3fn)
    c = host(ops.matmul_fp8(ad, bd, sa, sb))
    truth = O.batched_matmul_f64(adec, bdec, False, True) * (sa * sb)
    assert c.shape == (m, n)
    # same quantised operands on both sides: what remains is the accumulation of the 64-deep MFMA step
    assert O.rel_frobenius(c, truth) <= 1e-4
    # against the unquantised operands the error is the quantisation's
    cb = host(ops.matmul_fp8(ad, bd, sa, sb, out_dtype=torch.bfloat16).float())
    assert O.rel_frobenius(cb, truth) <= LOWP_TOL


def test_matmul_fp8_exact_small_integers_and_batch(ops):
    """Integers up to 8 are exact in e4m3 and their dot products are exact in fp32:
    the result must equal the oracle's integer arithmetic bit for bit (this pins the
    operand byte order inside the 64-deep MFMA step and the scale handling)."""
    rng = np.random.RandomState(11)
    a = rng.randint(-8, 9, size=(2, 128, 320)).astype(np.float32)
    bt = rng.randint(-8, 9, size=(2, 160, 320)).astype(np.float32)
    abits, bbits = O.to_fp8_bits(a), O.to_fp8_bits(bt)
    assert np.array_equal(O.from_fp8_bits(abits), a)
    c = host(ops.matmul_fp8(dev(abits).view(torch.float8_e4m3fn), dev(bbits).view(torch.float8_e4m3fn), 0.5, 4.0))
    truth = np.stack([O.matmul(a[i], bt[i].T.copy()) for i in range(2)]) * 2.0
    assert np.array_equal(c, truth)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (100, 77, 200), (512, 384, 128)])
def test_matmul_fp8_operand_layouts(ops, m, n, k, ta, tb):
    """Operands that are contiguous along m / n go through the byte-transposing loader."""
    a = O.normal((k, m) if ta else (m, k), stream=153)
    b = O.normal((n, k) if tb else (k, n), stream=154, std=0.02)
    sa, sb = float(np.abs(a).max()) / 448.0, float(np.abs(b).max()) / 448.0
    abits, bbits = O.to_fp8_bits(a, 1.0 / sa), O.to_fp8_bits(b, 1.0 / sb)
    print("matmul fp8 layouts", m, n, k, ta, tb, flush=True)
    c = host(ops.matmul_fp8(dev(abits).view(torch.float8_e4m3fn), dev(bbits).view(torch.float8_e4m3fn), sa, sb,
                            trans_a=ta, trans_b=tb))
    truth = O.batched_matmul_f64(O.from_fp8_bits(abits), O.from_fp8_bits(bbits), ta, tb) * (sa * sb)
    assert c.shape == (m, n)
    assert O.rel_frobenius(c, truth) <= 1e-4


@pytest.mark.parametrize("cfg", [{}, {"BTR": 0}, {"BM": 256, "BN": 256}, {"BM": 256, "BN": 256, "BTR": 0}, {"BM": 128, "BN": 128, "BK": 64},
                                 {"BM": 256, "BN": 256, "ROTATE": 0}, {"BM": 256, "BN": 256, "BTR": 0, "ROTATE": 1},
                                 {"BM": 128, "BN": 128, "BK": 256, "PREFETCH": 0, "ROTATE": 1}])
@pytest.mark.parametrize("m,n,k", [(128, 320, 160), (300, 272, 200), (256, 500, 130), (512, 512, 1024)])
def test_matmul_fp8_row_major_weights_exact(ops, m, n, k, cfg):
    """[K][N] weights in both forms: copied into LDS as they lie and transposed by the LDS reads (the default), or
    transposed in registers on the way in (BTR = 0); small integers, so every sum is exact and the two agree bit for
    bit with the plain nest.  Ragged extents, n not a multiple of 16 included (the guarded loader).  The 256 x 256
    tiles with the fragments re-read behind their last use (ROTATE, their default with these weights), without, with
    four k-steps per tile, and over several k-tiles (k = 1024)."""
    rng = np.random.RandomState(12 + m)
    a = rng.randint(-8, 9, size=(m, k)).astype(np.float32)
    b = rng.randint(-8, 9, size=(k, n)).astype(np.float32)
    print("matmul fp8 [K][N]", m, n, k, cfg, flush=True)
    c = host(ops.matmul_fp8(dev(O.to_fp8_bits(a)).view(torch.float8_e4m3fn), dev(O.to_fp8_bits(b)).view(torch.float8_e4m3fn),
                            1.0, 1.0, trans_b=False, **cfg))
    assert np.array_equal(c, O.matmul(a, b))


@pytest.mark.parametrize("m,n,k,cfg", [(256, 512, 128, {}), (512, 256, 256, {}), (256, 256, 384, dict(RELU=1)), (512, 768, 1024, {}),
                                       (512, 512, 640, dict(NT_STORE=1, STAGGER=2)), (512, 768, 384, dict(STAGE_C=0)), (256, 512, 256, dict(STAGE_C=0, RELU=1, NT_STORE=1)), (256, 256, 4096, {}), (256, 256, 8192, dict(D2L=1)),
                                       (4608, 4096, 256, dict(PERSIST=1)), (4352, 4096, 512, dict(PERSIST=1, STAGGER=0)),
                                       (6912, 6144, 256, dict(PERSIST=1, RELU=1))])
@pytest.mark.parametrize("tb", [True, False])
def test_matmul_fp8_on_16x16x128_mfma_with_direct_loads(ops, m, n, k, cfg, tb):
    """The fp8 kernel for full 256 x 256 x 128 tiles of two k-contiguous operands (v_mfma_f32_16x16x128, tiles straight
    from global memory into swizzled LDS rows, B fragments two columns ahead, one barrier per tile): one, two, three
    and many k-tiles, two batches, the fused Relu, the bf16 result, the non-temporal stores and the staggered start,
    fp32 results through LDS as whole rows (the default) and straight out of the accumulators (STAGE_C=0);
    persistent workgroups that take two output tiles each, two and one, or three and two (288, 272 and 648 tiles on
    256 workgroups).
    Integers up to 8 are exact in e4m3 and their dot products in fp32, so the result equals the integer arithmetic bit
    for bit whatever the order of the sums; N(0,1) operands check the scale handling against fp64."""
    from kernelcodegen_amd import runtime as R
    text, _ = R.emit_kernel("gemm_fp8", "kernel0", M=m, N=n, K=k, TB=int(tb), BM=256, BN=256, **cfg)
    assert "mfma_scale_f32_16x16x128_f8f6f4" in text and "global_load_lds_dwordx4" in text and ("#define G8_BTR 1" in text) == (not tb)
    rng = np.random.RandomState(m + n + k)
    nb = 1 if cfg.get("PERSIST") else 2
    a = rng.randint(-8, 9, size=(nb, m, k)).astype(np.float32)
    bt = rng.randint(-8, 9, size=(nb, n, k)).astype(np.float32)
    if cfg.get("PERSIST"):
        assert "#define G8_PERSIST 1" in R.emit_kernel("gemm_fp8", "kernel0", M=m, N=n, K=k, TB=int(tb), BM=256, BN=256, **cfg)[0]
    print("matmul fp8 16x16x128", m, n, k, cfg, tb, flush=True)
    as_b = (lambda x: x) if tb else (lambda x: np.ascontiguousarray(np.swapaxes(x, -1, -2)))     # [N][K], or row-major [K][N]
    ad, bd = dev(O.to_fp8_bits(a)).view(torch.float8_e4m3fn), dev(O.to_fp8_bits(as_b(bt))).view(torch.float8_e4m3fn)
    truth = np.stack([O.matmul(a[i], bt[i].T.copy()) for i in range(nb)]) * 0.5
    if cfg.get("RELU"):
        truth = np.maximum(truth, 0.0)
    c = host(ops.matmul_fp8(ad, bd, 0.25, 2.0, trans_b=tb, BM=256, BN=256, **cfg))
    assert np.array_equal(c, truth)
    cb = host(ops.matmul_fp8(ad, bd, 0.25, 2.0, trans_b=tb, out_dtype=torch.bfloat16, BM=256, BN=256, **dict(cfg, D2L=1)).float())
    assert np.array_equal(cb, O.round_bf16(truth))
    abits, bbits, adec, bdec, sa, sb = _fp8_operands(m, n, k)
    c = host(ops.matmul_fp8(dev(abits).view(torch.float8_e4m3fn), dev(as_b(bbits)).view(torch.float8_e4m3fn), sa, sb, trans_b=tb, BM=256, BN=256, **cfg))
    truth = O.batched_matmul_f64(adec, bdec, False, True) * (sa * sb)
    assert O.rel_frobenius(c, np.maximum(truth, 0.0) if cfg.get("RELU") else truth) <= 1e-4


def test_matmul_fp8_kernel_choice(ops):
    from kernelcodegen_amd import runtime as R
    d2l = lambda **kw: "global_load_lds_dwordx4" in R.emit_kernel("gemm_fp8", "kernel0", **kw)[0]
    assert d2l(M=4096, N=11008, K=4096, TB=1)
    text = R.emit_kernel("gemm_fp8", "kernel0", M=4096, N=11008, K=4096, TB=1)[0]
    assert "#define G8_NT_STORE 1" in text and "#define G8_STAGGER 1" in text and "#define G8_STAGE_C 1" in text   # more than one round of tiles
    text = R.emit_kernel("gemm_fp8", "kernel0", M=4096, N=11008, K=4096, TB=1, STAGE_C=0)[0]
    assert "#define G8_NT_STORE 1" in text and "#define G8_STAGGER 2" in text and "#define G8_STAGE_C 0" in text
    text = R.emit_kernel("gemm_fp8", "kernel0", M=4096, N=4096, K=4096, TB=1)[0]
    assert "#define G8_NT_STORE 0" in text and "#define G8_STAGGER 0" in text          # a single round
    text = R.emit_kernel("gemm_fp8", "kernel0", M=4096, N=11008, K=4096, TB=1, OUT_BF16=1)[0]       # a bf16 result: the same
    assert "global_load_lds_dwordx4" in text and "#define G8_NT_STORE 1" in text and "#define G8_STAGGER 1" in text and "#define G8_STAGE_C 1" in text
    text = R.emit_kernel("gemm_fp8", "kernel0", M=4096, N=11008, K=4096, TB=1, OUT_BF16=1, STAGE_C=0)[0]
    assert "#define G8_NT_STORE 0" in text                                               # no two-byte non-temporal stores
    assert d2l(M=4096, N=11008, K=4096, TB=0)
    assert d2l(M=4096, N=11008, K=8192, TB=1) and d2l(M=8192, N=8192, K=8192, TB=0)     # deep k: with more than one round of tiles
    for kw in (dict(TB=0, BTR=0), dict(TA=1, TB=1), dict(M=4000, TB=1), dict(K=4160, TB=1), dict(N=4096, K=8192, TB=1), dict(TB=1, BM=128, BN=128),
               dict(TB=1, D2L=0), dict(TB=1, PREFETCH=0)):
        p = dict(M=4096, N=11008, K=4096); p.update(kw)
        assert not d2l(**p), kw


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("op", ["Add", "Sub", "Mul", "Div", "Pow"])
@pytest.mark.parametrize("sa,sb", [((16, 1, 1, 256), (1, 128, 256)), ((4, 6), (6,)), ((3, 5, 7), (3, 5, 7)),
                                   ((64, 1024), (64, 1)), ((1001,), (1,)), ((2, 768, 768), (768,))])
def test_binary_broadcast_matches_numpy(ops, op, sa, sb):
    """Same fp32 operation per element as the reference's nest (Operators.cc:772-889): bit equality
    for the four arithmetic forms, 1e-6 for Pow (libm against the device's powf)."""
    x, y = O.uniform(sa, 161, 0.5, 2.0), O.uniform(sb, 162, 0.5, 2.0)
    z = host(ops.binary(dev(x), dev(y), op))
    ref = {"Add": x + y, "Sub": x - y, "Mul": x * y, "Div": x / y, "Pow": np.power(x.astype(np.float64), y)}[op]
    assert z.shape == ref.shape
    if op == "Pow":
        assert O.rel_frobenius(z, ref) <= 1e-6
    elif op == "Div":
        assert np.allclose(z, ref, rtol=2e-7, atol=0)      # correctly rounded up to one ulp
    else:
        assert np.array_equal(z, ref.astype(np.float32))


def test_binary_in_place(ops):
    x, y = O.uniform((32, 128), 163), O.uniform((128,), 164)
    xd = dev(x)
    out = ops.binary(xd, dev(y), "Add", inplace=True)
    assert out.data_ptr() == xd.data_ptr() and np.array_equal(host(xd), x + y)


@pytest.mark.parametrize("op", ["Equal", "Greater"])
@pytest.mark.parametrize("sa,sb", [((16, 1, 1, 256), (1, 128, 256)), ((4, 6), (6,)), ((5, 7), (5, 1)), ((1001,), (1001,))])
def test_binary_comparisons_match_numpy(ops, op, sa, sb):
    x, y = np.round(2 * O.normal(sa, stream=201)), np.round(2 * O.normal(sb, stream=202))
    print("binary", op, sa, sb, flush=True)
    z = ops.binary(dev(x), dev(y), op)
    assert z.dtype == torch.bool
    ref = (x == y) if op == "Equal" else (x > y)
    assert ref.any() and not ref.all()
    assert np.array_equal(z.cpu().numpy(), ref)
    nan = np.full(sb, np.nan, dtype=np.float32)          # ordered comparisons: false against NaN
    assert not ops.binary(dev(x), dev(nan), op).any().item()


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape,ishape,axis,dtype", [
    ((2, 5, 8), (2, 3), 1, "float32"),          # index dims in the middle
    ((1000, 256), (77,), 0, "float32"),         # rows of an embedding table, 16-byte units
    ((1000, 250), (64,), 0, "bfloat16"),        # 500-byte rows: 4-byte units
    ((3, 7), (5,), 1, "float32"),               # last axis: one element per row
    ((3, 7), (5,), 1, "bfloat16"),              # last axis, two-byte units
    ((4, 5, 6), (1,), 1, "float32"),            # a single index drops the dimension
    ((8, 33, 3), (4, 4), -2, "int64"),          # 24-byte rows: 8-byte units; negative axis
])
def test_gather_matches_oracle(ops, shape, ishape, axis, dtype):
    rng = np.random.RandomState(17)
    idx = rng.randint(0, shape[axis], size=ishape).astype(np.int64)
    if dtype == "int64":
        x = rng.randint(-2**40, 2**40, size=shape).astype(np.int64)
        xd = torch.from_numpy(x).cuda()
    else:
        x = O.normal(shape, stream=181)
        xd = dev(x).to(torch.bfloat16) if dtype == "bfloat16" else dev(x)
        if dtype == "bfloat16":
            x = O.round_bf16(x)
    print("gather", shape, ishape, axis, dtype, flush=True)
    out = ops.gather(xd, torch.from_numpy(idx).cuda(), axis)
    ref = O.gather(x, idx, axis)
    got = out.float().cpu().numpy() if dtype == "bfloat16" else out.cpu().numpy()
    assert got.shape == ref.shape and np.array_equal(got, ref)


def test_gather_clamps_indices_outside_the_axis(ops):
    """The kernel never reads outside the input: an index below 0 reads row 0, one past the end the last row."""
    x = O.normal((10, 16), stream=182)
    idx = np.array([-5, 0, 9, 10, 1 << 40], dtype=np.int64)
    out = ops.gather(dev(x), torch.from_numpy(idx).cuda(), 0).cpu().numpy()
    assert np.array_equal(out, x[np.clip(idx, 0, 9)])


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("inplace", [False, True])
@pytest.mark.parametrize("shape", [(4, 6, 512), (3, 100), (2, 2, 8, 2048), (5, 1001), (64, 16384), (2, 40000)])
def test_softmax_matches_oracle(ops, shape, inplace):
    x = O.normal(shape, stream=191, std=2.0)
    print("softmax", shape, inplace, flush=True)
    xd = dev(x)
    y = host(ops.softmax(xd, inplace=inplace))
    ref = O.softmax_f64(x)
    assert O.rel_frobenius(y, ref) <= FP32_TOL
    assert O.rel_frobenius(y, O.softmax(x.copy()).astype(np.float64)) <= FP32_TOL     # the reference nest without max subtraction
    assert np.abs(y.sum(-1) - 1.0).max() <= 1e-5
    if inplace:
        assert np.array_equal(host(xd), y)


def test_softmax_is_finite_where_the_plain_quotient_overflows(ops):
    x = O.normal((8, 256), stream=192)
    x[:, 7] = 300.0            # exp overflows fp32: the nest without max subtraction gives inf / inf
    y = host(ops.softmax(dev(x)))
    assert np.isfinite(y).all()
    assert O.rel_frobenius(y, O.softmax_f64(x)) <= FP32_TOL



# ---------------------------------------------------------------------------
def test_streaming_hint_does_not_change_results(ops):
    """STREAM=0 (plain loads, for an input that a producer has just left in the last-level cache) and STREAM=1
    (non-temporal loads, the default) are the same arithmetic: bit-equal outputs for softmax, LayerNorm + GELU
    and GELU."""
    from kernelcodegen_amd import runtime as R
    rows, n = 48, 4096
    x = dev(O.normal((rows, n), stream=331, std=1.5))
    g, b = dev(O.normal((n,), stream=332)), dev(O.normal((n,), stream=333))
    outs = {}
    for stream in (0, 1):
        print("streaming hint", stream, flush=True)
        y_sm, y_ln, y_ew = (torch.empty_like(x) for _ in range(3))
        R.get_kernel("softmax", ROWS=rows, N=n, INPLACE=0, STREAM=stream).launch(x, y_sm)
        R.get_kernel("layernorm", ROWS=rows, N=n, NG=n, NB=n, EPS=1e-5, GELU=1, STREAM=stream).launch(x, g, b, y_ln)
        R.get_kernel("elementwise", N=rows * n, OP="Gelu", INPLACE=0, IN_T="float", OUT_T="float",
                     STREAM=stream).launch(x, y_ew)
        torch.cuda.synchronize()
        outs[stream] = [host(t) for t in (y_sm, y_ln, y_ew)]
    for plain, hinted in zip(outs[0], outs[1]):
        assert np.array_equal(plain, hinted)
    assert O.rel_frobenius(outs[0][0], O.softmax_f64(host(x))) <= FP32_TOL


# ---------------------------------------------------------------------------
# IEEE half, the reference's "float16" (src/Frontend/Operators.cc:5-15): GEMM on v_mfma_f32_32x32x16_f16 and the
# elementwise maps.  numpy's float16 conversion (round to nearest even) rounds the operands.
@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (256, 384, 128), (100, 77, 33), (512, 512, 256)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_matmul_f16_matches_oracle(ops, m, n, k, ta, tb):
    a = O.normal((k, m) if ta else (m, k), stream=501).astype(np.float16)
    b = O.normal((n, k) if tb else (k, n), stream=502, std=0.05).astype(np.float16)
    print("matmul f16", m, n, k, ta, tb, flush=True)
    truth = O.batched_matmul_f64(a.astype(np.float32), b.astype(np.float32), ta, tb)
    c = host(ops.batched_matmul(dev(a), dev(b), trans_a=ta, trans_b=tb))
    assert c.shape == (m, n) and O.rel_frobenius(c, truth) <= 1e-5       # fp32 accumulate of exact half products
    ch = host(ops.batched_matmul(dev(a), dev(b), trans_a=ta, trans_b=tb, out_dtype=torch.float16).float())
    assert O.rel_frobenius(ch, truth) <= LOWP_TOL and O.rel_frobenius(ch, truth) <= 1e-3
    with pytest.raises(ValueError):
        ops.batched_matmul(dev(a), dev(b), trans_a=ta, trans_b=tb, out_dtype=torch.bfloat16)


def test_matmul_f16_exact_small_integers_on_256_tiles(ops):
    rng = np.random.RandomState(41)
    a = rng.randint(-4, 5, size=(512, 192)).astype(np.float16)
    b = rng.randint(-4, 5, size=(192, 768)).astype(np.float16)
    c = host(ops.batched_matmul(dev(a), dev(b), BM=256, BN=256))
    assert np.array_equal(c, O.matmul(a.astype(np.float32), b.astype(np.float32)))


@pytest.mark.parametrize("op", ["Tanh", "Sqrt", "Log", "Relu", "Gelu"])
def test_elementwise_f16_matches_oracle(ops, op):
    x = (O.uniform((3, 1000), stream=503, lo=0.05, hi=9.0) if op in ("Sqrt", "Log") else O.normal((3, 1000), stream=504, std=2.0))
    x = x.astype(np.float16)
    y = host(ops.elementwise(dev(x), op))
    assert y.dtype == np.float16
    ref = O.elementwise(x.astype(np.float32), op)          # the fp32 map of the same half values
    # the kernel computes in fp32 (the fast exp2-based forms: 1e-6 absolute) and rounds once to half
    assert np.allclose(y.astype(np.float32), ref, rtol=2.0 ** -10, atol=1e-6)


# LayerNorm, softmax and the binary operations on half tensors: half in memory, fp32 arithmetic, one rounding of the
# result.  Compared with the oracle's fp32 nests on the same half values; 2^-10 is half a unit in the last place of a
# half result, and the bound of 1e-2 for 16-bit element types holds with a wide margin.
@pytest.mark.parametrize("rows,n,gelu,cfg", [(64, 4096, False, {}), (33, 1000, True, {}), (7, 515, False, dict(VW=1)),
                                             (600, 1024, True, dict(GRID=4))])
def test_layernorm_f16_matches_oracle(ops, rows, n, gelu, cfg):
    x = O.normal((rows, n), stream=511, std=2.0).astype(np.float16)
    g = O.uniform((n,), stream=512, lo=0.5, hi=1.5).astype(np.float16)
    b = O.uniform((n,), stream=513, lo=-0.1, hi=0.1).astype(np.float16)
    print("layernorm f16", rows, n, gelu, cfg, flush=True)
    y = host(ops.layernorm(dev(x), dev(g), dev(b), 1, 1e-5, gelu=gelu, **cfg))
    assert y.dtype == np.float16 and y.shape == x.shape
    ref = O.layernorm(x.astype(np.float32), g.astype(np.float32), b.astype(np.float32), 1)
    if gelu:
        ref = O.elementwise(ref, "Gelu")
    assert O.rel_frobenius(y.astype(np.float32), ref) <= 2.0 ** -10 <= LOWP_TOL
    assert np.allclose(y.astype(np.float32), ref, rtol=2.0 ** -10, atol=2e-3)
    with pytest.raises(ValueError):
        ops.layernorm(dev(x), dev(g.astype(np.float32)), dev(b), 1)


@pytest.mark.parametrize("rows,n,inplace", [(64, 4096, False), (17, 1000, True), (5, 77, False)])
def test_softmax_f16_matches_oracle(ops, rows, n, inplace):
    x = O.normal((rows, n), stream=514, std=3.0).astype(np.float16)
    print("softmax f16", rows, n, inplace, flush=True)
    y = host(ops.softmax(dev(x), inplace=inplace))
    assert y.dtype == np.float16
    ref = O.softmax_f64(x.astype(np.float32))
    assert O.rel_frobenius(y.astype(np.float32), ref) <= 2.0 ** -10 <= LOWP_TOL
    assert np.allclose(y.astype(np.float64), ref, rtol=2.0 ** -10, atol=2.0 ** -24)      # half's smallest subnormal


@pytest.mark.parametrize("op", ["Add", "Sub", "Mul", "Div", "Equal", "Greater"])
@pytest.mark.parametrize("xs,ys", [((64, 4096), (4096,)), ((5, 1, 7), (3, 7)), ((9, 11), (9, 1))])
def test_binary_f16_is_the_correctly_rounded_half_result(ops, op, xs, ys):
    x = O.uniform(xs, stream=515, lo=0.5, hi=2.0).astype(np.float16)
    y = O.uniform(ys, stream=516, lo=0.5, hi=2.0).astype(np.float16)
    if op in ("Equal", "Greater"):
        y = np.broadcast_to(y, np.broadcast_shapes(xs, ys)).copy()
        y.flat[::3] = np.broadcast_to(x, y.shape).flat[::3]          # some equal pairs
        ys = y.shape
    z = host(ops.binary(dev(x), dev(y), op))
    f = {"Add": np.add, "Sub": np.subtract, "Mul": np.multiply, "Div": np.divide, "Equal": np.equal, "Greater": np.greater}[op]
    # numpy's half arithmetic is the fp32 operation rounded once to half: the same as the kernel's, bit for bit
    ref = f(x, y)
    assert z.shape == ref.shape and z.dtype == ref.dtype
    assert np.array_equal(z, ref)
