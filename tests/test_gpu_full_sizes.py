"""GPU parity of the code paths the benchmark times: the benchmark problem sizes with the default tiles, and
small ragged shapes on which the large workgroup tiles, the persistent LayerNorm loop and the two-units-per-lane
gather are forced through kernel parameters.  Inputs come from the oracle's seeded generator; the truth is the
oracle's fp64-accumulated product on the same (rounded / quantised) operands, on sampled full rows of C for the
large GEMMs and on the full tensor for LayerNorm."""
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


def sample_rows(m, tile=256, count=64):
    """`count` rows of an m-row result (m >= tile) such that every 32-row MFMA block position of a `tile`-row
    workgroup tile (so every wavefront row of it) and many different tiles are hit, plus the first and last row."""
    tiles = max(1, m // tile)
    rows = {0, m - 1}
    for i in range(count):
        rows.add(min(m - 1, (i * 5 % tiles) * tile + (i * 67 + 3) % tile))
    rows = sorted(rows)
    blocks = {(r % tile) // 32 for r in rows}
    assert len(blocks) == tile // 32
    return np.array(rows, dtype=np.int64)


# ---------------------------------------------------------------------------
# C5: 4096 x 11008 x 4096, bf16 and fp8 e4m3, default tiles (256 x 256)
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("out_bf16", [False, True])
def test_gemm_bf16_4096x11008x4096_sampled_rows(ops, tb, out_bf16):
    m, n, k = 4096, 11008, 4096
    a = O.round_bf16(O.normal((m, k), stream=401))
    bt = O.round_bf16(O.normal((n, k), stream=402, std=0.02))          # [N][K]
    b = bt if tb else np.ascontiguousarray(bt.T)
    print("gemm bf16 full size tb=%s out_bf16=%s" % (tb, out_bf16), flush=True)
    c = ops.batched_matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16), trans_b=tb,
                           out_dtype=torch.bfloat16 if out_bf16 else torch.float32)
    rows = sample_rows(m)
    truth = O.batched_matmul_f64(a[rows], bt, False, True)
    got = host(c[torch.from_numpy(rows).cuda()].float())
    assert got.shape == (len(rows), n)
    assert O.rel_frobenius(got, truth) <= (LOWP_TOL if out_bf16 else 1e-5)
    # every tile wrote something finite (a skipped tile would leave the buffer's zeros: probability ~0 otherwise)
    cs = c.float()
    assert torch.isfinite(cs).all().item()
    assert (cs.abs().reshape(m // 256, 256, n // 256, 256).amax(dim=(1, 3)) > 0).all().item()


@pytest.mark.parametrize("tb", [True, False])
def test_gemm_fp8_4096x11008x4096_sampled_rows(ops, tb):
    m, n, k = 4096, 11008, 4096
    a = O.normal((m, k), stream=403)
    bt = O.normal((n, k), stream=404, std=0.02)
    sa, sb = float(np.abs(a).max()) / 448.0, float(np.abs(bt).max()) / 448.0
    abits, bbits = O.to_fp8_bits(a, 1.0 / sa), O.to_fp8_bits(bt, 1.0 / sb)
    del a, bt
    print("gemm fp8 full size tb=%s" % tb, flush=True)
    bdev = dev(bbits if tb else np.ascontiguousarray(bbits.T)).view(torch.float8_e4m3fn)
    c = ops.matmul_fp8(dev(abits).view(torch.float8_e4m3fn), bdev, sa, sb, trans_b=tb)
    rows = sample_rows(m)
    truth = O.batched_matmul_f64(O.from_fp8_bits(abits[rows]), O.from_fp8_bits(bbits), False, True) * (sa * sb)
    got = host(c[torch.from_numpy(rows).cuda()])
    assert O.rel_frobenius(got, truth) <= 1e-4
    assert torch.isfinite(c).all().item()
    assert (c.abs().reshape(m // 256, 256, n // 256, 256).amax(dim=(1, 3)) > 0).all().item()


# ---------------------------------------------------------------------------
# C2: fp32 4096^3 and 16 x 1024^3 (256 x 256 x 16 tiles, 16 wavefronts)
def test_gemm_f32_4096_sampled_rows(ops):
    n = 4096
    a, b = O.uniform((n, n), stream=405), O.uniform((n, n), stream=406)
    print("gemm f32 4096", flush=True)
    c = ops.matmul(dev(a), dev(b))
    rows = sample_rows(n)
    truth = O.matmul_f64(a[rows], b)
    got = host(c[torch.from_numpy(rows).cuda()])
    assert O.rel_frobenius(got, truth) <= FP32_TOL
    assert O.rel_frobenius(got[:8], O.matmul(a[rows[:8]], b)) <= FP32_TOL      # the sequential fp32 nest
    assert (c.abs().reshape(16, 256, 16, 256).amax(dim=(1, 3)) > 0).all().item()


def test_batched_gemm_f32_16x1024_sampled_rows(ops):
    batch, n = 16, 1024
    a, b = O.uniform((batch, n, n), stream=407), O.uniform((batch, n, n), stream=408)
    print("bgemm f32 16 x 1024", flush=True)
    c = ops.batched_matmul(dev(a), dev(b))
    rows = sample_rows(n, count=32)
    for bi in (0, 5, 10, 15):
        truth = O.matmul_f64(a[bi][rows], b[bi])
        assert O.rel_frobenius(host(c[bi][torch.from_numpy(rows).cuda()]), truth) <= FP32_TOL
    assert (c.abs().reshape(batch, 4, 256, 4, 256).amax(dim=(2, 4)) > 0).all().item()


# ---------------------------------------------------------------------------
# C3: LayerNorm 16384 x 4096 + GELU, the whole tensor
@pytest.mark.parametrize("gelu", [True, False])
def test_layernorm_16384x4096_full_tensor(ops, gelu):
    rows, n = 16384, 4096
    x = O.normal((rows, n), stream=409)
    g = O.uniform((n,), stream=410, lo=0.5, hi=1.5)
    b = O.uniform((n,), stream=411, lo=-0.1, hi=0.1)
    print("layernorm 16384 x 4096 gelu=%s" % gelu, flush=True)
    y = host(ops.layernorm(dev(x), dev(g), dev(b), 1, 1e-5, gelu=gelu))
    ref = O.layernorm(x, g, b, 1)
    if gelu:
        ref = O.elementwise(ref, "Gelu")
    num = den = 0.0
    worst = 0.0
    for r0 in range(0, rows, 1024):           # in slices: the fp64 differences of 64 M elements need not exist at once
        d = y[r0:r0 + 1024].astype(np.float64) - ref[r0:r0 + 1024]
        num += float((d * d).sum())
        den += float((ref[r0:r0 + 1024].astype(np.float64) ** 2).sum())
        worst = max(worst, float(np.abs(d).max()))
    assert (num / den) ** 0.5 <= FP32_TOL
    assert worst <= 2e-5
    # a sample of rows against the fp64 form as well
    rs = sample_rows(rows, count=32)
    ref64 = O.layernorm_f64(x[rs], g, b, 1)
    if gelu:
        ref64 = O.gelu_f64(ref64.astype(np.float32))
    assert O.rel_frobenius(y[rs], ref64) <= FP32_TOL


@pytest.mark.parametrize("rows,n,grid", [(4096, 4096, 8), (1000, 1024, 3), (77, 4096, 2), (515, 1000, 4)])
@pytest.mark.parametrize("gelu", [False, True])
def test_layernorm_persistent_loop(ops, rows, n, grid, gelu):
    """GRID workgroups walk many row groups each: the next-row prefetch, the hand-over of the prefetched row and
    the reuse of the reduction cells across iterations all run; the last trip of some workgroups is past the end."""
    x = O.normal((rows, n), stream=412, std=1.7)
    g = O.uniform((n,), stream=413, lo=0.5, hi=1.5)
    b = O.uniform((n,), stream=414, lo=-0.1, hi=0.1)
    print("layernorm persistent", rows, n, grid, gelu, flush=True)
    y = host(ops.layernorm(dev(x), dev(g), dev(b), 1, 1e-5, gelu=gelu, GRID=grid))
    ref = O.layernorm(x, g, b, 1)
    if gelu:
        ref = O.elementwise(ref, "Gelu")
    assert O.rel_frobenius(y, ref) <= FP32_TOL
    assert np.allclose(y, ref, rtol=0, atol=2e-5)


# ---------------------------------------------------------------------------
# The large tiles on small ragged problems: tile choice and shape decoupled.
BIG_TILES = [(256, 256), (128, 128), (128, 64), (256, 128)]
RAGGED = [(512, 512, 256), (300, 520, 200), (257, 259, 72), (640, 384, 1024)]


@pytest.mark.parametrize("bm,bn", BIG_TILES)
@pytest.mark.parametrize("m,n,k", RAGGED)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_matmul_bf16_forced_tiles(ops, m, n, k, bm, bn, ta, tb):
    a = O.round_bf16(O.normal((k, m) if ta else (m, k), stream=421))
    b = O.round_bf16(O.normal((n, k) if tb else (k, n), stream=422, std=0.02))
    print("matmul bf16 tile", bm, bn, "shape", m, n, k, ta, tb, flush=True)
    c = host(ops.batched_matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16), trans_a=ta, trans_b=tb,
                                BM=bm, BN=bn))
    assert O.rel_frobenius(c, O.batched_matmul_f64(a, b, ta, tb)) <= 1e-5


@pytest.mark.parametrize("bm,bn", BIG_TILES)
@pytest.mark.parametrize("m,n,k", RAGGED)
@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, True)])
def test_matmul_fp8_forced_tiles(ops, m, n, k, bm, bn, ta, tb):
    a = O.normal((k, m) if ta else (m, k), stream=423)
    b = O.normal((n, k) if tb else (k, n), stream=424, std=0.02)
    sa, sb = float(np.abs(a).max()) / 448.0, float(np.abs(b).max()) / 448.0
    abits, bbits = O.to_fp8_bits(a, 1.0 / sa), O.to_fp8_bits(b, 1.0 / sb)
    print("matmul fp8 tile", bm, bn, "shape", m, n, k, ta, tb, flush=True)
    c = host(ops.matmul_fp8(dev(abits).view(torch.float8_e4m3fn), dev(bbits).view(torch.float8_e4m3fn), sa, sb,
                            trans_a=ta, trans_b=tb, BM=bm, BN=bn))
    truth = O.batched_matmul_f64(O.from_fp8_bits(abits), O.from_fp8_bits(bbits), ta, tb) * (sa * sb)
    assert O.rel_frobenius(c, truth) <= 1e-4


@pytest.mark.parametrize("bm,bn,bk", [(256, 256, 16), (128, 128, 32), (128, 128, 16), (64, 64, 32)])
@pytest.mark.parametrize("m,n,k", RAGGED)
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_matmul_f32_forced_tiles(ops, m, n, k, bm, bn, bk, ta, tb):
    a = O.uniform((k, m) if ta else (m, k), stream=425)
    b = O.uniform((n, k) if tb else (k, n), stream=426)
    print("matmul f32 tile", bm, bn, bk, "shape", m, n, k, ta, tb, flush=True)
    c = host(ops.batched_matmul(dev(a), dev(b), trans_a=ta, trans_b=tb, BM=bm, BN=bn, BK=bk))
    assert O.rel_frobenius(c, O.batched_matmul_f64(a, b, ta, tb)) <= FP32_TOL


def test_matmul_exact_small_integers_on_256_tiles(ops):
    """Bit equality on the 256 x 256 tiles of all three GEMM families (operand order inside the MFMA steps, the
    epilogue's row / column mapping and the batch offsets)."""
    rng = np.random.RandomState(21)
    a = rng.randint(-4, 5, size=(2, 512, 192)).astype(np.float32)
    b = rng.randint(-4, 5, size=(2, 192, 768)).astype(np.float32)
    truth = np.stack([O.matmul(a[i], b[i]) for i in range(2)])
    assert np.array_equal(host(ops.batched_matmul(dev(a), dev(b), BM=256, BN=256, BK=16)), truth)
    assert np.array_equal(host(ops.batched_matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16), BM=256, BN=256)),
                          truth)
    c8 = host(ops.matmul_fp8(dev(O.to_fp8_bits(a)).view(torch.float8_e4m3fn), dev(O.to_fp8_bits(b)).view(torch.float8_e4m3fn),
                             1.0, 1.0, trans_b=False, BM=256, BN=256))
    assert np.array_equal(c8, truth)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("unroll", [1, 2, 4])
@pytest.mark.parametrize("shape,nidx,dtype", [((32000, 4096), 1500, "bfloat16"), ((999, 250), 4097, "bfloat16"),
                                              ((77, 1000), 333, "float32")])
def test_gather_units_per_lane(ops, shape, nidx, dtype, unroll):
    """UNROLL units per lane (the default above a million units is 2), with a last workgroup that is partly
    past the end."""
    rng = np.random.RandomState(23)
    idx = rng.randint(0, shape[0], size=(nidx,)).astype(np.int64)
    x = O.normal(shape, stream=431)
    xd = dev(x).to(torch.bfloat16) if dtype == "bfloat16" else dev(x)
    if dtype == "bfloat16":
        x = O.round_bf16(x)
    print("gather unroll", unroll, shape, nidx, dtype, flush=True)
    out = ops.gather(xd, torch.from_numpy(idx).cuda(), 0, UNROLL=unroll)
    assert np.array_equal(host(out.float()), O.gather(x, idx, 0))


def test_gather_benchmark_shape_default_parameters(ops):
    """16384 rows out of a 32000 x 4096 bf16 table: the default picks two units per lane."""
    from kernelcodegen_amd import runtime as R
    _, info = R.emit_kernel("gather", "kernel0", OUTER=1, AXIS=32000, NIDX=16384, INNER=4096, ESIZE=2)
    assert info["grid"][0] == 16384 * 512 // (256 * 2)
    rng = np.random.RandomState(29)
    idx = rng.randint(0, 32000, size=(16384,)).astype(np.int64)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    table = torch.randn((32000, 4096), device="cuda", generator=g).bfloat16()
    out = ops.gather(table, torch.from_numpy(idx).cuda(), 0)
    assert torch.equal(out, table[torch.from_numpy(idx).cuda()])
    th = host(table[:64].float())
    assert np.array_equal(host(ops.gather(table[:64].contiguous(), torch.arange(63, -1, -1, device="cuda"), 0).float()),
                          O.gather(th, np.arange(63, -1, -1), 0))


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("causal", [False, True])
def test_fmha_bf16_full_size_all_wavefronts(ops, causal):
    """B8 H32 S2048 D128 with the oracle's generator: eight (batch, head) slabs, in each one row group per
    wavefront of a 256-query tile (eight wavefronts of 32 queries), in different query tiles."""
    b, h, s, d = 8, 32, 2048, 128
    shp = (b, h, s, d)
    scale = d ** -0.5
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (441, 442, 443))
    print("fmha full size, all wavefronts, causal=%s" % causal, flush=True)
    o = ops.fmha(*(dev(t).to(torch.bfloat16) for t in (q, k, v)), scale=scale, causal=causal, out_dtype=torch.float32)
    assert torch.isfinite(o).all().item()
    slabs = [(0, 0), (1, 9), (2, 18), (3, 27), (4, 4), (5, 13), (6, 22), (7, 31)]
    for n_, (bi, hi) in enumerate(slabs):
        got, want = [], []
        for w in range(8):
            tile = (n_ + 3 * w) % (s // 256)
            row0 = tile * 256 + w * 32 + (5 * n_ + w) % 29
            want.append(O.fmha_rows_f64(q[bi, hi], k[bi, hi], v[bi, hi], row0, 4, scale=scale, causal=causal))
            got.append(host(o[bi, hi, row0:row0 + 4]))
        assert O.rel_frobenius(np.concatenate(got), np.concatenate(want)) <= 4e-3


@pytest.mark.parametrize("d,causal,scale", [(64, False, 1.0), (128, True, None)])
def test_fmha_f32_full_size_all_wavefronts(ops, d, causal, scale):
    """fp32 attention at B8 H32 S2048: the reference's own graph (test/test.cc:107-147: head dim 64, no scale, no mask)
    and the benchmark's shape and semantics (head dim 128, 1/sqrt(D), causal) on the fp32 MFMA; eight (batch, head)
    slabs, in each one row group per wavefront of a 128-query tile, in different query tiles; the fp32 bar."""
    b, h, s = 8, 32, 2048
    shp = (b, h, s, d)
    scale = d ** -0.5 if scale is None else scale
    std = 1.0 if scale < 1.0 else d ** -0.25
    q, k, v = (O.normal(shp, stream=st, std=std) for st in (481, 482, 483))
    print("fmha f32 full size, head dim %d causal=%s" % (d, causal), flush=True)
    o = ops.fmha(*(dev(t) for t in (q, k, v)), scale=scale, causal=causal)
    assert o.dtype == torch.float32 and torch.isfinite(o).all().item()
    slabs = [(0, 0), (1, 9), (2, 18), (3, 27), (4, 4), (5, 13), (6, 22), (7, 31)]
    for n_, (bi, hi) in enumerate(slabs):
        got, want = [], []
        for w in range(4):
            tile = (n_ + 5 * w) % (s // 128)
            row0 = tile * 128 + w * 32 + (5 * n_ + w) % 29
            want.append(O.fmha_rows_f64(q[bi, hi], k[bi, hi], v[bi, hi], row0, 4, scale=scale, causal=causal))
            got.append(host(o[bi, hi, row0:row0 + 4]))
        assert O.rel_frobenius(np.concatenate(got), np.concatenate(want)) <= 1e-5


# Persistent workgroups (more query tiles than compute units): a workgroup takes its tiles one after the other, the
# key tiles of consecutive jobs forming one stream; 640 tiles (320 pairs under the mask) over 256 workgroups give
# workgroups with two and with three jobs.  bf16 result, which goes through the LDS-staged epilogue.
FMHA_VARIANTS = [
    dict(),                        # defaults: persistent, pairs under the mask, staged result tiles
    dict(PERSIST=0),               # one job per workgroup
    dict(STAGE_O=0),               # result rows written straight from the accumulator layout
    dict(PAIR=1),                  # (causal) the two query tiles of a job from one head instead of two
    dict(PAIR=0),                  # (causal) one query tile per job, not persistent
]


@pytest.mark.parametrize("cfg", FMHA_VARIANTS, ids=lambda c: "-".join("%s%d" % kv for kv in c.items()) or "default")
@pytest.mark.parametrize("causal", [False, True])
def test_fmha_bf16_persistent_workgroups(ops, causal, cfg):
    from kernelcodegen_amd import runtime as R
    b, h, s, d = 2, 80, 1024, 128
    _, info = R.emit_kernel("fmha_bf16", "kernel0", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=d ** -0.5, **cfg)
    persistent = cfg.get("PERSIST", 1) and not (causal and cfg.get("PAIR", 1) == 0)
    assert info["grid"][0] == (256 if persistent else (s // 256) * b * h // (2 if causal and cfg.get("PAIR", 1) else 1))
    shp = (b, h, s, d)
    scale = d ** -0.5
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (461, 462, 463))
    print("fmha persistent", causal, cfg, flush=True)
    o = ops.fmha(*(dev(t).to(torch.bfloat16) for t in (q, k, v)), scale=scale, causal=causal, **cfg)
    assert o.dtype == torch.bfloat16 and torch.isfinite(o.float()).all().item()
    # slabs that are a workgroup's first, second and third job, every query tile, every wavefront
    slabs = [(0, 0), (0, 37), (0, 70), (1, 3), (1, 50), (1, 79)]
    for n_, (bi, hi) in enumerate(slabs):
        got, want = [], []
        for w in range(8):
            tile = (n_ + w) % (s // 256)
            row0 = tile * 256 + w * 32 + (7 * n_ + 3 * w) % 29
            want.append(O.fmha_rows_f64(q[bi, hi], k[bi, hi], v[bi, hi], row0, 4, scale=scale, causal=causal))
            got.append(host(o[bi, hi, row0:row0 + 4].float()))
        assert O.rel_frobenius(np.concatenate(got), np.concatenate(want)) <= 1e-2      # bf16 result


# The same with other tiles: 128 queries per job (two diagonal tiles under the mask), 32-key tiles (no steady-state
# form: the general iteration carries the job stream alone), head dim 256 (result rows written without staging).
@pytest.mark.parametrize("b,h,s,d,cfg", [
    (4, 40, 512, 64, dict(BR=128, BC=64)),
    (4, 40, 512, 64, dict(BR=128, BC=32, PERSIST=1)),      # persistent on request (the default is not, without the steady-state form)
    (2, 80, 512, 256, dict()),
    (2, 80, 1024, 256, dict(PERSIST=1)),
    (3, 50, 768, 128, dict()),          # three query tiles: under the mask pairs across two heads, (2, 0) (1, 1) (0, 2)
    (3, 25, 768, 128, dict()),          # ... and an odd number of heads: no pairs, so not persistent under the mask
])
@pytest.mark.parametrize("causal", [False, True])
def test_fmha_bf16_persistent_other_tiles(ops, b, h, s, d, cfg, causal):
    from kernelcodegen_amd import runtime as R
    _, info = R.emit_kernel("fmha_bf16", "kernel0", B=b, H=h, S=s, D=d, CAUSAL=int(causal), SCALE=d ** -0.5, **cfg)
    br = cfg.get("BR", 256)
    nq = s // br
    # under the mask a workgroup takes two query tiles: of two heads where the number of heads is even, else of one head
    # where the number of query tiles is
    across = causal and (b * h) % 2 == 0
    paired = across or (causal and nq % 2 == 0)
    items = nq * (b * h // 2) if across else (nq // 2 if paired else nq) * b * h
    steady = cfg.get("BC", 64 if d <= 128 else 32) == 64 and d % 64 == 0
    assert info["grid"][0] == (256 if cfg.get("PERSIST", steady) and (not causal or paired) and items > 256 else items)
    shp = (b, h, s, d)
    scale = d ** -0.5
    q, k, v = (O.round_bf16(O.normal(shp, stream=st)) for st in (471, 472, 473))
    print("fmha persistent, other tiles", shp, cfg, causal, flush=True)
    o = ops.fmha(*(dev(t).to(torch.bfloat16) for t in (q, k, v)), scale=scale, causal=causal, **cfg)
    assert torch.isfinite(o.float()).all().item()
    for n_, (bi, hi) in enumerate([(0, 0), (0, h - 1), (b - 1, h // 2), (b - 1, h - 1), (b // 2, 7)]):
        got, want = [], []
        for w in range(4):
            row0 = ((n_ + w) % nq) * br + (w * 32 + 5 * n_) % (br - 4)
            want.append(O.fmha_rows_f64(q[bi, hi], k[bi, hi], v[bi, hi], row0, 4, scale=scale, causal=causal))
            got.append(host(o[bi, hi, row0:row0 + 4].float()))
        assert O.rel_frobenius(np.concatenate(got), np.concatenate(want)) <= 1e-2      # bf16 result


# ---------------------------------------------------------------------------
# Tail split of the bf16 GEMM (on request): the tiles behind the first SK_FULL are cut along k between SK_UNITS
# extra workgroups that leave partial sums in a workspace.
SPLITS = [
    # m, n, k, tile, SK_FULL, SK_UNITS
    (768, 768, 512, 128, 32, 16),      # 36 tiles, 4 in the tail: runs of 2 iterations, one segment each
    (640, 1024, 512, 128, 16, 32),     # 40 tiles, 24 in the tail, per-XCD runs of 6 of 8 iterations: two segments per unit
    (600, 1000, 512, 128, 16, 32),     # the same with ragged tiles
    (640, 1024, 1024, 128, 24, 24),    # 16 tail tiles over 24 units: runs of 12 of 16 iterations, three parts in some tiles
    (512, 768, 2048, 256, 0, 16),      # every tile split (6 tiles of 256 x 256 over 16 units, runs of 12 of 32)
]


@pytest.mark.parametrize("m,n,k,tile,full,units", SPLITS)
@pytest.mark.parametrize("ta,tb,out_bf16", [(False, False, False), (False, True, True), (True, False, False)])
def test_matmul_bf16_tail_split(ops, m, n, k, tile, full, units, ta, tb, out_bf16):
    a = O.round_bf16(O.normal((k, m) if ta else (m, k), stream=451))
    b = O.round_bf16(O.normal((n, k) if tb else (k, n), stream=452, std=0.02))
    print("matmul bf16 tail split", m, n, k, tile, full, units, ta, tb, out_bf16, flush=True)
    ad, bd = dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16)
    cfg = dict(BM=tile, BN=tile, SK_FULL=full, SK_UNITS=units)
    out_dtype = torch.bfloat16 if out_bf16 else torch.float32
    truth = O.batched_matmul_f64(a, b, ta, tb)
    first = ops.batched_matmul(ad, bd, trans_a=ta, trans_b=tb, out_dtype=out_dtype, **cfg)
    assert O.rel_frobenius(host(first.float()), truth) <= (LOWP_TOL if out_bf16 else 1e-5)
    # the same kernel object again, on the workspace the first launch left behind (its counters must be back at
    # zero), and bit-equal: the partial sums are added in k order whoever arrives last
    for _ in range(3):
        again = ops.batched_matmul(ad, bd, trans_a=ta, trans_b=tb, out_dtype=out_dtype, **cfg)
        assert torch.equal(first, again)
    # and within rounding of the unsplit kernel (the split changes the association of the k sum)
    whole = ops.batched_matmul(ad, bd, trans_a=ta, trans_b=tb, out_dtype=out_dtype, BM=tile, BN=tile, SK_UNITS=0)
    assert O.rel_frobenius(host(first.float()), host(whole.float()).astype(np.float64)) <= (4e-3 if out_bf16 else 2e-6)


def test_matmul_bf16_tail_split_exact_and_only_on_request(ops):
    from kernelcodegen_amd import runtime as R
    rng = np.random.RandomState(31)
    a = rng.randint(-4, 5, size=(640, 512)).astype(np.float32)
    b = rng.randint(-4, 5, size=(512, 1024)).astype(np.float32)
    c = ops.batched_matmul(dev(a).to(torch.bfloat16), dev(b).to(torch.bfloat16), BM=128, BN=128, SK_FULL=16, SK_UNITS=32)
    assert np.array_equal(host(c), O.matmul(a, b))
    # the benchmark shape on request: 688 tiles of 256 x 256 = 512 whole-tile workgroups + 256 units over 176 tail tiles
    _, info = R.emit_kernel("gemm_bf16", "kernel0", M=4096, N=11008, K=4096, SK_UNITS=256)
    assert info["grid"][0] == 768 and info["num_args"] == 4 and info["workspace_bytes"] == 4096 + 256 * 2 * 256 * 256 * 4
    # never by default
    for shape in (dict(M=4096, N=11008, K=4096), dict(M=4096, N=4096, K=4096), dict(M=1024, N=1024, K=1024)):
        _, info = R.emit_kernel("gemm_bf16", "kernel0", **shape)
        assert info["workspace_bytes"] == 0 and info["num_args"] == 3
