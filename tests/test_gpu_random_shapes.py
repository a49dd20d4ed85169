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
