"""Pins the CPU oracle: known answers, brute force on tiny shapes, closed forms
and invariants, chosen so that a dropped term, a transposed operand or a wrong
index fails at least one check.  The reference's own tests hold no numerical
vector for these operators, so these checks are what anchors the oracle."""
import math

import numpy as np
import pytest

import oracle_lib as O

f32 = np.float32


# ----------------------------------------------------------------------------
# generators
# ----------------------------------------------------------------------------
def test_generators_are_deterministic_and_shaped():
    a = O.uniform((1000,), stream=1)
    b = O.uniform((1000,), stream=1)
    c = O.uniform((1000,), stream=2)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert a.min() >= -1.0 and a.max() < 1.0
    # element i does not depend on how many elements are drawn
    assert np.array_equal(O.uniform((10,), stream=1), a[:10])
    n = O.normal((200000,), stream=3)
    assert abs(float(n.mean())) < 0.01 and abs(float(n.std()) - 1.0) < 0.01
    g = O.uniform((100000,), stream=4, lo=0.5, hi=1.5)
    assert g.min() >= 0.5 and g.max() <= 1.5 and abs(float(g.mean()) - 1.0) < 0.01


# ----------------------------------------------------------------------------
# bf16 / fp8
# ----------------------------------------------------------------------------
def test_bf16_round_to_nearest_even():
    L = O.lib()
    assert L.kcg_oracle_f32_to_bf16(1.0) == 0x3F80
    # 1 + 2^-8 is exactly half way between 1 and 1+2^-7: ties to even -> 1.0
    assert L.kcg_oracle_f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    # 1 + 3*2^-8 is half way between 1+2^-7 (odd) and 1+2^-6 (even) -> up
    assert L.kcg_oracle_f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82
    assert L.kcg_oracle_f32_to_bf16(-2.5) == 0xC020
    # every bf16 pattern that is a finite number survives a round trip
    bits = np.arange(0, 65536, dtype=np.uint16)
    vals = O.from_bf16_bits(bits)
    finite = np.isfinite(vals)
    assert np.array_equal(O.to_bf16_bits(vals[finite]), bits[finite])
    # against torch-free numpy arithmetic: value error below half an ulp
    x = O.normal((10000,), stream=9)
    r = O.round_bf16(x)
    assert np.all(np.abs(r - x) <= np.abs(x) * 2.0 ** -8 + 1e-45)


def test_fp8_e4m3fn_tables():
    L = O.lib()
    dec = L.kcg_oracle_fp8e4m3_to_f32
    assert dec(0x00) == 0.0 and dec(0x38) == 1.0 and dec(0x7E) == 448.0
    assert dec(0x01) == 2.0 ** -9 and dec(0x08) == 2.0 ** -6 and dec(0xB8) == -1.0
    assert math.isnan(dec(0x7F)) and math.isnan(dec(0xFF))
    # all 254 non-NaN patterns round-trip exactly (0x80 is -0 and keeps its sign bit)
    bits = np.array([b for b in range(256) if (b & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(O.to_fp8_bits(O.from_fp8_bits(bits)), bits)
    enc = L.kcg_oracle_f32_to_fp8e4m3
    assert enc(1000.0) == 0x7E and enc(-1000.0) == 0xFE      # saturate, no inf
    assert enc(1.0625) == 0x38                              # tie 1.0 | 1.125 -> even (1.0)
    assert enc(1.1875) == 0x3A                              # tie 1.125 | 1.25 -> even (1.25)
    assert enc(2.0 ** -10) == 0x00 and enc(3 * 2.0 ** -10) == 0x02  # subnormal ties to even
    # nearest: brute force against the decode table
    table = O.from_fp8_bits(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)
    x = np.abs(O.normal((4000,), stream=11, std=20.0)).astype(np.float64)
    got = O.from_fp8_bits(O.to_fp8_bits(x.astype(f32))).astype(np.float64)
    best = np.abs(table[None, :] - np.minimum(x, 448.0)[:, None]).min(axis=1)
    assert np.allclose(np.abs(got - np.minimum(x, 448.0)), best, rtol=0, atol=1e-12)


def test_codecs_agree_with_torch_bit_patterns():
    """An independent implementation of the same two formats (OCP e4m3fn, bfloat16)."""
    torch = pytest.importorskip("torch")
    bits = np.arange(256, dtype=np.uint8)
    ours = O.from_fp8_bits(bits)
    theirs = torch.from_numpy(bits.copy()).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(theirs))
    assert np.array_equal(ours[~np.isnan(ours)], theirs[~np.isnan(theirs)])
    x = np.concatenate([O.normal((20000,), stream=12, std=30.0), O.normal((20000,), stream=13, std=0.01)])
    x = np.clip(x, -448.0, 448.0).astype(f32)          # torch's conversion does not saturate: compare in range
    assert np.array_equal(O.to_fp8_bits(x), torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    assert np.array_equal(O.round_bf16(x), torch.from_numpy(x).bfloat16().float().numpy())


# ----------------------------------------------------------------------------
# matmul
# ----------------------------------------------------------------------------
def _brute_matmul(A, B):
    M, K = A.shape
    N = B.shape[1]
    Cm = np.zeros((M, N), dtype=f32)
    for i in range(M):
        for j in range(N):
            acc = f32(0)
            for k in range(K):
                acc = f32(f32(A[i, k] * B[k, j]) + acc)
            Cm[i, j] = acc
    return Cm


def test_matmul_brute_force_tiny_non_square():
    A = O.uniform((3, 7), stream=1)
    B = O.uniform((7, 5), stream=2)
    ref = _brute_matmul(A, B)
    assert np.array_equal(O.matmul(A, B), ref)
    assert np.array_equal(O.matmul(A, B, nest=True), ref)


def test_matmul_hand_value():
    A = np.array([[1, 2], [3, 4]], dtype=f32)
    B = np.array([[5, 6, 7], [8, 9, 10]], dtype=f32)
    assert np.array_equal(O.matmul(A, B), np.array([[21, 24, 27], [47, 54, 61]], dtype=f32))


def test_matmul_nest_and_interchange_agree_bitwise():
    A = O.uniform((33, 129), stream=3)
    B = O.uniform((129, 65), stream=4)
    assert np.array_equal(O.matmul(A, B), O.matmul(A, B, nest=True))


def test_matmul_identity_transpose_linearity():
    A = O.uniform((16, 16), stream=5)
    B = O.uniform((16, 24), stream=6)
    assert np.array_equal(O.matmul(A, np.eye(16, dtype=f32)), A)
    assert np.array_equal(O.matmul(np.eye(16, dtype=f32), B), B)
    # (AB)^T = B^T A^T holds bit for bit: each element sums the same products in the same order
    assert np.array_equal(O.matmul(A, B).T, O.matmul(B.T.copy(), A.T.copy()))
    # scaling by a power of two is exact
    assert np.array_equal(O.matmul(A * f32(2), B), O.matmul(A, B) * f32(2))
    # fp64 truth and linearity
    t = O.matmul_f64(A, B)
    assert np.allclose(t, A.astype(np.float64) @ B.astype(np.float64), rtol=1e-14, atol=1e-14)
    assert O.rel_frobenius(O.matmul(A, B), t) < 1e-6
    assert np.allclose(O.matmul_rows_f64(A, B, 4, 3), t[4:7], rtol=0, atol=0)


def test_batched_matmul_layouts():
    A = O.uniform((2, 3, 5, 7), stream=7)           # [.., m, k]
    B = O.uniform((2, 3, 7, 4), stream=8)           # [.., k, n]
    ref = np.stack([[_brute_matmul(A[b, h], B[b, h]) for h in range(3)] for b in range(2)])
    assert np.array_equal(O.batched_matmul(A, B), ref)
    Bt = np.ascontiguousarray(np.swapaxes(B, -1, -2))  # [.., n, k]  (colMajor B)
    assert np.array_equal(O.batched_matmul(A, Bt, transB=True), ref)
    At = np.ascontiguousarray(np.swapaxes(A, -1, -2))  # [.., k, m]  (colMajor A)
    assert np.array_equal(O.batched_matmul(At, B, transA=True), ref)
    assert np.array_equal(O.batched_matmul(At, Bt, transA=True, transB=True), ref)
    assert np.allclose(O.batched_matmul_f64(A, Bt, transB=True),
                       A.astype(np.float64) @ B.astype(np.float64), rtol=1e-14, atol=1e-14)


# ----------------------------------------------------------------------------
# softmax
# ----------------------------------------------------------------------------
def test_softmax_closed_form_and_invariants():
    x = np.array([[0.0, math.log(2.0), math.log(3.0)]], dtype=f32)
    assert np.allclose(O.softmax(x), [[1 / 6, 2 / 6, 3 / 6]], rtol=3e-7)
    x = O.normal((5, 4, 37), stream=12)
    p = O.softmax(x)
    assert p.shape == x.shape
    assert np.allclose(p.sum(axis=-1), 1.0, atol=2e-6)
    # naive form equals the max-subtracted form (shift invariance)
    xs = x.astype(np.float64)
    e = np.exp(xs - xs.max(axis=-1, keepdims=True))
    assert np.allclose(p, e / e.sum(axis=-1, keepdims=True), rtol=2e-6)
    assert np.allclose(O.softmax_f64(x), e / e.sum(axis=-1, keepdims=True), rtol=1e-13)
    # the reference's form has no max subtraction: exp(89) overflows fp32 and the row becomes inf/inf
    big = np.array([[89.0, 0.0]], dtype=f32)
    with np.errstate(all="ignore"):
        out = O.softmax(big)
    assert math.isnan(out[0, 0]) and out[0, 1] == 0.0


# ----------------------------------------------------------------------------
# layernorm
# ----------------------------------------------------------------------------
def _golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")) as f:
        return json.load(f)


def test_layernorm_known_answers():
    # fixture written by tests/golden/make_known_answers.py (numpy fp32, the reference's operation order);
    # the first case is also the closed form +-3/sqrt(5), +-1/sqrt(5) up to eps
    for case in _golden()["layernorm"]:
        x = np.array([case["x"]], dtype=f32)
        y = O.layernorm(x, np.array(case["gamma"], f32), np.array(case["beta"], f32), axis=1)
        assert np.allclose(y, [case["y"]], rtol=0, atol=2.4e-7)
    first = _golden()["layernorm"][0]["y"]
    assert np.allclose(first, np.array([-3, -1, 1, 3]) / np.sqrt(5.0 + 4e-5), rtol=0, atol=1e-6)
    assert np.allclose(first, [-1.3416354656, -0.4472118318, 0.4472118318, 1.3416354656], rtol=0, atol=1.2e-7)


def test_layernorm_op_order_matches_numpy_fp32_restatement():
    x = O.normal((3, 50), stream=13)
    g = O.uniform((50,), stream=14, lo=0.5, hi=1.5)
    b = O.uniform((50,), stream=15, lo=-0.1, hi=0.1)
    y = O.layernorm(x, g, b, axis=1)
    ref = np.empty_like(x)
    for r in range(3):
        s = f32(0)
        for v in x[r]:
            s = f32(v + s)
        mean = f32(s / f32(50))
        d = (x[r] - mean).astype(f32)
        v = f32(0)
        for t in d:
            v = f32(f32(t * t) + v)
        den = np.sqrt(f32(f32(v / f32(50)) + f32(1e-5)), dtype=f32)
        ref[r] = (g * (d / den).astype(f32)).astype(f32) + b
    assert np.array_equal(y, ref)


def test_layernorm_invariants_and_axis_grouping():
    x = O.normal((4, 6, 8), stream=16)
    one, zero = np.ones(8, f32), np.zeros(8, f32)
    y = O.layernorm(x, one, zero, axis=2)
    assert np.allclose(y.mean(axis=-1), 0, atol=1e-6)
    assert np.allclose(y.var(axis=-1), 1, atol=1e-4)
    # affine invariance (a > 0), eps small against the variance
    y2 = O.layernorm(x * f32(4) + f32(3), one, zero, axis=2)
    assert np.allclose(y, y2, atol=2e-5)
    # axis=1 normalises over the trailing 6*8 elements, gamma/beta of shape [6,8]
    g = O.uniform((6, 8), stream=17, lo=0.5, hi=1.5)
    b = O.uniform((6, 8), stream=18, lo=-0.1, hi=0.1)
    y3 = O.layernorm(x, g, b, axis=1)
    xs = x.astype(np.float64).reshape(4, 48)
    t = (xs - xs.mean(1, keepdims=True)) / np.sqrt(xs.var(1, keepdims=True) + 1e-5)
    t = t * g.reshape(1, 48) + b.reshape(1, 48)
    assert np.allclose(y3.reshape(4, 48), t, atol=2e-6)
    assert np.allclose(O.layernorm_f64(x, g, b, axis=1).reshape(4, 48), t, atol=1e-7)
    # gamma of shape [8] broadcast over the [6,8] group
    y4 = O.layernorm(x, g[0], b[0], axis=1)
    t4 = (xs - xs.mean(1, keepdims=True)) / np.sqrt(xs.var(1, keepdims=True) + 1e-5)
    t4 = t4.reshape(4, 6, 8) * g[0] + b[0]
    assert np.allclose(y4, t4, atol=2e-6)


# ----------------------------------------------------------------------------
# elementwise
# ----------------------------------------------------------------------------
GELU_KAT = {
    -3.0: -0.0036373436, -1.0: -0.1588081419, -0.5: -0.1542860568, 0.0: 0.0,
    0.5: 0.3457139432, 1.0: 0.8411918879, 2.0: 1.9545974731, 3.0: 2.9963626862,
}


def test_gelu_known_answers_truncated_constants():
    xs = np.array(sorted(GELU_KAT), dtype=f32)
    got = O.elementwise(xs, "Gelu")
    want = np.array([GELU_KAT[float(x)] for x in xs], dtype=np.float64)
    assert np.allclose(got, want, rtol=0, atol=2.4e-7)
    gold = _golden()["gelu"]
    assert np.allclose(O.elementwise(np.array(gold["x"], f32), "Gelu"), gold["y"], rtol=0, atol=1.2e-7)
    # and against an independent fp64 evaluation of the same formula
    ref = 0.5 * xs.astype(np.float64) * (1 + np.tanh(float(f32(0.797884)) * (
        xs.astype(np.float64) + float(f32(0.044715)) * xs.astype(np.float64) ** 3)))
    assert np.allclose(got, ref, rtol=0, atol=2.4e-7)
    assert np.allclose(O.gelu_f64(xs), ref, rtol=1e-14, atol=1e-16)


def test_elementwise_ops_match_libm_forms():
    x = O.uniform((1000,), stream=19, lo=0.1, hi=4.0)
    assert np.allclose(O.elementwise(x, "Sqrt"), np.sqrt(x.astype(np.float64)), rtol=1e-7)
    assert np.allclose(O.elementwise(x, "Log"), np.log(x.astype(np.float64)), rtol=2e-7, atol=1e-7)
    z = O.normal((1000,), stream=20)
    assert np.allclose(O.elementwise(z, "Tanh"), np.tanh(z.astype(np.float64)), rtol=3e-7, atol=1e-7)
    assert np.array_equal(O.elementwise(z, "Relu"), np.maximum(z, 0))


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------
def test_fmha_is_the_composition_of_the_three_nests():
    Q = O.normal((2, 2, 9, 8), stream=21)
    K = O.normal((2, 2, 9, 8), stream=22)
    V = O.normal((2, 2, 9, 8), stream=23)
    S = O.batched_matmul(Q, K, transB=True)
    P = O.softmax(S)
    ref = O.batched_matmul(P, V)
    assert np.array_equal(O.fmha(Q, K, V), ref)
    assert O.rel_frobenius(O.fmha(Q, K, V), O.fmha_f64(Q, K, V)) < 1e-6


def test_fmha_invariants_scale_and_causal():
    S_, D = 17, 8
    Q = O.normal((3, S_, D), stream=24)
    K = O.normal((3, S_, D), stream=25)
    V = O.normal((3, S_, D), stream=26)
    # V constant => O constant
    Vc = np.full_like(V, 0.75)
    assert np.allclose(O.fmha(Q, K, Vc, scale=0.3), 0.75, atol=1e-6)
    # causal: row 0 sees only key 0
    oc = O.fmha(Q, K, V, scale=0.5, causal=True)
    assert np.allclose(oc[:, 0], V[:, 0], atol=1e-6)
    # last row of causal equals non-causal
    on = O.fmha(Q, K, V, scale=0.5, causal=False)
    assert np.allclose(oc[:, -1], on[:, -1], atol=1e-6)
    # textbook definition in fp64
    s = np.einsum("bid,bjd->bij", Q.astype(np.float64), K.astype(np.float64)) * 0.5
    mask = np.tril(np.ones((S_, S_), dtype=bool))
    sc = np.where(mask, s, -np.inf)
    for name, sm, causal in (("full", s, False), ("causal", sc, True)):
        p = np.exp(sm - sm.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        t = p @ V.astype(np.float64)
        assert np.allclose(O.fmha_f64(Q, K, V, scale=0.5, causal=causal), t, rtol=1e-12, atol=1e-14), name
        assert np.allclose(O.fmha(Q, K, V, scale=0.5, causal=causal), t, atol=3e-6), name
        assert np.allclose(O.fmha_rows_f64(Q[1], K[1], V[1], 5, 4, scale=0.5, causal=causal),
                           t[1, 5:9], rtol=1e-12, atol=1e-14), name
    # scaling Q by c equals scaling the logits by c
    assert np.allclose(O.fmha_f64(Q * f32(0.5), K, V, scale=1.0), O.fmha_f64(Q, K, V, scale=0.5),
                       rtol=1e-12, atol=1e-14)


def test_gather_matches_numpy_take_and_a_plain_loop():
    """Pins kcg_oracle_gather: numpy.take is the same definition as a library routine; a pure-Python loop
    over a tiny case restates it independently; identity indices return the input; an index outside the
    axis is refused."""
    x = O.normal((3, 5, 4), stream=401)
    for axis, idx in [(0, np.array([2, 0, 2, 1])), (1, np.array([[4, 0], [1, 1], [3, 2]])), (2, np.array([3])), (-1, np.array([0, 3, 3]))]:
        got = O.gather(x, idx, axis)
        want = np.take(x, idx[0] if idx.shape == (1,) else idx, axis=axis)
        assert got.shape == want.shape and np.array_equal(got, want)
    idx = np.array([[4, 0], [1, 1]])
    got = O.gather(x, idx, 1)
    for o in range(3):
        for i0 in range(2):
            for i1 in range(2):
                for r in range(4):
                    assert got[o, i0, i1, r] == x[o, idx[i0, i1], r]
    assert np.array_equal(O.gather(x, np.arange(5), 1), x)
    b = O.to_bf16_bits(x)                      # two-byte elements move as bytes
    assert np.array_equal(O.gather(b, np.array([1, 1, 0]), 0), np.take(b, [1, 1, 0], axis=0))
    with pytest.raises(IndexError):
        O.gather(x, np.array([5]), 1)
    with pytest.raises(IndexError):
        O.gather(x, np.array([-1, 0]), 1)

