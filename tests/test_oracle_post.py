"""Pins the oracle's restatement of the step between the QKV projection and the cache (RMS normalisation, partial
rotary embedding, 128-point signed Hadamard rotation) against numpy fp64 forms and structural properties.  CPU only."""
import numpy as np
import pytest
from scipy.linalg import hadamard

from oracle import yko


def _h(x):
    return np.asarray(x, np.uint16).view(np.float16).astype(np.float64)


def test_rotate128_is_signed_sylvester_matrix_exact_on_integers():
    rng = np.random.default_rng(1)
    x = rng.integers(-8, 9, size=(8, 128)).astype(np.float32)
    H = hadamard(128).astype(np.float64)
    s = yko.kvx_signs()[:128].astype(np.float64)
    for factor in (0.125, 0.0625):
        fwd = (H @ (x * s).T).T * factor
        assert np.array_equal(yko.rotate128(x, False, factor), fwd.astype(np.float32))
        inv = (H @ x.astype(np.float64).T).T * factor * s
        assert np.array_equal(yko.rotate128(x, True, factor), inv.astype(np.float32))


def test_rotation_factors_compose_to_identity_and_keep_dot_products():
    rng = np.random.default_rng(2)
    q = rng.standard_normal((16, 128)).astype(np.float32)
    k = rng.standard_normal((16, 128)).astype(np.float32)
    rq, rk = yko.rotate128(q, False, 0.0625), yko.rotate128(k, False, 0.125)
    assert np.allclose((rq.astype(np.float64) * rk).sum(1), (q.astype(np.float64) * k).sum(1), rtol=0, atol=2e-5)
    back = yko.rotate128(yko.rotate128(k, False, 0.125), True, 0.0625)   # V forward, output inverse
    assert np.abs(back - k).max() < 2e-6


def _post_numpy(y, w16, eps, cs, rd):
    """fp64 RMS normalisation + rotary as complex multiplication, no intermediate rounding"""
    y = y.astype(np.float64)
    r = 1.0 / np.sqrt((y * y).mean() + eps)
    xn = y * r * (1.0 + _h(w16))
    hr = rd // 2
    z = (xn[:hr] + 1j * xn[hr:rd]) * (cs[:, 0] + 1j * cs[:, 1])
    out = xn.copy(); out[:hr] = z.real; out[hr:rd] = z.imag
    return out


def test_post_rows_match_fp64_forms():
    rng = np.random.default_rng(3)
    M, H, KVH, rd, pos = 5, 24, 4, 32, 37
    xq = (rng.standard_normal((M, H, 128)) * 3).astype(np.float32)
    xk = (rng.standard_normal((M, KVH, 128)) * 0.5).astype(np.float32)
    xv = rng.standard_normal((M, KVH, 128)).astype(np.float32)
    qw = (rng.standard_normal(128) * 0.1).astype(np.float16).view(np.uint16)
    kw = (rng.standard_normal(128) * 0.1).astype(np.float16).view(np.uint16)
    rope = yko.rope_table(64, rd)
    q16, k16, v16 = yko.attn_post(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot=0)
    for t in range(M):
        cs = rope[pos + t].astype(np.float64)
        for h in range(H):
            ref = _post_numpy(xq[t, h], qw, 1e-6, cs, rd)
            # three fp16 roundings on the rotary channels, one elsewhere
            assert np.abs(_h(q16[t, h]) - ref).max() <= 2.5e-3 * max(1.0, np.abs(ref).max())
        for h in range(KVH):
            ref = _post_numpy(xk[t, h], kw, 1e-6, cs, rd)
            assert np.abs(_h(k16[t, h]) - ref).max() <= 2.5e-3 * max(1.0, np.abs(ref).max())
    # V rows: plain rounding to fp16
    assert np.array_equal(v16, xv.astype(np.float16).view(np.uint16))
    # channels past rd carry no rotary change: the entry rounding and one more
    r16 = lambda a: a.astype(np.float16).astype(np.float32)
    ref = _post_numpy(r16(xq[0, 0]), qw, 1e-6, rope[pos].astype(np.float64), rd)
    assert np.abs(_h(q16[0, 0, rd:]) - ref[rd:]).max() <= 1.0e-3 * max(1.0, np.abs(ref).max())


def test_post_structure():
    rng = np.random.default_rng(4)
    rd = 32
    x = rng.standard_normal((1, 1, 128)).astype(np.float32)
    zero_w = np.zeros(128, np.uint16)
    rope = yko.rope_table(16, rd)
    # position 0: cos = 1, sin = 0 -> the rotary step changes nothing; unit RMS after normalisation
    q16, _, _ = yko.attn_post(x, x[:, :1], x[:, :1], zero_w, zero_w, 0.0, rope, rd, 0, 0)
    assert abs(np.sqrt((_h(q16) ** 2).mean()) - 1.0) < 1e-3
    qb, _, _ = yko.attn_post(x, x[:, :1], x[:, :1], zero_w, zero_w, 0.0, rope, rd, 7, 0)
    a, b = _h(q16)[0, 0], _h(qb)[0, 0]
    hr = rd // 2
    assert np.allclose(a[:hr] ** 2 + a[hr:rd] ** 2, b[:hr] ** 2 + b[hr:rd] ** 2, atol=2e-2)   # each pair only turns
    assert np.array_equal(a[rd:], b[rd:])
    assert not np.array_equal(a[:rd], b[:rd])
    # scale invariance of the normalisation (power-of-two factor: exact)
    qc, _, _ = yko.attn_post(x * 4, x[:, :1], x[:, :1], zero_w, zero_w, 0.0, rope, rd, 7, 0)
    assert np.array_equal(qb, qc)


def test_post_with_rotation_equals_rotation_of_post():
    rng = np.random.default_rng(5)
    M, H, KVH, rd = 3, 24, 4, 32
    xq = rng.standard_normal((M, H, 128)).astype(np.float32)
    xk = rng.standard_normal((M, KVH, 128)).astype(np.float32)
    xv = rng.standard_normal((M, KVH, 128)).astype(np.float32)
    w = (rng.standard_normal(128) * 0.1).astype(np.float16).view(np.uint16)
    rope = yko.rope_table(16, rd)
    q0, k0, v0 = yko.attn_post(xq, xk, xv, w, w, 1e-6, rope, rd, 2, 0)
    q1, k1, v1 = yko.attn_post(xq, xk, xv, w, w, 1e-6, rope, rd, 2, 1)
    f = lambda u: u.view(np.float16).astype(np.float32).reshape(-1, 128)
    assert np.array_equal(q1.reshape(-1, 128), yko.rotate128(f(q0), False, 0.0625).astype(np.float16).view(np.uint16))
    assert np.array_equal(k1.reshape(-1, 128), yko.rotate128(f(k0), False, 0.125).astype(np.float16).view(np.uint16))
    xv16 = xv.astype(np.float16).astype(np.float32)                    # the projection is rounded on entry
    assert np.array_equal(v1.reshape(-1, 128), yko.rotate128(xv16.reshape(-1, 128), False, 0.125).astype(np.float16).view(np.uint16))
    # scores survive the rotation up to the fp16 rounding of the rotated rows
    s0 = (f(q0)[:24].astype(np.float64) * f(k0)[0]).sum(1)
    s1 = (f(q1)[:24].astype(np.float64) * f(k1)[0]).sum(1)
    assert np.abs(s0 - s1).max() < 0.05


def test_unrotate_out_inverts_v_rotation():
    rng = np.random.default_rng(6)
    v = rng.standard_normal((10, 128)).astype(np.float32)
    rv = yko.rotate128(v, False, 0.125)
    out = yko.unrotate_out(rv)
    assert np.abs(_h(out) - v).max() < 2e-3


# ---- the same step for 256-channel heads ----

def _post_numpy_d(y, w16, eps, cs, rd):
    return _post_numpy(y, w16, eps, cs, rd)       # the fp64 form does not depend on the row length


def test_post256_rows_match_fp64_forms_and_rotation():
    rng = np.random.default_rng(13)
    M, H, KVH, rd, pos = 3, 24, 4, 64, 21
    xq = (rng.standard_normal((M, H, 256)) * 3).astype(np.float32)
    xk = (rng.standard_normal((M, KVH, 256)) * 0.5).astype(np.float32)
    xv = rng.standard_normal((M, KVH, 256)).astype(np.float32)
    qw = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    kw = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    rope = yko.rope_table(32, rd)
    q16, k32, v32 = yko.attn_post256(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot=0)
    # the projected value is rounded to the 16-bit type before anything else (src/q35_kernels.cu:1030)
    r16 = lambda a: a.astype(np.float16).astype(np.float32)
    for t in range(M):
        cs = rope[pos + t].astype(np.float64)
        for h in range(H):
            ref = _post_numpy_d(r16(xq[t, h]), qw, 1e-6, cs, rd)
            assert np.abs(_h(q16[t, h]) - ref).max() <= 2.5e-3 * max(1.0, np.abs(ref).max())
        for h in range(KVH):
            ref = _post_numpy_d(r16(xk[t, h]), kw, 1e-6, cs, rd)
            assert np.abs(k32[t, h] - ref).max() <= 2.5e-3 * max(1.0, np.abs(ref).max())
    # K rows without rotation are fp16 valued; V rows are the rounded projection
    assert np.array_equal(k32, k32.astype(np.float16).astype(np.float32))
    assert np.array_equal(v32, r16(xv))
    # channels past rd carry no rotary change: one more rounding only
    ref = _post_numpy_d(r16(xq[0, 0]), qw, 1e-6, rope[pos].astype(np.float64), rd)
    assert np.abs(_h(q16[0, 0, rd:]) - ref[rd:]).max() <= 1.0e-3 * max(1.0, np.abs(ref).max())
    # with the rotation on: exactly the pinned 256-point rotation of the un-rotated rows (Q rounded to fp16 after it)
    q16r, k32r, v32r = yko.attn_post256(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot=1)
    qf = q16.view(np.float16).astype(np.float32).reshape(-1, 256)
    assert np.array_equal(q16r.reshape(-1, 256), yko.kvx_rotate256(qf).astype(np.float16).view(np.uint16))
    assert np.array_equal(k32r.reshape(-1, 256), yko.kvx_rotate256(k32.reshape(-1, 256)))
    assert np.array_equal(v32r.reshape(-1, 256), yko.kvx_rotate256(r16(xv).reshape(-1, 256)))


def test_post256_structure():
    rng = np.random.default_rng(14)
    rd = 64
    x = rng.standard_normal((1, 1, 256)).astype(np.float32)
    zero_w = np.zeros(256, np.uint16)
    rope = yko.rope_table(16, rd)
    q16, _, _ = yko.attn_post256(x, x[:, :1], x[:, :1], zero_w, zero_w, 0.0, rope, rd, 0, 0)
    assert abs(np.sqrt((_h(q16) ** 2).mean()) - 1.0) < 1e-3                 # unit RMS; position 0 turns nothing
    qb, _, _ = yko.attn_post256(x, x[:, :1], x[:, :1], zero_w, zero_w, 0.0, rope, rd, 7, 0)
    a, b = _h(q16)[0, 0], _h(qb)[0, 0]
    hr = rd // 2
    assert np.allclose(a[:hr] ** 2 + a[hr:rd] ** 2, b[:hr] ** 2 + b[hr:rd] ** 2, atol=2e-2)
    assert np.array_equal(a[rd:], b[rd:]) and not np.array_equal(a[:rd], b[:rd])
    qc, _, _ = yko.attn_post256(x * 4, x[:, :1], x[:, :1], zero_w, zero_w, 0.0, rope, rd, 7, 0)
    assert np.array_equal(qb, qc)                                            # power-of-two scale invariance: exact
    # the sum of squares is exact on small integers whatever the order (so the order of the reference, 32-channel runs
    # folded in sequence, src/q35_kernels.cu:1051-1056, cannot show here): r = 1 / sqrt(ss / 256)
    xi = rng.integers(-3, 4, size=(1, 1, 256)).astype(np.float32)
    qi, _, _ = yko.attn_post256(xi, xi[:, :1], xi[:, :1], zero_w, zero_w, 0.0, rope, 0, 0, 0)
    r = np.float32(1.0) / np.sqrt(np.float32((xi.astype(np.float64) ** 2).sum() / 256.0))
    assert np.array_equal(qi[0, 0], (xi[0, 0] * r).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("D", [128, 256])
def test_sum_of_squares_follows_the_reference_order(D):
    """ss = the sums of 32-channel runs (each a butterfly a[i] += a[i ^ o], o = 16 .. 1) folded in sequence from 0
    (src/q35_kernels.cu:1050-1056).  With one large square per run and tiny ones beside it the fp32 result depends on
    the association; the row's normalisation factor must be the one this order gives."""
    rng = np.random.default_rng(15 + D)
    zero_w = np.zeros(D, np.uint16)
    rope = np.zeros((1, 1, 2), np.float32)
    post = yko.attn_post256 if D == 256 else yko.attn_post
    for trial in range(20):
        x = (rng.standard_normal(D) * 10.0 ** rng.integers(-3, 3, size=D)).astype(np.float16).astype(np.float32)
        sq = (x * x).astype(np.float32)
        runs = []
        for w in range(D // 32):
            a = sq[32 * w:32 * w + 32].copy()
            for o in (16, 8, 4, 2, 1):
                a = (a + a[np.arange(32) ^ o]).astype(np.float32)
            runs.append(a[0])
        tot = np.float32(0.0)
        for r_ in runs:
            tot = np.float32(tot + r_)
        r = np.float32(1.0) / np.sqrt(np.float32(tot / np.float32(D)))
        q16, _, _ = post(x.reshape(1, 1, D), x.reshape(1, 1, D), x.reshape(1, 1, D), zero_w, zero_w, 0.0, rope, 0, 0, 0)
        expect = (x * r).astype(np.float32).astype(np.float16).view(np.uint16)
        assert np.array_equal(q16[0, 0], expect), trial
