"""Pins the oracle's restatement of the reference's 256-channel row codec (rotation, flat int4 with MSB-first packing,
int8 rows) against independent implementations and the closed forms the arithmetic fixes.  CPU only."""
import numpy as np
import pytest
from scipy.linalg import hadamard

from oracle import yko


def _sign_ref(d):
    # src/kvx_codec.cuh:28-32 with Python integers and explicit 32-bit wrap
    x = (d + 1) & 0xFFFFFFFF
    x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return -1.0 if (x & 1) else 1.0


def test_sign_hash_matches_big_integer_evaluation():
    s = yko.kvx_signs()
    ref = np.array([_sign_ref(d) for d in range(256)], np.float32)
    assert np.array_equal(s, ref)
    assert 96 < int((s < 0).sum()) < 160          # a hash, not a constant


def test_rotation_is_signed_sylvester_hadamard_exact_on_integers():
    # integer inputs keep every butterfly sum exact in fp32, so the result must EQUAL the matrix form; a swapped
    # subtraction, a wrong stage order or a missing sign changes it
    rng = np.random.default_rng(1)
    x = rng.integers(-8, 9, size=(16, 256)).astype(np.float32)
    H = hadamard(256).astype(np.float64)
    s = yko.kvx_signs().astype(np.float64)
    fwd = (H @ (x.astype(np.float64) * s).T).T / 16.0
    assert np.array_equal(yko.kvx_rotate256(x), fwd.astype(np.float32))
    inv = (H @ x.astype(np.float64).T).T / 16.0 * s
    assert np.array_equal(yko.kvx_rotate256(x, inverse=True), inv.astype(np.float32))


def test_rotation_involution_and_norm():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((32, 256)).astype(np.float32)
    y = yko.kvx_rotate256(x)
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-5)
    back = yko.kvx_rotate256(y, inverse=True)
    assert np.abs(back - x).max() < 1e-5
    # one-hot in: a signed row of the matrix out
    e = np.zeros((1, 256), np.float32); e[0, 5] = 1.0
    row = yko.kvx_rotate256(e)[0]
    assert np.array_equal(np.abs(row), np.full(256, 0.0625, np.float32))
    assert np.array_equal(row, (hadamard(256)[:, 5] * _sign_ref(5) * 0.0625).astype(np.float32))


def _flat4_numpy(r):
    r = r.astype(np.float32)
    am = np.abs(r).max(axis=1).astype(np.float32)
    s7 = (am / np.float32(7.0)).astype(np.float32)
    s7[s7 == 0] = 1.0
    q = np.clip(np.rint((r / s7[:, None]).astype(np.float32)), -7, 7)
    fields = (q + 8).astype(np.uint8)
    bits = ((fields[:, :, None] >> np.array([3, 2, 1, 0], np.uint8)) & 1).reshape(r.shape[0], 1024)
    words = np.packbits(bits, axis=1).view(">u4").astype(np.uint32)
    return words, s7, (q.astype(np.float32) * s7[:, None]).astype(np.float32), fields


def test_flat4_closed_forms():
    z = np.zeros((1, 256), np.float32)
    w, s, xq = yko.flat4_encode256(z)
    assert s[0] == 1.0 and np.all(w == 0x88888888) and np.all(xq == 0)
    x = np.zeros((1, 256), np.float32); x[0, 0] = -3.5; x[0, 9] = 1.0
    w, s, xq = yko.flat4_encode256(x)
    assert s[0] == np.float32(3.5) / np.float32(7)
    assert (w[0, 0] >> 28) == 1                         # field of element 0 = -7 + 8, top nibble of word 0
    assert ((w[0, 1] >> 24) & 15) == 10                 # element 9 = second nibble of word 1: rint(1/0.5) = 2 -> 10
    # ties go to even: s7 = 1 (max 7), values k + 0.5
    t = np.zeros((1, 256), np.float32); t[0, 0] = 7.0; t[0, 1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    w, s, xq = yko.flat4_encode256(t)
    assert s[0] == 1.0 and list(xq[0, 1:7]) == [0.0, 2.0, 2.0, -0.0, -2.0, -2.0]


def test_flat4_matches_numpy_restatement_and_packbits():
    rng = np.random.default_rng(3)
    r = (rng.standard_normal((64, 256)) * rng.uniform(1e-3, 50, size=(64, 1))).astype(np.float32)
    r[5] *= 0
    w, s, xq = yko.flat4_encode256(r)
    w2, s2, xq2, fields = _flat4_numpy(r)
    assert np.array_equal(s, s2) and np.array_equal(w, w2) and np.array_equal(xq, xq2)
    assert fields.min() >= 1 and fields.max() <= 15
    y = yko.flat4_decode256(w, s)
    assert np.array_equal(y, xq)                        # decode reproduces the encoder's reconstruction bit for bit
    # every non-zero row reaches +-7
    nz = np.abs(r).max(axis=1) > 0
    assert np.all(np.abs(fields[nz].astype(int) - 8).max(axis=1) == 7)


def test_int8_rows():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((32, 256)).astype(np.float32)
    x[3] = 0
    q, s = yko.int8_encode256(x)
    am = np.abs(x).max(axis=1).astype(np.float32)
    s2 = (am / np.float32(127)).astype(np.float32)
    assert np.array_equal(s, s2)
    with np.errstate(divide="ignore", invalid="ignore"):
        q2 = np.where(s2[:, None] > 0, np.rint((x / s2[:, None]).astype(np.float32)), 0)
    assert np.array_equal(q, np.clip(q2, -127, 127).astype(np.int8))
    assert s[3] == 0 and np.all(q[3] == 0)
    assert np.all(np.abs(q[s > 0]).max(axis=1) == 127)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("rot", [0, 1])
def test_probe_round_trip_error(mode, rot):
    rng = np.random.default_rng(5 + mode * 2 + rot)
    x = rng.standard_normal((16, 256)).astype(np.float32)
    q8, words, scales, y = yko.kvx_probe256(x, mode, rot)
    rel = np.linalg.norm(y - x) / np.linalg.norm(x)
    assert rel < (0.012 if mode == 0 else 0.16)         # 8-bit vs 4-bit uniform quantization of Gaussian rows
    if mode == 1 and not rot:
        w, s, xq = yko.flat4_encode256(x)
        assert np.array_equal(words, w) and np.array_equal(scales, s) and np.array_equal(y, xq)


# ---- the step after attention: sigmoid gate, signs, 512-point Hadamard transform, int8 groups of 512 ----

def test_attn_out_transform_is_sylvester_512_exact_on_integers():
    from scipy.linalg import hadamard as had
    rng = np.random.default_rng(21)
    M, H = 2, 24
    y = rng.integers(-4, 5, size=(M, H, 256)).astype(np.float16)
    gate = np.full((M, H, 256), 60.0, np.float16)          # sigmoid(60) rounds to 1: the gate is open
    signs = rng.choice(np.array([-1, 1], np.int8), size=H * 256)
    qx, alpha = yko.attn_out256(y, gate, signs)
    u = (y.astype(np.float64).reshape(M, -1) * signs).reshape(M, -1, 512)
    v = (u @ had(512).astype(np.float64)) * np.float32(0.044194173824159216)
    v = v.astype(np.float32).astype(np.float16).astype(np.float32)      # integer sums are exact; one fp32 product, one fp16 rounding
    al = (np.abs(v).max(-1) / np.float32(127)).astype(np.float32)
    assert np.array_equal(alpha, al)
    q = np.clip(np.rint((v / al[..., None]).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(qx, q.reshape(M, -1))
    assert np.all(np.abs(qx.reshape(M, -1, 512)).max(-1) == 127)


def test_attn_out_gate_and_zero_group():
    rng = np.random.default_rng(22)
    M, H = 3, 24
    y = rng.standard_normal((M, H, 256)).astype(np.float16)
    gate = (rng.standard_normal((M, H, 256)) * 3).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), size=H * 256)
    y[1, 4:6] = 0                                          # one whole group of 512 is zero: alpha 0, codes 0
    qx, alpha = yko.attn_out256(y, gate, signs)
    assert alpha[1, 2] == 0 and np.all(qx[1, 1024:1536] == 0)
    from scipy.linalg import hadamard as had
    sg = 1.0 / (1.0 + np.exp(-gate.astype(np.float64)))
    u = (y.astype(np.float64) * sg).reshape(M, -1) * signs
    v = (u.reshape(M, -1, 512) @ had(512).astype(np.float64)) / np.sqrt(512.0)
    deq = qx.reshape(M, -1, 512).astype(np.float64) * alpha[..., None]
    # three fp16 roundings and an 8-bit grid: 127 levels over the group's range
    err = np.abs(deq - v).max(-1)
    assert np.all(err <= np.abs(v).max(-1) * (0.5 / 127 + 4e-3) + 1e-6)
    # the transform is orthonormal: the energy of a group survives up to the quantization error
    assert np.allclose(np.linalg.norm(deq, axis=-1), np.linalg.norm(u.reshape(M, -1, 512), axis=-1), rtol=0.02, atol=1e-6)
