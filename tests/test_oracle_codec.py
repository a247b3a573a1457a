"""Pins the oracle's codec against what the mathematics fixes (the reference holds no vectors for this path).

Reference arithmetic restated by the oracle: src/kvq_fast.cuh:194-198 (am/7, zero guard, rintf, clamp, +8),
decode src/kvq_attn.cuh:52-54, nibble order src/post_kernels.cu:77-80.
"""
import numpy as np
import pytest


def _np_quant_group(x16):
    """Independent restatement in numpy: float32 arithmetic with numpy's IEEE division and rint."""
    x = x16.astype(np.float32)
    am = np.float32(np.abs(x).max())
    s16 = np.float16(am / np.float32(7.0))
    if s16 == 0:
        s16 = np.float16(1.0)
    sd = np.float32(s16)
    q = np.clip(np.rint(x / sd), -7, 7).astype(np.int32)
    return q, s16


def test_h2f_matches_numpy_on_every_bit_pattern(oracle):
    got = oracle.h2f_all()
    want = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    ok = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert ok.all()


def test_f2h_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    vals = [np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)]        # every fp16 value
    h = vals[0][np.isfinite(vals[0])]
    nxt = np.nextafter(h, np.float32(np.inf)).astype(np.float32)
    vals.append(((h.astype(np.float64) + nxt.astype(np.float64)) / 2).astype(np.float32))  # near-midpoints
    hs = np.sort(h)
    mid = ((hs[:-1].astype(np.float64) + hs[1:].astype(np.float64)) / 2).astype(np.float32)  # exact ties between fp16 neighbours
    vals += [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))]
    vals.append(rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32))
    vals.append(np.array([65504, 65519.99, 65520, 65536, 1e30, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -26, 0.0, -0.0], np.float32))
    x = np.concatenate(vals)
    x = x[~np.isnan(x)]
    got = oracle.f2h(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert (got == want).all(), f"{(got != want).sum()} mismatches"


def test_pack_unpack_all_bytes_and_nibble_order(oracle):
    fields = np.array([[lo, hi] for hi in range(16) for lo in range(16)], np.uint8).ravel()
    packed = oracle.pack_nibbles(fields)
    assert (packed == np.arange(256, dtype=np.uint8)).all()        # byte = even field | odd field << 4
    assert (oracle.unpack_nibbles(packed) == fields).all()


def test_zero_group_gives_scale_one_and_zero_codes(oracle):
    codes, scales = oracle.quant_rows(np.zeros((1, 128), np.float16))
    assert (scales.view(np.float16) == 1.0).all()
    assert (codes == 0x88).all()                                    # q = 0 stored as 8 in both nibbles
    assert (oracle.dequant_rows(codes, scales) == 0).all()


def test_max_element_encodes_to_plus_minus_7_and_clamp_is_live(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((4000, 128)) * 3).astype(np.float16)
    codes, scales = oracle.quant_rows(x)
    q = oracle.unpack_nibbles(codes.ravel()).reshape(-1, 4, 32).astype(np.int32) - 8
    xa = np.abs(x.astype(np.float32)).reshape(-1, 4, 32)
    arg = xa.argmax(-1)
    qmax = np.take_along_axis(q, arg[..., None], -1)[..., 0]
    assert (np.abs(qmax) == 7).all()
    assert q.min() >= -7 and q.max() <= 7
    # the stored scale is fp16(am/7); when it was rounded down, am/scale exceeds 7 and only the clamp keeps |q| <= 7
    am = xa.max(-1)
    sd = scales.view(np.float16).astype(np.float32).reshape(-1, 4)
    assert (am / sd > 7.0).any()


def test_ties_round_to_even(oracle):
    # scale exactly 1 (max = 7): x = k + 0.5 must go to the even neighbour
    x = np.zeros((1, 128), np.float16)
    x[0, 0] = 7.0
    x[0, 1:8] = [0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5]
    codes, scales = oracle.quant_rows(x)
    assert scales.view(np.float16)[0, 0] == 1.0
    q = oracle.unpack_nibbles(codes.ravel()).astype(np.int32)[:8] - 8
    assert q.tolist() == [7, 0, 2, 2, 4, 0, -2, -2]


def test_single_value_groups_over_every_finite_fp16(oracle):
    # group = (v, 0, 0, ...): scale = fp16(|v|/7) (1 if that is 0); code of v = clamp(rint(v/scale))
    bits = np.arange(65536, dtype=np.uint16)
    v = bits.view(np.float16)
    fin = np.isfinite(v)
    x = np.zeros((fin.sum(), 32), np.float16)
    x[:, 0] = v[fin]
    codes, scales = oracle.quant_rows(x.reshape(-1, 128)) if (fin.sum() % 4 == 0) else oracle.quant_rows(x, dim=32)
    codes = codes.reshape(-1, 16); scales = scales.reshape(-1)
    q0 = (codes[:, 0] & 15).astype(np.int32) - 8
    vf = v[fin].astype(np.float32)
    with np.errstate(over="ignore"):
        s16 = (np.abs(vf) / np.float32(7)).astype(np.float16)
    s16 = np.where(s16 == 0, np.float16(1), s16)
    assert (scales.view(np.float16) == s16).all()
    want = np.clip(np.rint(vf / s16.astype(np.float32)), -7, 7).astype(np.int32)
    assert (q0 == want).all()
    assert ((codes[:, 1:] == 0x88).all()) and ((codes[:, 0] >> 4) == 8).all()


def test_random_groups_against_independent_numpy(oracle):
    rng = np.random.default_rng(3)
    scale = np.float32(10.0) ** rng.uniform(-6, 3.5, (3000, 1)).astype(np.float32)
    x = (rng.standard_normal((3000, 32)).astype(np.float32) * scale).astype(np.float16)
    x[::7, 5] *= np.float16(8)
    codes, scales = oracle.quant_rows(x, dim=32)
    q = oracle.unpack_nibbles(codes.ravel()).reshape(-1, 32).astype(np.int32) - 8
    for r in range(x.shape[0]):
        qr, sr = _np_quant_group(x[r])
        assert scales[r, 0] == sr.view(np.uint16), r
        assert (q[r] == qr).all(), r


def test_dequant_is_exact_product_for_all_codes_and_scales(oracle):
    sc = np.arange(65536, dtype=np.uint16)
    sc = sc[np.isfinite(sc.view(np.float16))]
    for code in range(1, 16):
        codes = np.full((sc.size, 16), code | (code << 4), np.uint8)
        y = oracle.dequant_rows(codes, sc.reshape(-1, 1), dim=32)
        want = (np.float64(code - 8) * sc.view(np.float16).astype(np.float64)).astype(np.float32)   # exact in double, then exact in float
        assert (y[:, 0].view(np.uint32) == want.view(np.uint32)).all()
        assert (y == y[:, :1]).all()


def test_requantizing_dequantized_values_is_idempotent(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2000, 128)).astype(np.float16)
    codes, scales = oracle.quant_rows(x)
    y = oracle.dequant_rows(codes, scales)
    y16 = y.astype(np.float16)
    exact = (y16.astype(np.float32) == y).reshape(-1, 4, 32).all(-1)     # groups whose decoded values are fp16-representable
    c2, s2 = oracle.quant_rows(y16)
    same_s = (s2 == scales)
    same_c = (c2.reshape(-1, 4, 16) == codes.reshape(-1, 4, 16)).all(-1)
    assert exact.sum() > 100
    assert (same_s & same_c)[exact].all()


def test_append_places_rows_and_overwrites(oracle):
    rng = np.random.default_rng(5)
    c = oracle.Cache(256)
    k = rng.standard_normal((5, 4, 128)).astype(np.float16)
    v = rng.standard_normal((5, 4, 128)).astype(np.float16)
    c.append(k, v, 10)
    codes, scales = oracle.quant_rows(k.reshape(-1, 128))
    assert (c.kc[:, 10:15] == codes.reshape(5, 4, 64).transpose(1, 0, 2)).all()
    assert (c.ks[:, 10:15] == scales.reshape(5, 4, 4).transpose(1, 0, 2)).all()
    assert (c.kc[:, :10] == 0).all() and (c.kc[:, 15:] == 0).all()
    c.append(v[:2], k[:2], 12)                                         # rejected rows are simply overwritten
    codes2, _ = oracle.quant_rows(v[:2].reshape(-1, 128))
    assert (c.kc[:, 12:14] == codes2.reshape(2, 4, 64).transpose(1, 0, 2)).all()
    assert (c.kc[:, 14] == codes.reshape(5, 4, 64)[4]).all()
