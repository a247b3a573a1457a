"""Pins the oracle's attention over the reference's own rows (head_dim 256, flat int4, one fp32 scale per row, MSB-first
words) against numpy on independently decoded tensors and against the invariants of split-KV attention.  CPU only."""
import numpy as np
import pytest

from oracle import yko

NH, KVH, D = 24, 4, 256


def _inputs(seed, ctx, M):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((M, NH, D)).astype(np.float16)
    k = rng.standard_normal((ctx + M, KVH, D)).astype(np.float32)
    k[:, :, [5, 77, 130, 201]] *= 8
    v = rng.standard_normal((ctx + M, KVH, D)).astype(np.float16)
    return q, k.astype(np.float16), v


def _decode_numpy(words, scales):
    """[..., 32] u32 words + [...] f32 scales -> [..., 256] f64, via numpy bit unpacking of the big-endian byte image"""
    b = np.ascontiguousarray(words.astype(">u4")).view(np.uint8)
    bits = np.unpackbits(b, axis=-1).reshape(words.shape[:-1] + (256, 4))
    nib = (bits * np.array([8, 4, 2, 1])).sum(-1).astype(np.int64)
    # the decoded value is the fp32 product (src/kvq_attn.cuh:54, __fmul_rn): with an fp32 scale it is rounded
    return ((nib - 8).astype(np.float32) * scales[..., None].astype(np.float32)).astype(np.float64)


def _cache(q, k, v, ctx):
    c = yko.Cache(ctx + 64, NH, KVH, D)
    c.append(k, v, 0)
    return c


def test_append_is_the_reference_row_encoder_on_the_widened_inputs():
    q, k, v = _inputs(1, 40, 3)
    c = _cache(q, k, v, 43)
    n = k.shape[0]
    for h in range(KVH):
        w, s, _ = yko.flat4_encode256(k[:, h].astype(np.float32))
        assert np.array_equal(c.kc[h, :n], w) and np.array_equal(c.ks[h, :n], s)
        w, s, _ = yko.flat4_encode256(v[:, h].astype(np.float32))
        assert np.array_equal(c.vc[h, :n], w) and np.array_equal(c.vs[h, :n], s)


@pytest.mark.parametrize("ctx,M", [(1, 1), (37, 1), (200, 5)])
def test_f64_attention_matches_numpy_softmax(ctx, M):
    q, k, v = _inputs(2 + ctx, ctx, M)
    c = _cache(q, k, v, ctx)
    out = c.attend_f64(q, ctx)
    kd = _decode_numpy(c.kc, c.ks); vd = _decode_numpy(c.vc, c.vs)
    qf = q.astype(np.float64)
    for t in range(M):
        n = ctx + t + 1
        for h in range(NH):
            s = kd[h // 6, :n] @ qf[t, h] / 16.0
            p = np.exp(s - s.max()); p /= p.sum()
            assert np.abs(out[t, h] - p @ vd[h // 6, :n]).max() < 1e-12


def test_f32_streaming_attention_close_to_f64_and_split_independent():
    ctx, M = 700, 4
    q, k, v = _inputs(9, ctx, M)
    c = _cache(q, k, v, ctx)
    ref = c.attend_f64(q, ctx)
    _, o1 = c.attend_f32(q, ctx, splits=1, want_f32=True)
    _, o42 = c.attend_f32(q, ctx, splits=0, want_f32=True)
    _, o7 = c.attend_f32(q, ctx, splits=7, threads=4, want_f32=True)
    for o in (o1, o42, o7):
        assert np.abs(o - ref).max() < 1e-5
    # a window equals its rows taken one at a time (bit for bit when unsplit)
    for t in range(M):
        dep = np.array([t], np.uint8)
        _, single = c.attend_f32(q[t:t + 1], ctx, depth=dep, splits=1, want_f32=True)
        assert np.array_equal(single[0], o1[t])


def test_closed_forms():
    ctx = 64
    q, k, v = _inputs(11, ctx, 1)
    v[:] = v[0:1]                                           # every V row the same -> output = that (decoded) row
    c = _cache(q, k, v, ctx)
    out = c.attend_f64(q, ctx)
    vd = _decode_numpy(c.vc, c.vs)
    for h in range(NH):
        assert np.abs(out[0, h] - vd[h // 6, 0]).max() < 1e-12
    # one dominant key
    q2, k2, v2 = _inputs(12, ctx, 1)
    k2[:] = 0
    k2[17, :, :] = (q2[0, ::6, :].astype(np.float32) * 4).astype(np.float16)      # aligned with head 0 of each group
    c2 = _cache(q2, k2, v2, ctx)
    out2 = c2.attend_f64(q2, ctx)
    vd2 = _decode_numpy(c2.vc, c2.vs)
    assert np.abs(out2[0, 0] - vd2[0, 17]).max() < 1e-6
