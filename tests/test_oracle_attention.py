"""Pins the oracle's attention against an independent numpy float64 softmax(QK^T/sqrt(d))V and against closed forms.

Reference behaviour restated by the oracle: online softmax per split (src/attention_kv4q.cu:19-31,71-146), combiner
with empty-split sentinel (src/attention_kv4q.cu:325-332), row t of a window sees keys [0, pos+depth(t)+1)
(src/q35_atx.cu:110-118), appended rows are visible to the pass that appends them (src/engine35.cpp:911-930).
"""
import numpy as np
import pytest

from tests.tolerances import attn_errors


def _numpy_attention(cache, q16, pos, depth, oracle):
    """Textbook attention in float64 on tensors dequantized by numpy (not by the oracle's dequantizer)."""
    kvh, T = cache.kc.shape[0], cache.kc.shape[1]
    def deq(codes, scales):
        lo = (codes & 15).astype(np.int32) - 8
        hi = (codes >> 4).astype(np.int32) - 8
        q = np.stack([lo, hi], -1).reshape(kvh, T, 128)
        s = scales.view(np.float16).astype(np.float64)
        return q * np.repeat(s, 32, axis=-1)
    K, V = deq(cache.kc, cache.ks), deq(cache.vc, cache.vs)
    M, NH, D = q16.shape
    out = np.zeros((M, NH, D))
    for t in range(M):
        L = pos + (t if depth is None else int(depth[t])) + 1
        for h in range(NH):
            s = K[h // 6, :L] @ q16[t, h].astype(np.float64) / np.sqrt(D)
            p = np.exp(s - s.max())
            out[t, h] = (p[:, None] * V[h // 6, :L]).sum(0) / p.sum()
    return out


def _setup(oracle, seed, ctx, M, max_ctx=None):
    q, k, v, kn, vn, ch = oracle.make_inputs(seed, ctx, M)
    c = oracle.Cache(max_ctx or ((ctx + M + 255) // 256) * 256)
    if ctx:
        c.append(k, v, 0)
    c.append(kn, vn, ctx)
    return c, q


@pytest.mark.parametrize("ctx,M", [(0, 1), (1, 1), (37, 3), (300, 8), (1000, 1)])
def test_f64_and_f32_match_numpy(oracle, ctx, M):
    c, q = _setup(oracle, 100 + ctx, ctx, M)
    want = _numpy_attention(c, q, ctx, None, oracle)
    got64 = c.attend_f64(q, ctx)
    assert np.abs(got64 - want).max() < 1e-12
    o16, o32 = c.attend_f32(q, ctx, want_f32=True)
    ma, rl = attn_errors(o32, want)
    assert ma < 5e-6 and rl < 5e-6, (ma, rl)
    assert (o16.view(np.uint16) == o32.astype(np.float16).view(np.uint16)).all()   # output is the fp16 rounding of the fp32 result


def test_split_count_and_threads_do_not_matter(oracle):
    c, q = _setup(oracle, 7, 5000, 4)
    base, b32 = c.attend_f32(q, 5000, want_f32=True)
    for splits, threads in [(1, 1), (3, 1), (31, 4), (42, 8), (128, 2)]:
        _, o32 = c.attend_f32(q, 5000, splits=splits, threads=threads, want_f32=True)
        ma, rl = attn_errors(o32, b32)
        assert ma < 1e-5 and rl < 1e-5, (splits, ma, rl)   # fp32 accumulation order differs, nothing else
    # threads only change who computes a split, never the arithmetic
    a = c.attend_f32(q, 5000, splits=42, threads=1)
    b = c.attend_f32(q, 5000, splits=42, threads=8)
    assert (a.view(np.uint16) == b.view(np.uint16)).all()


def test_scalar_build_gives_the_same_bits(oracle):
    """The benchmark's second CPU baseline (the same sources without the vectoriser) computes the same values."""
    c, q = _setup(oracle, 9, 3000, 5)
    a, a32 = c.attend_f32(q, 3000, want_f32=True)
    b, b32 = c.attend_f32(q, 3000, want_f32=True, scalar_build=True)
    assert (a.view(np.uint16) == b.view(np.uint16)).all() and (a32.view(np.uint32) == b32.view(np.uint32)).all()


def test_reference_split_policy_switches_at_4096(oracle):
    # rows below 4096 keys use 31 splits, rows at or above use 42 (src/q35_atxpk.cu:404-409): a window that straddles must still be right
    c, q = _setup(oracle, 8, 4090, 16)
    want = c.attend_f64(q, 4090)
    _, o32 = c.attend_f32(q, 4090, want_f32=True)
    ma, rl = attn_errors(o32, want)
    assert ma < 5e-6 and rl < 5e-6


def test_window_equals_single_rows_bit_for_bit(oracle):
    # the reference demands an M-row pass == M one-row passes (src/kvx_probe.cu:425-436)
    c, q = _setup(oracle, 9, 700, 6)
    full = c.attend_f32(q, 700, splits=8)
    for t in range(6):
        one = c.attend_f32(q[t:t + 1], 700 + t, splits=8)
        # same keys, but a different split partition of them: equal within rounding, and equal bit for bit when unsplit
        ma, rl = attn_errors(one, full[t:t + 1])
        assert ma <= 2e-3 * 1e-2
    full1 = c.attend_f32(q, 700, splits=1)
    for t in range(6):
        one = c.attend_f32(q[t:t + 1], 700 + t, splits=1)
        assert (one.view(np.uint16) == full1[t:t + 1].view(np.uint16)).all()


def test_depth_table_overrides_causal_order(oracle):
    c, q = _setup(oracle, 10, 200, 5)
    depth = np.array([0, 1, 1, 2, 0], np.uint8)       # side candidates: rows 1,2 share depth 1 (src/q35_atx.cu:111)
    got = c.attend_f64(q, 200, depth)
    want = _numpy_attention(c, q, 200, depth, oracle)
    assert np.abs(got - want).max() < 1e-12
    o16, o32 = c.attend_f32(q, 200, depth, want_f32=True)
    assert attn_errors(o32, want)[1] < 5e-6
    plain = c.attend_f64(q, 200)
    assert np.abs(got[0] - plain[0]).max() == 0 and np.abs(got[4] - plain[0 + 0]).max() > 0   # row 4 sees 201 keys but has its own query


def test_uniform_v_returns_v(oracle):
    # every V row identical => output equals that row whatever the scores are
    c, q = _setup(oracle, 11, 500, 2)
    c.vc[:] = c.vc[:, :1]
    c.vs[:] = c.vs[:, :1]
    vrow = oracle.dequant_rows(c.vc[:, 0], c.vs[:, 0])            # [kvh, 128]
    o16, o32 = c.attend_f32(q, 500, want_f32=True)
    want = np.repeat(vrow, 6, axis=0)[None].repeat(2, 0)
    assert np.abs(o32 - want).max() < 1e-5 * np.abs(want).max()


def test_dominant_key_returns_its_v(oracle):
    # one key aligned with the query and 64x larger than the rest => softmax is a delta on it
    rng = np.random.default_rng(12)
    ctx = 300
    q = rng.standard_normal((1, 24, 128)).astype(np.float16)
    k = (rng.standard_normal((ctx + 1, 4, 128)) * 0.05).astype(np.float16)
    v = rng.standard_normal((ctx + 1, 4, 128)).astype(np.float16)
    k[123] = (q[0, ::6].astype(np.float32) * 8).astype(np.float16)   # key 123 of kv head h = 8 * query of head 6h
    c = oracle.Cache(512)
    c.append(k, v, 0)
    o16, o32 = c.attend_f32(q, ctx, want_f32=True)
    v123 = oracle.dequant_rows(c.vc[:, 123], c.vs[:, 123])
    for h in range(4):
        assert np.abs(o32[0, 6 * h] - v123[h]).max() < 1e-4


def test_combine_identity_and_empty_split_sentinel(oracle):
    rng = np.random.default_rng(13)
    S, rows, dim, n = 5, 3, 16, 40
    s = rng.standard_normal((rows, n)) * 3
    v = rng.standard_normal((n, dim))
    want = np.stack([(np.exp(s[r] - s[r].max())[:, None] * v).sum(0) / np.exp(s[r] - s[r].max()).sum() for r in range(rows)])
    pm = np.full((S, rows), -1e30, np.float32); pl = np.zeros((S, rows), np.float32); pacc = np.zeros((S, rows, dim), np.float32)
    bounds = [0, 7, 7, 20, 33, 40]                      # split 1 is empty and keeps the sentinel (m=-1e30, l=0)
    for sp in range(S):
        a, b = bounds[sp], bounds[sp + 1]
        if a == b:
            continue
        for r in range(rows):
            m = s[r, a:b].max(); p = np.exp(s[r, a:b] - m)
            pm[sp, r] = m; pl[sp, r] = p.sum(); pacc[sp, r] = (p[:, None] * v[a:b]).sum(0)
    y = oracle.combine(pm, pl, pacc)
    assert np.abs(y - want).max() < 1e-5


def test_appended_rows_are_visible_to_later_rows_of_the_same_window(oracle):
    c, q = _setup(oracle, 14, 64, 4)
    base = c.attend_f64(q, 64)
    # change the K/V appended at window row 1: rows 0 must not move, rows 1..3 must
    rng = np.random.default_rng(15)
    c.append(rng.standard_normal((1, 4, 128)).astype(np.float16), rng.standard_normal((1, 4, 128)).astype(np.float16), 65)
    again = c.attend_f64(q, 64)
    assert np.abs(again[0] - base[0]).max() == 0
    for t in (1, 2, 3):
        assert np.abs(again[t] - base[t]).max() > 0


def test_generator_is_counter_based_and_has_the_stated_distribution(oracle):
    ch = oracle.outlier_channels(42)
    assert len(set(ch.tolist())) == 4 and ch.min() >= 0 and ch.max() < 128
    a = oracle.fill_normal_f16(5, 64, 128, ch, 8.0)
    b = oracle.fill_normal_f16(5, 32, 128, ch, 8.0, first=32 * 128)
    assert (a[32:].view(np.uint16) == b.view(np.uint16)).all()      # value i does not depend on how the stream is cut
    big = oracle.fill_normal_f16(6, 4096, 128, ch, 8.0).astype(np.float32)
    rest = np.delete(big, ch, axis=1)
    assert abs(rest.mean()) < 0.01 and abs(rest.std() - 1.0) < 0.01
    assert abs(big[:, ch].std() - 8.0) < 0.15
