"""The step between the QKV projection and the cache on the GPU (RMS normalisation, rotary embedding, optional signed
Hadamard rotation, fused quantize-on-append) against the oracle: Q rows and the stored codes / scales bit-exact,
attention over the rotated cache with un-rotated outputs within the attention bars."""
import numpy as np
import pytest

from tolerances import assert_attn_close, attn_errors

pytestmark = pytest.mark.gpu


def _inputs(seed, M, scale_k=0.7):
    rng = np.random.default_rng(seed)
    xq = (rng.standard_normal((M, 24, 128)) * 2.0).astype(np.float32)
    xk = (rng.standard_normal((M, 4, 128)) * scale_k).astype(np.float32)
    xk[:, :, [3, 40, 77, 120]] *= 8.0                      # outlier channels, as in the measured inputs
    xv = rng.standard_normal((M, 4, 128)).astype(np.float32)
    qw = (rng.standard_normal(128) * 0.1).astype(np.float16)
    kw = (rng.standard_normal(128) * 0.1).astype(np.float16)
    return xq, xk, xv, qw, kw


@pytest.mark.parametrize("paged", [False, True])
@pytest.mark.parametrize("rot", [0, 1])
@pytest.mark.parametrize("rd", [0, 32, 128])
def test_post_rows_bit_exact(native, oracle, paged, rot, rd):
    M, pos, ctx = 13, 250, 512                             # the rows straddle a 256-token page
    xq, xk, xv, qw, kw = _inputs(10 + rd + rot, M)
    xq[2] = 0.0; xk[2] = 0.0; xv[2] = 0.0                  # an all-zero token: eps keeps the norm finite, scales become 1
    rope = oracle.rope_table(ctx, rd) if rd else None
    rq, rk, rv = oracle.attn_post(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot)
    ref = oracle.Cache(ctx)
    ref.append(rk, rv, pos)
    with native.KvCache(max_ctx=ctx, paged=paged) as kv:
        if paged:
            kv.set_page_table(np.array([1, 0], np.int32))
        q16 = kv.attn_post_host(0, xq, xk, xv, pos, qw, kw, 1e-6, rope, rd, rotate=bool(rot))
        kc, ks, vc, vs = kv.export_rows(0, pos, M)
    assert np.array_equal(q16.view(np.uint16), rq)
    assert np.array_equal(ks, ref.ks[:, pos:pos + M]) and np.array_equal(vs, ref.vs[:, pos:pos + M])
    assert np.array_equal(kc, ref.kc[:, pos:pos + M]) and np.array_equal(vc, ref.vc[:, pos:pos + M])


def test_post_equals_append_of_the_fp16_rows(native, oracle):
    # the fused kernel must store exactly what yka_append stores for the fp16 rows the unfused path would have written
    M, pos, ctx, rd = 64, 0, 256, 32
    xq, xk, xv, qw, kw = _inputs(77, M)
    rope = oracle.rope_table(ctx, rd)
    _, rk, rv = oracle.attn_post(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, 1)
    with native.KvCache(n_layers=2, max_ctx=ctx) as kv:
        kv.attn_post_host(0, xq, xk, xv, pos, qw, kw, 1e-6, rope, rd, rotate=True)
        kv.append_host(1, rk, rv, pos)
        a = kv.export_rows(0, pos, M); b = kv.export_rows(1, pos, M)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("M", [1, 16])
def test_attention_over_rotated_cache(native, oracle, M):
    ctx_fill, ctx, rd = 700, 1024, 32
    xq, xk, xv, qw, kw = _inputs(5, ctx_fill + M)
    rope = oracle.rope_table(ctx, rd)
    outs = {}
    for rot in (0, 1):
        rq, rk, rv = oracle.attn_post(xq, xk, xv, qw, kw, 1e-6, rope, rd, 0, rot)
        ref = oracle.Cache(ctx)
        ref.append(rk, rv, 0)
        r16, r32 = ref.attend_f32(rq[ctx_fill:], ctx_fill, want_f32=True)
        expect = oracle.unrotate_out(r32).view(np.float16) if rot else r16
        with native.KvCache(max_ctx=ctx) as kv:
            kv.set_opt(4, rot)
            for t0 in range(0, ctx_fill + M, 64):
                n = min(64, ctx_fill + M - t0)
                q16 = kv.attn_post_host(0, xq[t0:t0 + n], xk[t0:t0 + n], xv[t0:t0 + n], t0, qw, kw, 1e-6, rope, rd, rotate=bool(rot))
                assert np.array_equal(q16.view(np.uint16), rq[t0:t0 + n])
            out = kv.layer_call(0, rq[ctx_fill:].view(np.float16), None, None, ctx_fill)
        assert_attn_close(out, expect, f"rot={rot} M={M}")
        outs[rot] = out.astype(np.float64)
    # the rotation changes which values get quantized, not what is computed: both pipelines agree up to int4 noise.
    # A wrong inverse factor (x2, x1/2) or a missing sign would show as an error of order 1.
    _, rl = attn_errors(outs[1], outs[0])
    assert 0.0 < rl < 0.25, rl


def test_post_rejects_bad_arguments(native, oracle):
    xq, xk, xv, qw, kw = _inputs(1, 2)
    with native.KvCache(max_ctx=256) as kv:
        with pytest.raises(native.YkaError):
            kv.attn_post_host(0, xq, xk, xv, 255, qw, kw, 1e-6, None, 0)          # rows past the container
        with pytest.raises(native.YkaError):
            kv.attn_post_host(0, xq, xk, xv, 0, qw, kw, 1e-6, oracle.rope_table(1, 32), 32)   # table shorter than pos + M
        with pytest.raises(native.YkaError):
            kv.attn_post_host(0, xq, xk, xv, 0, qw, kw, 1e-6, oracle.rope_table(8, 6)[:, :1], 3)   # odd rope_dims


# ---- the same step for 256-channel heads (handles opened with head_dim = 256) ----

def _inputs256(seed, M):
    rng = np.random.default_rng(seed)
    xq = (rng.standard_normal((M, 24, 256)) * 2.0).astype(np.float32)
    xk = (rng.standard_normal((M, 4, 256)) * 0.7).astype(np.float32)
    xk[:, :, [5, 77, 130, 201]] *= 8.0
    xv = rng.standard_normal((M, 4, 256)).astype(np.float32)
    qw = (rng.standard_normal(256) * 0.1).astype(np.float16)
    kw = (rng.standard_normal(256) * 0.1).astype(np.float16)
    return xq, xk, xv, qw, kw


@pytest.mark.parametrize("paged", [False, True])
@pytest.mark.parametrize("rot", [0, 1])
@pytest.mark.parametrize("rd", [0, 64, 256])
def test_post256_rows_bit_exact(native, oracle, paged, rot, rd):
    M, pos, ctx = 11, 250, 512                             # the rows straddle a 256-token page
    xq, xk, xv, qw, kw = _inputs256(40 + rd + rot, M)
    xq[2] = 0.0; xk[2] = 0.0; xv[2] = 0.0                  # an all-zero token: eps keeps the norm finite, scales become 1
    rope = oracle.rope_table(ctx, rd) if rd else None
    rq, rk32, rv32 = oracle.attn_post256(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot)
    with native.KvCache(head_dim=256, max_ctx=ctx, paged=paged) as kv:
        if paged:
            kv.set_page_table(np.array([1, 0], np.int32))
        q16 = kv.attn_post_host(0, xq, xk, xv, pos, qw, kw, 1e-6, rope, rd, rotate=bool(rot))
        kw_, ks_, vw_, vs_ = kv.export_rows(0, pos, M)
    assert np.array_equal(q16.view(np.uint16), rq)
    for h in range(4):
        words, scale, _ = oracle.flat4_encode256(rk32[:, h])
        assert np.array_equal(kw_[h], words) and np.array_equal(ks_[h].view(np.uint32), scale.view(np.uint32))
        words, scale, _ = oracle.flat4_encode256(rv32[:, h])
        assert np.array_equal(vw_[h], words) and np.array_equal(vs_[h].view(np.uint32), scale.view(np.uint32))


def test_attention_over_rows_the_post256_step_stored(native, oracle):
    # projection rows -> post step with rotation -> cache; Q rows of the pass attend to them; outputs rotated back
    ctx, M, rd = 300, 4, 64
    xq, xk, xv, qw, kw = _inputs256(50, ctx + M)
    rope = oracle.rope_table(512, rd)
    ref = oracle.Cache(512, 24, 4, 256)
    with native.KvCache(head_dim=256, max_ctx=512, max_rows=64) as kv:
        qs = []
        for p in range(0, ctx + M, 64):
            m = min(64, ctx + M - p)
            qs.append(kv.attn_post_host(0, xq[p:p + m], xk[p:p + m], xv[p:p + m], p, qw, kw, 1e-6, rope, rd, rotate=True))
            _, rk32, rv32 = oracle.attn_post256(xq[p:p + m], xk[p:p + m], xv[p:p + m], qw, kw, 1e-6, rope, rd, p, 1)
            for h in range(4):
                ref.kc[h, p:p + m], ref.ks[h, p:p + m], _ = oracle.flat4_encode256(rk32[:, h])
                ref.vc[h, p:p + m], ref.vs[h, p:p + m], _ = oracle.flat4_encode256(rv32[:, h])
        q16 = np.concatenate(qs)[ctx:]
        kv.set_opt(4, 1)
        out = kv.layer_call(0, q16, None, None, ctx)
    _, o32 = ref.attend_f32(q16, ctx, want_f32=True)
    expect = oracle.kvx_rotate256(o32.reshape(-1, 256), inverse=True).astype(np.float16).reshape(M, 24, 256)
    assert_attn_close(out, expect, "attention over post256 rows, outputs un-rotated")
