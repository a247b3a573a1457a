"""Full-size configurations of the measurement contract, checked through size-independent properties and sampled rows.

Config 1/2: 32768 cached tokens, decode and a 64-row verify window, against the threaded oracle.
Config 3: a 2048-row prefill chunk on 131072 cached tokens: sampled rows against single-row oracle calls.
Config 4: 262144 cached tokens in 256-token pages shuffled by a seeded permutation: bit-identical to the contiguous
layout for decode and verify-64, and decode against the oracle.
"""
import numpy as np
import pytest

from tests.tolerances import assert_attn_close

pytestmark = pytest.mark.gpu


def _inputs(oracle, seed, ctx, M):
    ch = oracle.outlier_channels(seed)
    q = oracle.fill_normal_f16(seed + 1, M * 24).reshape(M, 24, 128)
    k = oracle.fill_normal_f16(seed + 2, (ctx + M) * 4, 128, ch, 8.0).reshape(ctx + M, 4, 128)
    v = oracle.fill_normal_f16(seed + 3, (ctx + M) * 4).reshape(ctx + M, 4, 128)
    return q, k, v


def _fill(kv, k, v, ctx, chunk=8192):
    for p in range(0, ctx, chunk):
        n = min(chunk, ctx - p)
        kv.append_host(0, k[p:p + n], v[p:p + n], p)


def _planes_match_the_oracle_quantizer(oracle, oc, k, v, spans):
    """The cache the GPU built (exported into oc) is what the oracle's own quantizer gives for the same fp16 rows: all four
    planes, bit for bit, over each (first row, count) span."""
    for lo, n in spans:
        chk = oracle.Cache(((n + 255) // 256) * 256)
        chk.append(k[lo:lo + n], v[lo:lo + n], 0)
        for name, plane_chk, plane_gpu in (("K codes", chk.kc, oc.kc), ("K scales", chk.ks, oc.ks), ("V codes", chk.vc, oc.vc), ("V scales", chk.vs, oc.vs)):
            assert (plane_chk[:, :n] == plane_gpu[:, lo:lo + n]).all(), f"{name} differ in rows {lo}..{lo + n - 1}"


def _oracle_cache(oracle, kv, n, max_ctx):
    oc = oracle.Cache(max_ctx)
    oc.kc[:, :n], oc.ks[:, :n], oc.vc[:, :n], oc.vs[:, :n] = kv.export_rows(0, 0, n)
    return oc


@pytest.mark.parametrize("M", [1, 16, 32, 64])
def test_config_1_2_decode_and_verify_at_32k(native, oracle, M):
    ctx = 32768
    q, k, v = _inputs(oracle, 900 + M, ctx, M)
    with native.KvCache(max_ctx=33024) as kv:
        _fill(kv, k, v, ctx)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)
        oc = _oracle_cache(oracle, kv, ctx + M, 33024)
        # the cache the GPU built is what the oracle's quantizer gives: all four planes of the first 2048 rows, of the last
        # 2048 cached rows and of the rows this call appended
        _planes_match_the_oracle_quantizer(oracle, oc, k, v, ((0, 2048), (ctx - 2048, 2048 + M)))
        ref16, ref32 = oc.attend_f32(q, ctx, threads=16, want_f32=True)
        assert_attn_close(out, ref32, f"32k M={M}")
        assert np.abs(out.astype(np.float64) - ref32).max() <= 2e-3   # at the measured size the plain absolute bar holds against the unrounded result too


def test_config_3_prefill_chunk_2048_on_131072(native, oracle):
    ctx, M = 131072, 2048
    q, k, v = _inputs(oracle, 930, ctx, M)
    max_ctx = ctx + M
    with native.KvCache(max_ctx=max_ctx, max_rows=2048) as kv:
        _fill(kv, k, v, ctx)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)      # quantizes the chunk into the cache
        oc = _oracle_cache(oracle, kv, ctx + M, max_ctx)
        # the rows the chunk appended (all 2048) and 2048 cached rows from the middle of the context, against the oracle's
        # own quantizer
        _planes_match_the_oracle_quantizer(oracle, oc, k, v, ((ctx, M), (65536 - 1024, 2048)))
        # every 16th row of the chunk plus the first and the last row of every 64-row group: the rows of one group are one
        # oracle call (a window at position ctx + 64 g whose depth table names the sampled rows)
        for g in range(M // 64):
            sel = np.array([0, 16, 32, 48, 63], dtype=np.uint8)
            rows = 64 * g + sel.astype(np.int64)
            ref32 = oc.attend_f32(q[rows], ctx + 64 * g, depth=sel, threads=16, want_f32=True)[1]
            assert_attn_close(out[rows], ref32, f"prefill rows {rows.tolist()}")
        # causality: changing the K/V of chunk row 1000 must leave rows < 1000 untouched
        k2, v2 = k[ctx:].copy(), v[ctx:].copy()
        k2[1000] = -k2[1000]; v2[1000] = -v2[1000]
        out2 = kv.layer_call(0, q, k2, v2, ctx)
        assert (out2[:1000].view(np.uint16) == out[:1000].view(np.uint16)).all()
        assert (out2[1000:].view(np.uint16) != out[1000:].view(np.uint16)).any()


def test_config_4_paged_262144(native, oracle):
    ctx = 262144
    q, k, v = _inputs(oracle, 940, ctx, 64)
    max_ctx = ctx + 256
    rng = np.random.default_rng(940)
    outs = {}
    for paged in (False, True):
        with native.KvCache(max_ctx=max_ctx, paged=paged) as kv:
            if paged:
                kv.set_page_table(rng.permutation(max_ctx // 256).astype(np.int32))
            _fill(kv, k, v, ctx, chunk=16384)
            outs[paged, 1] = kv.layer_call(0, q[:1], k[ctx:ctx + 1], v[ctx:ctx + 1], ctx)
            outs[paged, 64] = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)
            if paged:
                oc = _oracle_cache(oracle, kv, ctx + 64, max_ctx)
                # the rows the window appended and 2048 cached rows that straddle pages, read back through the page table
                _planes_match_the_oracle_quantizer(oracle, oc, k, v, ((ctx, 64), (131072 - 1000, 2048)))
    for M in (1, 64):
        assert (outs[False, M].view(np.uint16) == outs[True, M].view(np.uint16)).all(), f"paged != contiguous at M={M}"
    ref32 = oc.attend_f32(q[:1], ctx, threads=16, want_f32=True)[1]
    # after the 64-row call row ctx holds K/V of window row 0 = the decode call's new row, so the decode reference is valid
    assert_attn_close(outs[True, 1], ref32, "262144 decode")
    ref64 = oc.attend_f32(q[60:64], ctx + 60, depth=np.arange(4, dtype=np.uint8), threads=16, want_f32=True)[1]
    assert_attn_close(outs[True, 64][60:64], ref64, "262144 verify rows 60..63")
    # rows from all four 16-row quarters of the window (one oracle call: a window at ctx whose depth table names them)
    sel = np.array([0, 21, 42, 63], dtype=np.uint8)
    ref_sel = oc.attend_f32(q[sel.astype(np.int64)], ctx, depth=sel, threads=16, want_f32=True)[1]
    assert_attn_close(outs[True, 64][sel.astype(np.int64)], ref_sel, "262144 verify rows 0, 21, 42, 63")
