"""The reference's own rows on the GPU (head_dim 256, flat int4, one fp32 scale per row, MSB-first words) against the
oracle: appended words and scales bit-exact, attention outputs within the attention bars."""
import numpy as np
import pytest

from tolerances import assert_attn_close

pytestmark = pytest.mark.gpu
NH, KVH, D = 24, 4, 256


def _inputs(seed, ctx, M):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((M, NH, D)).astype(np.float16)
    k = rng.standard_normal((ctx + M, KVH, D)).astype(np.float32)
    k[:, :, [5, 77, 130, 201]] *= 8                       # outlier channels
    v = rng.standard_normal((ctx + M, KVH, D)).astype(np.float16)
    return q, k.astype(np.float16), v


def _fill(kv, ref, k, v, ctx):
    for p in range(0, ctx, 64):
        n = min(64, ctx - p)
        kv.append_host(0, k[p:p + n], v[p:p + n], p)
    if ctx:
        ref.append(k[:ctx], v[:ctx], 0)


@pytest.mark.parametrize("paged", [False, True])
def test_append_bit_exact_and_image_round_trip(native, oracle, paged):
    ctx = 300
    q, k, v = _inputs(1, ctx, 4)
    k[7] = 0; v[7] = 0                                    # zero rows: scale 1, every field 8
    k[9, :, 1:] = 0                                       # one non-zero element per row
    ref = oracle.Cache(512, NH, KVH, D)
    with native.KvCache(n_layers=2, head_dim=D, max_ctx=512, paged=paged) as kv:
        if paged:
            kv.set_page_table(np.array([1, 0], np.int32))
        _fill(kv, ref, k, v, ctx)
        kw, ks, vw, vs = kv.export_rows(0, 0, ctx)
        assert np.array_equal(kw, ref.kc[:, :ctx]) and np.array_equal(vw, ref.vc[:, :ctx])
        assert np.array_equal(ks.view(np.uint32), ref.ks[:, :ctx].view(np.uint32))
        assert np.array_equal(vs.view(np.uint32), ref.vs[:, :ctx].view(np.uint32))
        assert np.all(kw[:, 7] == 0x88888888) and np.all(ks[:, 7] == 1.0)
        kv.import_rows(1, 100, kw[:, :50], ks[:, :50], vw[:, :50], vs[:, :50])
        back = kv.export_rows(1, 100, 50)
        for a, b in zip(back, (kw[:, :50], ks[:, :50], vw[:, :50], vs[:, :50])):
            assert np.array_equal(a, b)


@pytest.mark.parametrize("ctx,M", [(0, 1), (0, 5), (31, 1), (32, 2), (257, 3), (1000, 1), (1000, 16), (4096, 1), (2500, 64)])
def test_attention_matches_oracle(native, oracle, ctx, M):
    q, k, v = _inputs(10 + ctx + M, ctx, M)
    max_ctx = ((ctx + M + 255) // 256) * 256
    ref = oracle.Cache(max_ctx, NH, KVH, D)
    with native.KvCache(head_dim=D, max_ctx=max_ctx) as kv:
        _fill(kv, ref, k, v, ctx)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)
        got = kv.export_rows(0, ctx, M)
    ref.append(k[ctx:], v[ctx:], ctx)
    # rows stored by the pass itself (inside the attention launch: by the workgroups whose key range holds them): bit-exact
    assert np.array_equal(got[0], ref.kc[:, ctx:ctx + M]) and np.array_equal(got[2], ref.vc[:, ctx:ctx + M])
    assert np.array_equal(got[1].view(np.uint32), ref.ks[:, ctx:ctx + M].view(np.uint32))
    assert np.array_equal(got[3].view(np.uint32), ref.vs[:, ctx:ctx + M].view(np.uint32))
    assert_attn_close(out, ref.attend_f32(q, ctx, threads=8), f"ctx={ctx} M={M}")


def test_depth_table_splits_and_pages(native, oracle):
    ctx, M = 700, 6
    q, k, v = _inputs(77, ctx, M)
    depth = np.array([0, 1, 1, 2, 2, 3], np.uint8)
    ref = oracle.Cache(1024, NH, KVH, D)
    outs = []
    for paged in (False, True):
        with native.KvCache(head_dim=D, max_ctx=1024, paged=paged) as kv:
            if paged:
                kv.set_page_table(np.array([2, 0, 3, 1], np.int32))
            _fill(kv, ref if not paged else oracle.Cache(1024, NH, KVH, D), k, v, ctx)
            outs.append(kv.layer_call(0, q, k[ctx:], v[ctx:], ctx, depth=depth))
            if not paged:
                kv.set_opt(1, 3)
                few = kv.layer_call(0, q, None, None, ctx, depth=depth)
                kv.set_opt(1, 97)
                many = kv.layer_call(0, q, None, None, ctx, depth=depth)
                kv.set_opt(1, 200)                                            # more than 128: the combiner's widest form
                most = kv.layer_call(0, q, None, None, ctx, depth=depth)
    ref.append(k[ctx:], v[ctx:], ctx)
    expect = ref.attend_f32(q, ctx, depth=depth)
    assert_attn_close(outs[0], expect, "depth table")
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))      # paged == contiguous, bit for bit
    assert_attn_close(few, expect, "3 splits"); assert_attn_close(many, expect, "97 splits"); assert_attn_close(most, expect, "200 splits")


@pytest.mark.parametrize("ctx", [31, 1023])
def test_rows_no_query_row_sees_are_still_stored(native, oracle, ctx):
    """Sibling rows (depth table [0, 0]) whose second row opens a new 32-key tile: stored although no key range holds it."""
    M = 2
    q, k, v = _inputs(90 + ctx, ctx, M)
    depth = np.array([0, 0], np.uint8)
    ref = oracle.Cache(1280, NH, KVH, D)
    with native.KvCache(head_dim=D, max_ctx=1280) as kv:
        _fill(kv, ref, k, v, ctx)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx, depth=depth)
        got = kv.export_rows(0, ctx, M)
    ref.append(k[ctx:], v[ctx:], ctx)
    assert np.array_equal(got[0], ref.kc[:, ctx:ctx + M]) and np.array_equal(got[2], ref.vc[:, ctx:ctx + M])
    assert np.array_equal(got[1].view(np.uint32), ref.ks[:, ctx:ctx + M].view(np.uint32))
    assert np.array_equal(got[3].view(np.uint32), ref.vs[:, ctx:ctx + M].view(np.uint32))
    assert_attn_close(out, ref.attend_f32(q, ctx, depth=depth), f"siblings at ctx={ctx}")


def _rows_bit_exact(got, ref, ctx, M, what):
    assert np.array_equal(got[0], ref.kc[:, ctx:ctx + M]) and np.array_equal(got[2], ref.vc[:, ctx:ctx + M]), what
    assert np.array_equal(got[1].view(np.uint32), ref.ks[:, ctx:ctx + M].view(np.uint32)), what
    assert np.array_equal(got[3].view(np.uint32), ref.vs[:, ctx:ctx + M].view(np.uint32)), what


WINDOW_CASES = {
    # a 64-row window that starts at an odd row of page 1 and ends in page 2 (rows of one wave lie in two pages)
    "across a page, odd start": (2 * 256 - 21, 64, None),
    # two row blocks
    "two row blocks": (777, 40, None),
    # siblings: no query row sees rows 1024..1028, which open a new tile past every key range
    "unseen rows past the last tile": (1023, 6, [0] * 6),
    # three row blocks, none of which sees past row 1000: rows 1024..1063 lie past the last tile of all of them
    "64 siblings": (1000, 64, [0] * 64),
    # the first row block reads further than the last one
    "deep first block, shallow last": (900, 64, [63] * 32 + [0] * 32),
}


@pytest.mark.parametrize("paged", [False, True])
@pytest.mark.parametrize("case", list(WINDOW_CASES))
def test_windows_store_their_own_rows(native, oracle, case, paged):
    """Passes of 3..64 rows quantize and store their rows inside the attention launch: every row bit-exact in the cache
    afterwards, whichever workgroup held its tile, and the outputs as if the rows had been there before."""
    ctx, M, dp = WINDOW_CASES[case]
    depth = None if dp is None else np.array(dp, np.uint8)
    q, k, v = _inputs(300 + ctx + M, ctx, M)
    ref = oracle.Cache(1280, NH, KVH, D)
    with native.KvCache(head_dim=D, max_ctx=1280, paged=paged) as kv:
        if paged:
            kv.set_page_table(np.array([3, 0, 4, 1, 2], np.int32))
        _fill(kv, ref, k, v, ctx)
        before = kv.export_rows(0, 0, ctx)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx, depth=depth)
        got = kv.export_rows(0, ctx, M)
        after = kv.export_rows(0, 0, ctx)
    for a, b in zip(before, after):                       # nothing else was written
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), case
    ref.append(k[ctx:], v[ctx:], ctx)
    _rows_bit_exact(got, ref, ctx, M, case)
    assert_attn_close(out, ref.attend_f32(q, ctx, depth=depth, threads=8), case)


def test_seeded_sweep_of_windows(native, oracle):
    """40 seeded cases: context lengths around tile and page boundaries, 1..64 rows, a random depth table (row t sees up
    to t rows of the pass) or none, paged or contiguous: stored rows bit-exact, outputs within the attention bars."""
    rng = np.random.default_rng(4256)
    for case in range(40):
        ctx = int(rng.choice([0, 1, 31, 32, 33, 255, 256, 257, 511, int(rng.integers(0, 2200)), int(rng.integers(0, 2200))]))
        M = int(rng.choice([1, 2, 3, 5, 16, 21, 22, 23, 43, 64, int(rng.integers(1, 65))]))
        depth = None
        if rng.random() < 0.5:
            depth = np.array([int(rng.integers(0, t + 1)) for t in range(M)], np.uint8)
        paged = bool(rng.random() < 0.5)
        max_ctx = ((ctx + M + 255) // 256 + int(rng.integers(0, 2))) * 256
        what = f"case {case}: ctx={ctx} M={M} depth={'yes' if depth is not None else 'no'} paged={paged} max_ctx={max_ctx}"
        print(what, flush=True)
        q, k, v = _inputs(5000 + case, ctx, M)
        ref = oracle.Cache(max_ctx, NH, KVH, D)
        with native.KvCache(head_dim=D, max_ctx=max_ctx, paged=paged) as kv:
            if paged:
                kv.set_page_table(rng.permutation(max_ctx // 256).astype(np.int32))
            _fill(kv, ref, k, v, ctx)
            out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx, depth=depth)
            got = kv.export_rows(0, ctx, M)
        ref.append(k[ctx:], v[ctx:], ctx)
        _rows_bit_exact(got, ref, ctx, M, what)
        assert_attn_close(out, ref.attend_f32(q, ctx, depth=depth, threads=8), what)


def test_entry_points_of_the_other_format_refuse(native):
    with native.KvCache(head_dim=D, max_ctx=256) as kv:
        with pytest.raises(native.YkaError, match="128"):
            kv.dequant_rows(0, 0, 1)
    with native.KvCache(max_ctx=256) as kv:
        with pytest.raises(native.YkaError, match="256"):
            native._chk(native.lib().yka_kv_export_rows256(kv._h, 0, 0, 1, None, None, None, None))


def test_rotated_rows_and_unrotated_outputs(native, oracle):
    """fp32 rows -> signed Hadamard rotation -> flat int4 rows (the reference's kvx_rotate + row quantizer), rotated Q rows,
    attention, outputs rotated back."""
    ctx, M = 500, 5
    rng = np.random.default_rng(2024)
    k32 = rng.standard_normal((ctx + M, KVH, D)).astype(np.float32)
    k32[:, :, [5, 77, 130, 201]] *= 8
    v32 = rng.standard_normal((ctx + M, KVH, D)).astype(np.float32)
    q32 = rng.standard_normal((M, NH, D)).astype(np.float32)
    n = ctx + M
    ref = oracle.Cache(768, NH, KVH, D)
    for h in range(KVH):
        ref.kc[h, :n], ref.ks[h, :n], _ = oracle.flat4_encode256(oracle.kvx_rotate256(k32[:, h]))
        ref.vc[h, :n], ref.vs[h, :n], _ = oracle.flat4_encode256(oracle.kvx_rotate256(v32[:, h]))
    qrot = oracle.kvx_rotate256(q32.reshape(-1, D)).astype(np.float16).reshape(M, NH, D)
    got_q = native.rotate_q256(q32)
    assert np.array_equal(got_q.view(np.uint16), qrot.view(np.uint16))
    with native.KvCache(head_dim=D, max_ctx=768) as kv:
        for p in range(0, n, 64):
            m = min(64, n - p)
            kv.append256_f32_host(0, k32[p:p + m], v32[p:p + m], p, rotate=True)
        kw, ks, vw, vs = kv.export_rows(0, 0, n)
        assert np.array_equal(kw, ref.kc[:, :n]) and np.array_equal(vw, ref.vc[:, :n])
        assert np.array_equal(ks.view(np.uint32), ref.ks[:, :n].view(np.uint32)) and np.array_equal(vs.view(np.uint32), ref.vs[:, :n].view(np.uint32))
        kv.set_opt(4, 1)
        out = kv.layer_call(0, got_q, None, None, ctx)
        kv.set_opt(4, 0)
        raw = kv.layer_call(0, got_q, None, None, ctx)
    _, o32 = ref.attend_f32(qrot, ctx, want_f32=True)
    expect = oracle.kvx_rotate256(o32.reshape(-1, D), inverse=True).astype(np.float16).reshape(M, NH, D)
    assert_attn_close(out, expect, "un-rotated outputs")
    assert_attn_close(raw, o32, "outputs left in the rotated basis")
    # the whole pipeline approximates plain attention on the unrotated fp32 data (int4 noise only); a wrong factor or a
    # missing sign in either rotation would show as an error of order 1
    worst = 0.0
    for t in range(M):
        for h in (0, 7, 23):
            s = k32[:ctx + t + 1, h // 6].astype(np.float64) @ q32[t, h].astype(np.float64) / 16.0
            p = np.exp(s - s.max()); p /= p.sum()
            plain = p @ v32[:ctx + t + 1, h // 6].astype(np.float64)
            worst = max(worst, np.linalg.norm(out[t, h].astype(np.float64) - plain) / np.linalg.norm(plain))
    assert worst < 0.35, worst


def test_output_step_gate_hadamard_int8(native, oracle):
    rng = np.random.default_rng(31)
    M, H = 7, 24
    y = rng.standard_normal((M, H, D)).astype(np.float16)
    gate = (rng.standard_normal((M, H, D)) * 3).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), size=H * D)
    y[2, 6:8] = 0                                          # a zero group: scale 0, codes 0
    y[3] = np.round(y[3].astype(np.float32) * 2); gate[3] = 60.0   # integers with the gate open: every operation exact
    qx, alpha = native.attn_out256(y, gate, signs)
    rq, ra = oracle.attn_out256(y, gate, signs)
    assert np.array_equal(qx[3], rq[3]) and np.array_equal(alpha[3].view(np.uint32), ra[3].view(np.uint32))
    assert alpha[2, 3] == 0 and not qx[2, 1536:2048].any()
    # elsewhere the only operation that may differ between device and host is expf inside the sigmoid, whose result is
    # rounded to fp16 right away: scales agree to fp16 resolution, codes differ by at most one step and almost never
    assert np.allclose(alpha, ra, rtol=2e-3, atol=0)
    diff = np.abs(qx.astype(np.int32) - rq.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01, (diff.max(), (diff != 0).mean())


@pytest.mark.parametrize("M", [1, 5, 8])
def test_output_step_interleaved_small_batch_layout(native, M):
    """The reference's interleaved layout for passes of at most 8 tokens (a8_lo_off, src/a8_prologue.cuh:121): the same
    codes as the plain layout, element i of token t of group g at g*4096 + (i/256)*2048 + ((i/16)%4)*512 + t*64 +
    ((i/64)%4)*16 + i%16; positions of tokens that are not part of the pass stay untouched (zero in the host form)."""
    rng = np.random.default_rng(41 + M)
    H = 24
    y = rng.standard_normal((M, H, D)).astype(np.float16)
    gate = (rng.standard_normal((M, H, D)) * 3).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), size=H * D)
    qx, alpha = native.attn_out256(y, gate, signs)
    lo, alpha_lo = native.attn_out256_lo(y, gate, signs)
    assert np.array_equal(alpha.view(np.uint32), alpha_lo.view(np.uint32))
    # the index map, spelled from its bit fields: i = (b8, b76, b54, b3210) -> (b8, b54, t, b76, b3210)
    i = np.arange(512)
    place = ((i >> 8) << 11) | (((i >> 4) & 3) << 9) | (((i >> 6) & 3) << 4) | (i & 15)
    assert len(set(place.tolist())) == 512 and (place & (7 << 6)).max() == 0        # one-to-one, and it leaves the token field free
    seen = np.zeros((H // 2, 4096), bool)
    for t in range(M):
        for g in range(H // 2):
            assert np.array_equal(lo[g, place | (t << 6)], qx[t, g * 512:(g + 1) * 512]), (t, g)
            seen[g, place | (t << 6)] = True
    assert not lo[~seen].any()
    with pytest.raises(native.YkaError, match="1 to 8 tokens"):
        native.attn_out256_lo(np.zeros((9, H, D), np.float16), np.zeros((9, H, D), np.float16), signs)


@pytest.mark.parametrize("M", [1, 16, 64])
def test_full_length_32768(native, oracle, M):
    """32,768 cached tokens (4,096 distinct rows tiled over the context): decode, and windows on the 128-row workgroups,
    against the threaded oracle on the cache image the GPU built"""
    ctx, U = 32768, 4096
    rng = np.random.default_rng(3300 + M)
    k = rng.standard_normal((U + M, KVH, D)).astype(np.float32); k[:, :, [5, 77, 130, 201]] *= 8
    k = k.astype(np.float16)
    v = rng.standard_normal((U + M, KVH, D)).astype(np.float16)
    q = rng.standard_normal((M, NH, D)).astype(np.float16)
    ref = oracle.Cache(ctx + 256, NH, KVH, D)
    with native.KvCache(head_dim=D, max_ctx=ctx + 256) as kv:
        for p in range(0, ctx, 64):
            s0 = p % U
            kv.append_host(0, k[s0:s0 + 64], v[s0:s0 + 64], p)
        out = kv.layer_call(0, q, k[U:], v[U:], ctx)
        kw, ks, vw, vs = kv.export_rows(0, 0, ctx + M)
    ref.kc[:, :ctx + M], ref.ks[:, :ctx + M], ref.vc[:, :ctx + M], ref.vs[:, :ctx + M] = kw, ks, vw, vs
    chk = oracle.Cache(256, NH, KVH, D)                    # the image is what the oracle's quantizer gives (first rows)
    chk.append(k[:200], v[:200], 0)
    assert np.array_equal(chk.kc[:, :200], kw[:, :200]) and np.array_equal(chk.vs[:, :200].view(np.uint32), vs[:, :200].view(np.uint32))
    expect = ref.attend_f32(q, ctx, threads=16, want_f32=True)[1]
    assert_attn_close(out, expect, f"32k M={M}")
    assert np.abs(out.astype(np.float64) - expect).max() <= 2e-3
