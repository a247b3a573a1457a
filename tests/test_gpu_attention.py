"""GPU attention through the C ABI vs the oracle: max-abs 2e-3 and relative L2 1e-3 (tests/tolerances.py)."""
import numpy as np
import pytest

from tests.tolerances import assert_attn_close, attn_errors

pytestmark = pytest.mark.gpu


def _fill(native, oracle, seed, ctx, M, max_ctx=None, **kw):
    """Cache with `ctx` rows quantized by the oracle and imported, plus seeded q and new k/v for an M-row window."""
    q, k, v, kn, vn, ch = oracle.make_inputs(seed, ctx, M)
    max_ctx = max_ctx or ((ctx + M + 255) // 256) * 256
    oc = oracle.Cache(max_ctx)
    kv = native.KvCache(max_ctx=max_ctx, **kw)
    if ctx:
        oc.append(k, v, 0)
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
    return kv, oc, q, kn, vn


@pytest.mark.parametrize("ctx", [0, 1, 31, 32, 33, 255, 256, 1000, 4096])
def test_decode_matches_oracle(native, oracle, ctx):
    kv, oc, q, kn, vn = _fill(native, oracle, 300 + ctx, ctx, 1)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        ref16, ref32 = oc.attend_f32(q, ctx, want_f32=True)
        assert_attn_close(out, ref32, f"decode ctx={ctx} vs fp32")
        assert_attn_close(out, ref16, f"decode ctx={ctx} vs fp16")


@pytest.mark.parametrize("M", [2, 3, 7, 16, 33, 64])
def test_window_matches_oracle(native, oracle, M):
    ctx = 1500
    kv, oc, q, kn, vn = _fill(native, oracle, 400 + M, ctx, M)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        ref16, ref32 = oc.attend_f32(q, ctx, threads=8, want_f32=True)
        assert_attn_close(out, ref32, f"window M={M}")
        # appended rows are in the cache, bit-exact
        got = kv.export_rows(0, ctx, M)
        assert (got[0] == oc.kc[:, ctx:ctx + M]).all() and (got[1] == oc.ks[:, ctx:ctx + M]).all()
        assert (got[2] == oc.vc[:, ctx:ctx + M]).all() and (got[3] == oc.vs[:, ctx:ctx + M]).all()


def test_window_equals_single_row_calls(native, oracle):
    # reference invariant (src/kvx_probe.cu:425-436): an M-row pass equals M one-row passes
    ctx, M = 900, 9
    kv, oc, q, kn, vn = _fill(native, oracle, 500, ctx, M)
    with kv:
        full = kv.layer_call(0, q, kn, vn, ctx)
        for t in range(M):
            one = kv.layer_call(0, q[t:t + 1], None, None, ctx + t)
            ma, rl = attn_errors(one, full[t:t + 1])
            assert ma <= 2e-3 and rl <= 1e-3, (t, ma, rl)


def test_split_count_does_not_matter(native, oracle):
    ctx = 3000
    kv, oc, q, kn, vn = _fill(native, oracle, 501, ctx, 2)
    with kv:
        oc.append(kn, vn, ctx)
        ref = oc.attend_f32(q, ctx, want_f32=True)[1]
        outs = []
        for S in (1, 2, 7, 32, 128):
            kv.set_opt(1, S)
            outs.append(kv.layer_call(0, q, kn, vn, ctx))
            assert_attn_close(outs[-1], ref, f"splits={S}")


@pytest.mark.parametrize("M,ctx,S", [(1, 3000, 0), (2, 3000, 0), (1, 70, 0), (2, 40000, 0), (1, 40000, 200), (2, 9000, 1)])
def test_merge_inside_the_launch_equals_second_launch(native, oracle, M, ctx, S):
    """With option key 7 the decode kernel merges its splits in the workgroup that finishes last (tickets); by default the
    merge is the combiner launch.  Both are checked against the oracle, against each other (same partials, different summation
    order: a few fp16 spacings at most), and the one-launch form over repeated calls (the tickets return to zero)."""
    q, k, v, kn, vn, ch = oracle.make_inputs(520 + M, ctx, M)
    oc = oracle.Cache(ctx + 64); oc.append(k, v, 0); oc.append(kn, vn, ctx)
    ref = oc.attend_f32(q, ctx, want_f32=True)[1]
    with native.KvCache(max_ctx=((ctx + 64 + 255) // 256) * 256) as kv:
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
        if S:
            kv.set_opt(1, S)
        two = kv.layer_call(0, q, kn, vn, ctx)
        assert_attn_close(two, ref, "two launches")
        kv.set_opt(7, 1)
        for rep in range(4):
            one = kv.layer_call(0, q, kn, vn, ctx)
            assert_attn_close(one, ref, f"one launch, call {rep}")
            assert np.abs(one.astype(np.float64) - two.astype(np.float64)).max() <= 2e-3
            if rep:
                assert (one.view(np.uint16) == first.view(np.uint16)).all(), rep
            first = one


@pytest.mark.parametrize("M,S", [(3, 1), (22, 5), (43, 7), (64, 21), (64, 32), (33, 13), (150, 3)])
def test_wide_grid_layout_reaches_every_row_block_and_split(native, oracle, M, S):
    """The wide kernel's one-dimensional grid is laid out for the round robin over the XCDs: whole (split, kv head) pairs
    per XCD first, the leftover workgroups in order.  Split counts that leave leftovers (pairs x row blocks not a multiple
    of 8) and counts that do not must both cover every (pair, row block) exactly once: any hole or double shows in the
    output of the rows it belongs to."""
    ctx = 2600
    kv, oc, q, kn, vn = _fill(native, oracle, 530 + M + S, ctx, M, max_rows=max(M, 64))
    with kv:
        kv.set_opt(2, S)
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"M={M} splits={S}")


def test_depth_table(native, oracle):
    ctx, M = 700, 6
    kv, oc, q, kn, vn = _fill(native, oracle, 502, ctx, M)
    depth = np.array([0, 1, 1, 2, 2, 3], np.uint8)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx, depth=depth)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, depth, want_f32=True)[1], "depth table")


def test_paged_layout_is_bit_identical_to_contiguous(native, oracle):
    ctx, M = 2000, 5
    q, k, v, kn, vn, ch = oracle.make_inputs(503, ctx, M)
    oc = oracle.Cache(2304); oc.append(k, v, 0)
    rng = np.random.default_rng(503)
    outs = []
    for paged in (False, True):
        with native.KvCache(max_ctx=2304, paged=paged) as kv:
            if paged:
                kv.set_page_table(rng.permutation(9).astype(np.int32))
            kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
            outs.append(kv.layer_call(0, q, kn, vn, ctx))
    assert (outs[0].view(np.uint16) == outs[1].view(np.uint16)).all()
    oc.append(kn, vn, ctx)
    assert_attn_close(outs[1], oc.attend_f32(q, ctx, want_f32=True)[1], "paged")


def test_uniform_v_and_dominant_key(native, oracle):
    ctx = 1200
    kv, oc, q, kn, vn = _fill(native, oracle, 504, ctx, 1)
    with kv:
        vc = np.repeat(oc.vc[:, :1], ctx, axis=1); vs = np.repeat(oc.vs[:, :1], ctx, axis=1)
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], vc, vs)
        out = kv.layer_call(0, q, None, None, ctx - 1).astype(np.float32)
        vrow = np.repeat(oracle.dequant_rows(oc.vc[:, 0], oc.vs[:, 0]), 6, axis=0)
        assert np.abs(out[0] - vrow).max() <= 2e-3 * max(1.0, np.abs(vrow).max())


def test_multi_layer_containers_are_independent(native, oracle):
    ctx = 400
    q, k, v, kn, vn, ch = oracle.make_inputs(505, ctx, 1)
    q2, k2, v2, kn2, vn2, _ = oracle.make_inputs(506, ctx, 1)
    with native.KvCache(n_layers=3, max_ctx=512) as kv:
        oa, ob = oracle.Cache(512), oracle.Cache(512)
        oa.append(k, v, 0); ob.append(k2, v2, 0)
        kv.import_rows(0, 0, oa.kc[:, :ctx], oa.ks[:, :ctx], oa.vc[:, :ctx], oa.vs[:, :ctx])
        kv.import_rows(2, 0, ob.kc[:, :ctx], ob.ks[:, :ctx], ob.vc[:, :ctx], ob.vs[:, :ctx])
        o0 = kv.layer_call(0, q, kn, vn, ctx); o2 = kv.layer_call(2, q, kn, vn, ctx)
        oa.append(kn, vn, ctx); ob.append(kn, vn, ctx)
        assert_attn_close(o0, oa.attend_f32(q, ctx, want_f32=True)[1], "layer 0")
        assert_attn_close(o2, ob.attend_f32(q, ctx, want_f32=True)[1], "layer 2")
        kv.replicate_layer(0)
        o2b = kv.layer_call(2, q, None, None, ctx)
        assert (o2b.view(np.uint16) == o0.view(np.uint16)).all()


@pytest.mark.parametrize("M", [65, 66])
def test_tail_slice_of_one_or_two_rows(native, oracle, M):
    # a pass of 65 or 66 rows is a prefill chunk: one append launch for all its rows, then one slice (up to 1024 tokens)
    # on the wide kernel whose last 128-row workgroup holds only the 6 or 12 rows beyond row 384
    ctx = 700
    kv, oc, q, kn, vn = _fill(native, oracle, 600 + M, ctx, M, max_rows=128)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"{M}-row pass")
        got = kv.export_rows(0, ctx, M)
        for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
            assert (a == b[:, ctx:ctx + M]).all()


def test_wide_pass_is_cut_into_slices(native, oracle):
    # the reference cuts passes wider than 64 rows into 64-row slices (src/engine35.cpp:935-947); here such a pass is a
    # prefill chunk: its rows are appended by one launch, then slices of up to 1024 tokens run on the wide kernel
    ctx, M = 300, 150
    kv, oc, q, kn, vn = _fill(native, oracle, 507, ctx, M, max_rows=256)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], "150-row pass")
        # the rows the append launch stored, bit-exact
        got = kv.export_rows(0, ctx, M)
        for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
            assert (a == b[:, ctx:ctx + M]).all()


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("merge_in_launch", [0, 1])
def test_decode_waves_with_many_few_and_no_tiles_in_one_launch(native, oracle, M, merge_in_launch):
    """8 splits over 73 tiles: splits 0..6 hold 10 tiles each (waves 0 and 1 take three tiles - the double-buffered loop -,
    waves 2 and 3 two - the branch without a loop), split 7 holds 3 (waves 0..2 one tile, wave 3 none): every way a wave of
    the decode kernel waits for its query rows runs in the same launch."""
    ctx = 73 * 32 - 20 - (M - 1)
    kv, oc, q, kn, vn = _fill(native, oracle, 650 + M, ctx, M)
    with kv:
        kv.set_opt(1, 8)
        kv.set_opt(7, merge_in_launch)
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"8 splits over 73 tiles, M={M}")
        got = kv.export_rows(0, ctx, M)
        for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
            assert (a == b[:, ctx:ctx + M]).all()


def test_errors_are_reported_not_thrown(native):
    with native.KvCache(max_ctx=256, max_rows=4) as kv:
        q = np.zeros((5, 24, 128), np.float16)
        with pytest.raises(native.YkaError, match="max_rows"):
            kv.layer_call(0, q, None, None, 0)
        with pytest.raises(native.YkaError, match="layer"):
            kv.layer_call(3, q[:1], None, None, 0)
        with pytest.raises(native.YkaError, match="max_ctx"):
            kv.layer_call(0, q[:4], None, None, 254)
        with pytest.raises(native.YkaError, match="contiguous"):
            kv.set_page_table(np.zeros(1, np.int32))
    with native.KvCache(max_ctx=512, paged=True) as kv:
        with pytest.raises(native.YkaError, match="permutation"):
            kv.set_page_table(np.array([0, 0], np.int32))


def test_bench_hook_runs_and_agrees_with_single_call(native, oracle):
    ctx = 2048
    q, k, v, kn, vn, ch = oracle.make_inputs(508, ctx, 1)
    with native.KvCache(n_layers=4, max_ctx=2304) as kv:
        oc = oracle.Cache(2304); oc.append(k, v, 0)
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
        kv.replicate_layer(0)
        one = kv.layer_call(3, q, kn, vn, ctx)
        for graph in (False, True):
            ms, out = kv.bench(q, kn, vn, ctx, mode=0, use_graph=graph, reps=3)
            assert (ms > 0).all()
            assert (out.view(np.uint16) == one.view(np.uint16)).all()


def _rows_equal(kv, oc, ctx, M):
    got = kv.export_rows(0, ctx, M)
    for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
        assert (a == b[:, ctx:ctx + M]).all()


@pytest.mark.parametrize("ctx,M", [(0, 64), (0, 3), (5, 33), (31, 64), (32, 16), (250, 64), (4000, 64)])
def test_wide_window_on_short_contexts_stores_its_rows(native, oracle, ctx, M):
    # the window's rows are quantized inside the attention launch by the split that owns their tiles; with few or no
    # cached tokens that split is the only one with keys
    kv, oc, q, kn, vn = _fill(native, oracle, 600 + ctx + M, ctx, M)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"ctx={ctx} M={M}")
        _rows_equal(kv, oc, ctx, M)


def test_fused_append_equals_separate_append(native, oracle):
    # yka_append + yka_attend against yka_append_attend: same cache rows, same outputs bit for bit (one split geometry)
    ctx, M = 1234, 40
    q, k, v, kn, vn, ch = oracle.make_inputs(610, ctx, M)
    oc = oracle.Cache(1536); oc.append(k, v, 0)
    outs = []
    for fused in (True, False):
        with native.KvCache(max_ctx=1536) as kv:
            kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
            if fused:
                outs.append(kv.layer_call(0, q, kn, vn, ctx))
            else:
                kv.append_host(0, kn, vn, ctx)
                outs.append(kv.layer_call(0, q, None, None, ctx))
            rows = kv.export_rows(0, ctx, M)
            outs.append(rows)
    assert (outs[0].view(np.uint16) == outs[2].view(np.uint16)).all()
    for a, b in zip(outs[1], outs[3]):
        assert (a == b).all()


def test_window_across_a_page_boundary_in_shuffled_pages(native, oracle):
    ctx, M = 2 * 256 - 20, 64                    # rows 492..555: the window starts in page 1 and ends in page 2
    q, k, v, kn, vn, ch = oracle.make_inputs(611, ctx, M)
    oc = oracle.Cache(1024); oc.append(k, v, 0)
    with native.KvCache(max_ctx=1024, paged=True) as kv:
        kv.set_page_table(np.array([2, 0, 3, 1], np.int32))
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], "paged window")
        _rows_equal(kv, oc, ctx, M)


@pytest.mark.parametrize("ctx", [31, 1023, 1024])
def test_rows_no_query_row_sees_are_still_stored(native, oracle, ctx):
    """Two sibling rows (depth table [0, 0]): no query row of the pass sees the second row, and when it opens a new 32-key
    tile (ctx + 1 a multiple of 32) no workgroup's key range holds it - the decode launch must store it all the same."""
    M = 2
    kv, oc, q, kn, vn = _fill(native, oracle, 640 + ctx, ctx, M)
    depth = np.array([0, 0], np.uint8)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx, depth=depth)
        oc.append(kn, vn, ctx)
        got = kv.export_rows(0, ctx, M)
        assert (got[0] == oc.kc[:, ctx:ctx + M]).all() and (got[1] == oc.ks[:, ctx:ctx + M]).all()
        assert (got[2] == oc.vc[:, ctx:ctx + M]).all() and (got[3] == oc.vs[:, ctx:ctx + M]).all()
        assert_attn_close(out, oc.attend_f32(q, ctx, depth, want_f32=True)[1], f"siblings at ctx={ctx}")


def test_depth_table_on_a_wide_window(native, oracle):
    ctx, M = 900, 24
    kv, oc, q, kn, vn = _fill(native, oracle, 612, ctx, M)
    depth = np.minimum(np.arange(M) // 2, 9).astype(np.uint8)     # a tree: rows see fewer keys than their index
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx, depth=depth)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, depth, threads=8, want_f32=True)[1], "depth table, wide")
        _rows_equal(kv, oc, ctx, M)


@pytest.mark.parametrize("hint", [64, 100000])
def test_context_hint_only_sizes_the_grid(native, oracle, hint):
    # option key 5 names the context the caller expects; any actual position stays correct
    for ctx, M in ((3000, 1), (3000, 64), (40, 2)):
        kv, oc, q, kn, vn = _fill(native, oracle, 620 + M, ctx, M, max_ctx=4096)
        with kv:
            kv.set_opt(5, hint)
            out = kv.layer_call(0, q, kn, vn, ctx)
            oc.append(kn, vn, ctx)
            assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"hint={hint} ctx={ctx} M={M}")
            _rows_equal(kv, oc, ctx, M)


def test_machine_probe_figures_are_plausible(native):
    """The in-library machine probe (fixed instruction mixes that time themselves): every kind runs, and what the waves
    measured is in the range this architecture can produce (an MFMA 32x32x16 takes 8 passes of 4 cycles)."""
    it = 500
    r = native.machine_probe(0, 0, it, 256, 256)
    assert 31.0 < r["cycles"] / (it * 4) < 40.0 and 1000 < r["shader_mhz"] < 3000, r
    r6 = native.machine_probe(0, 6, it, 256, 256)
    assert r6["cycles"] >= r["cycles"]
    for op in range(9):
        v = native.machine_probe(2, op, it, 64, 256)
        assert 1.0 < v["cycles"] / (it * 32) < 40.0, (op, v)
    x = native.machine_probe(5, 1, it, 64, 512)
    assert x["cycles"] > 0 and x["cycles_b"] > 0
    assert native.machine_probe(1, 0, it, 64, 256)["cycles"] > 0
    assert native.machine_probe(3, it, it, 64, 512)["cycles_b"] > 0
    rd = native.machine_probe(4, 0, 64, 1024, 256)
    assert 64 * 1048576 / (rd["ms"] * 1e-3) / 1e9 > 100.0          # GB/s: a 64 MiB read, mostly from cache
    with pytest.raises(native.YkaError):
        native.machine_probe(9, 0, it, 64, 256)
