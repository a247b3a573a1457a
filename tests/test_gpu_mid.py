"""The kernel for windows of 3..16 rows (attend_mid.hip) through the C ABI against the oracle: outputs within the attention
bars (tests/tolerances.py), appended rows bit for bit, and against the wide kernel on the same inputs."""
import numpy as np
import pytest

from tests.tolerances import assert_attn_close, attn_errors

pytestmark = pytest.mark.gpu


def _fill(native, oracle, seed, ctx, M, max_ctx=None, **kw):
    q, k, v, kn, vn, ch = oracle.make_inputs(seed, ctx, M)
    max_ctx = max_ctx or ((ctx + M + 255) // 256) * 256
    oc = oracle.Cache(max_ctx)
    kv = native.KvCache(max_ctx=max_ctx, **kw)
    kv.set_opt(8, 16)              # every window of up to 16 rows through this kernel (by default the wide kernel takes over earlier)
    if ctx:
        oc.append(k, v, 0)
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
    return kv, oc, q, kn, vn


def _rows_equal(kv, oc, ctx, M):
    got = kv.export_rows(0, ctx, M)
    for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
        assert (a == b[:, ctx:ctx + M]).all()


@pytest.mark.parametrize("M", [3, 4, 5, 6, 8, 9, 10, 11, 12, 13, 14, 16])
def test_window_matches_oracle(native, oracle, M):
    """Every row-tile count of the kernel (2..6 tiles of 16 rows), full and ragged last tiles."""
    ctx = 1500
    kv, oc, q, kn, vn = _fill(native, oracle, 7000 + M, ctx, M)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"window M={M}")
        _rows_equal(kv, oc, ctx, M)


@pytest.mark.parametrize("ctx", [0, 1, 17, 31, 32, 33, 100, 127, 128, 129, 255, 256, 257])
@pytest.mark.parametrize("M", [3, 16])
def test_short_contexts(native, oracle, ctx, M):
    """Few tiles: waves without tiles, one workgroup in use, the window inside / across the first tiles and a page boundary."""
    kv, oc, q, kn, vn = _fill(native, oracle, 7100 + 17 * ctx + M, ctx, M, max_ctx=512)
    with kv:
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=4, want_f32=True)[1], f"ctx={ctx} M={M}")
        _rows_equal(kv, oc, ctx, M)


@pytest.mark.parametrize("S", [1, 2, 3, 7, 31, 64, 128])
def test_split_count_does_not_matter(native, oracle, S):
    ctx, M = 5000, 12
    kv, oc, q, kn, vn = _fill(native, oracle, 7200, ctx, M)
    with kv:
        kv.set_opt(9, S)
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"splits={S}")
        _rows_equal(kv, oc, ctx, M)


def test_equals_the_wide_kernel_within_the_bars(native, oracle):
    """Option key 8 = 0 sends the same window through the 128-row workgroups of the wide kernel."""
    ctx, M = 2600, 16
    kv, oc, q, kn, vn = _fill(native, oracle, 7300, ctx, M)
    with kv:
        mid = kv.layer_call(0, q, kn, vn, ctx)
        kv.set_opt(8, 0)
        wide = kv.layer_call(0, q, kn, vn, ctx)
        ma, rl = attn_errors(mid, wide)
        assert ma <= 2e-3 and rl <= 1e-3, (ma, rl)
        assert not (mid.view(np.uint16) == wide.view(np.uint16)).all()      # two different kernels did run


@pytest.mark.parametrize("M", [17, 33, 64])
def test_wider_windows_as_row_blocks(native, oracle, M):
    """Option key 8 = 64: windows wider than 16 rows run as blocks of 16 tokens (grid z); every block stores the rows it reads."""
    ctx = 1300
    kv, oc, q, kn, vn = _fill(native, oracle, 7400 + M, ctx, M)
    with kv:
        kv.set_opt(8, 64)
        out = kv.layer_call(0, q, kn, vn, ctx)
        oc.append(kn, vn, ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], f"M={M} in blocks")
        _rows_equal(kv, oc, ctx, M)


def test_depth_table_and_unseen_rows(native, oracle):
    """A depth table (siblings: rows that no later row sees) - lengths differ inside a row tile, and a row that opens a new
    32-key tile which no query row can see still has to be stored."""
    for ctx, depth in ((700, [0, 1, 1, 2, 2, 3, 3, 3]), (31, [0, 0, 0, 0]), (63, [0, 0, 0]), (95, [0, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1])):
        M = len(depth)
        dp = np.array(depth, np.uint8)
        kv, oc, q, kn, vn = _fill(native, oracle, 7500 + ctx, ctx, M, max_ctx=1024)
        with kv:
            out = kv.layer_call(0, q, kn, vn, ctx, depth=dp)
            oc.append(kn, vn, ctx)
            assert_attn_close(out, oc.attend_f32(q, ctx, dp, want_f32=True)[1], f"depth table ctx={ctx}")
            _rows_equal(kv, oc, ctx, M)


def test_paged_is_bit_identical_to_contiguous(native, oracle):
    ctx, M = 2000, 11
    q, k, v, kn, vn, ch = oracle.make_inputs(7600, ctx, M)
    oc = oracle.Cache(2304); oc.append(k, v, 0)
    rng = np.random.default_rng(7600)
    outs = []
    for paged in (False, True):
        with native.KvCache(max_ctx=2304, paged=paged) as kv:
            kv.set_opt(8, 16)
            if paged:
                kv.set_page_table(rng.permutation(9).astype(np.int32))
            kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
            outs.append(kv.layer_call(0, q, kn, vn, ctx))
    assert (outs[0].view(np.uint16) == outs[1].view(np.uint16)).all()
    oc.append(kn, vn, ctx)
    assert_attn_close(outs[1], oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], "paged")


def test_window_rows_equal_single_row_calls(native, oracle):
    """The reference's built-in invariant (src/kvx_probe.cu:425-436) in its tolerance form: row t of the window against a
    one-row pass at position ctx + t over the rows the window stored."""
    ctx, M = 900, 16
    kv, oc, q, kn, vn = _fill(native, oracle, 7700, ctx, M)
    with kv:
        full = kv.layer_call(0, q, kn, vn, ctx)
        for t in range(M):
            one = kv.layer_call(0, q[t:t + 1], None, None, ctx + t)
            ma, rl = attn_errors(one, full[t:t + 1])
            assert ma <= 2e-3 and rl <= 1e-3, (t, ma, rl)


def test_large_scores_raise_the_running_maximum(native, oracle):
    """Scores that grow along the context (every later tile beats the running maximum by more than the lazy-raise slack):
    the rescale path of the accumulators runs on many tiles."""
    ctx, M = 1024, 8
    rng = np.random.default_rng(7800)
    k = rng.standard_normal((ctx + M, 4, 128)).astype(np.float32)
    ramp = np.linspace(0.2, 6.0, ctx + M, dtype=np.float32)[:, None, None]
    base = rng.standard_normal((1, 4, 128)).astype(np.float32)
    k = (0.3 * k + base * ramp).astype(np.float16)
    v = rng.standard_normal((ctx + M, 4, 128)).astype(np.float16)
    q = np.repeat(base, 6, axis=1).repeat(M, axis=0).astype(np.float16)       # aligned with the ramp direction
    oc = oracle.Cache(1280); oc.append(k[:ctx], v[:ctx], 0)
    with native.KvCache(max_ctx=1280) as kv:
        kv.set_opt(8, 16)
        kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)
        oc.append(k[ctx:], v[ctx:], ctx)
        assert_attn_close(out, oc.attend_f32(q, ctx, threads=8, want_f32=True)[1], "growing scores")


@pytest.mark.parametrize("M", [4, 8, 16])
def test_windows_at_32k(native, oracle, M):
    """The measured size: 32768 cached tokens (1025 tiles over 256 waves), rows quantized by the library itself."""
    ctx = 32768
    ch = oracle.outlier_channels(7900 + M)
    q = oracle.fill_normal_f16(7901 + M, M * 24).reshape(M, 24, 128)
    k = oracle.fill_normal_f16(7902 + M, (ctx + M) * 4, 128, ch, 8.0).reshape(ctx + M, 4, 128)
    v = oracle.fill_normal_f16(7903 + M, (ctx + M) * 4).reshape(ctx + M, 4, 128)
    with native.KvCache(max_ctx=33024) as kv:
        kv.set_opt(8, 16)
        for p in range(0, ctx, 8192):
            kv.append_host(0, k[p:p + 8192], v[p:p + 8192], p)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)
        oc = oracle.Cache(33024)
        n = ctx + M
        oc.kc[:, :n], oc.ks[:, :n], oc.vc[:, :n], oc.vs[:, :n] = kv.export_rows(0, 0, n)
        chk = oracle.Cache(256)
        chk.append(k[ctx:], v[ctx:], 0)
        for a, b in zip((chk.kc, chk.ks, chk.vc, chk.vs), (oc.kc, oc.ks, oc.vc, oc.vs)):
            assert (a[:, :M] == b[:, ctx:ctx + M]).all()                     # the rows the kernel stored: the oracle's quantizer, bit for bit
        ref32 = oc.attend_f32(q, ctx, threads=16, want_f32=True)[1]
        assert_attn_close(out, ref32, f"32k M={M}")
        assert np.abs(out.astype(np.float64) - ref32).max() <= 2e-3
