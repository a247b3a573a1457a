"""Randomized shapes of the 128-channel path against the oracle: a seeded, bounded sweep over window widths, contexts,
depth tables, paged containers and split options, and the two shapes of an earlier (longer) sweep in which one output
value each landed two fp16 spacings from the oracle's - beyond the plain 2e-3 bar (tests/tolerances.py says why)."""
import numpy as np
import pytest

from tests.tolerances import MAX_ABS, assert_attn_close, attn_report

pytestmark = pytest.mark.gpu


def _run(native, oracle, seed, M, ctx, max_ctx, perm=None, depth=None, opts=()):
    q, k, v, kn, vn, ch = oracle.make_inputs(seed, ctx, M)
    oc = oracle.Cache(max_ctx)
    with native.KvCache(max_ctx=max_ctx, max_rows=max(M, 64), paged=perm is not None) as kv:
        if perm is not None:
            kv.set_page_table(np.asarray(perm, np.int32))
        if ctx:
            oc.append(k, v, 0)
            kv.import_rows(0, 0, oc.kc[:, :ctx], oc.ks[:, :ctx], oc.vc[:, :ctx], oc.vs[:, :ctx])
        for key, val in opts:
            kv.set_opt(key, val)
        out = kv.layer_call(0, q, kn, vn, ctx, depth=depth)
        got = kv.export_rows(0, ctx, M)
    oc.append(kn, vn, ctx)
    for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
        assert (a == b[:, ctx:ctx + M]).all(), "appended rows differ"
    return out, oc.attend_f32(q, ctx, depth, threads=8, want_f32=True)[1]


@pytest.mark.parametrize("seed,M,ctx,max_ctx,perm,opts", [
    (1210, 1025, 64, 1280, [2, 1, 3, 0, 4], [(5, 1011)]),       # a prefill chunk on 64 cached tokens, paged, context hint
    (1114, 388, 0, 512, None, [(1, 104)]),                      # a 388-row pass on an empty container
])
def test_shapes_that_reached_two_spacings(native, oracle, seed, M, ctx, max_ctx, perm, opts):
    out, ref = _run(native, oracle, seed, M, ctx, max_ctx, perm, None, opts)
    assert_attn_close(out, ref, f"M={M} ctx={ctx}", two_spacings=True)
    plain, scaled, rl, _ = attn_report(out, ref)
    print(f"M={M} ctx={ctx}: plain max-abs {plain:.3e} ({'over' if plain > MAX_ABS else 'within'} the plain bar), rel-L2 {rl:.3e}")


def test_seeded_randomized_sweep(native, oracle):
    rng = np.random.default_rng(2024)
    over = []
    for case in range(60):
        kind = rng.integers(0, 10)
        M = int(rng.integers(1, 65)) if kind < 6 else int(rng.integers(65, 300)) if kind < 9 else int(rng.choice([64, 65, 66, 127, 128, 129]))
        ctx = int(rng.choice([0, 1, 5, 31, 32, 33, 63, 64, 65, 255, 256, 257, int(rng.integers(0, 3000)), int(rng.integers(0, 3000))]))
        paged = bool(rng.integers(0, 2))
        max_ctx = ((ctx + M + 255) // 256 + int(rng.integers(0, 3))) * 256
        depth = None
        if M <= 64 and rng.integers(0, 3) == 0:
            d = [0]
            for t in range(1, M):
                d.append(int(rng.integers(max(0, d[-1] - 2), min(t, d[-1] + 1) + 1)))
            depth = np.array(d, np.uint8)
        perm = rng.permutation(max_ctx // 256).astype(np.int32) if paged else None
        opt = int(rng.integers(0, 8))
        opts = {1: [(2, int(rng.integers(1, 40)))], 2: [(1, int(rng.integers(1, 200)))], 3: [(5, int(rng.integers(0, max_ctx + 1)))],
                4: [(7, 1)], 5: [(8, int(rng.choice([0, 16, 64])))], 6: [(9, int(rng.integers(1, 100))), (8, 16)]}.get(opt, [])
        out, ref = _run(native, oracle, 5000 + case, M, ctx, max_ctx, perm, depth, opts)
        what = f"case {case}: M {M} ctx {ctx} max_ctx {max_ctx} paged {paged} depth {depth is not None} opts {opts}"
        assert_attn_close(out, ref, what, two_spacings=True)
        plain = attn_report(out, ref)[0]
        if plain > MAX_ABS:
            over.append((what, plain))
    # values two spacings off are possible (see the module docstring) but rare: none or a few of the 60 shapes
    assert len(over) <= 3, over


@pytest.mark.parametrize("M", [1, 2, 8, 16, 64, 130])
def test_large_magnitudes(native, oracle, M):
    """Every kernel at the far end of the fp16 range: K rows of magnitude up to 6e4 (group scales up to 9e3), V rows of
    magnitude up to 3e4, small queries so that the scores still discriminate.  The scaled K images of the mid kernel, the
    exact codes x fp32 scales of the other two and the scaled V images all have to stay finite and exact."""
    rng = np.random.default_rng(8800 + M)
    ctx = 600
    k = np.clip(rng.standard_normal((ctx + M, 4, 128)) * 9000.0, -60000, 60000).astype(np.float16)
    v = np.clip(rng.standard_normal((ctx + M, 4, 128)) * 6000.0, -30000, 30000).astype(np.float16)
    q = (rng.standard_normal((M, 24, 128)) * 1e-3).astype(np.float16)
    max_ctx = 1024
    oc = oracle.Cache(max_ctx)
    with native.KvCache(max_ctx=max_ctx, max_rows=max(M, 64)) as kv:
        kv.set_opt(8, 16)
        kv.append_host(0, k[:ctx], v[:ctx], 0)
        out = kv.layer_call(0, q, k[ctx:], v[ctx:], ctx)
        oc.append(k, v, 0)
        got = kv.export_rows(0, 0, ctx + M)
        for a, b in zip(got, (oc.kc, oc.ks, oc.vc, oc.vs)):
            assert (a == b[:, :ctx + M]).all()
    ref32 = oc.attend_f32(q, ctx, threads=8, want_f32=True)[1]
    assert np.isfinite(out.astype(np.float32)).all()
    a, b = out.astype(np.float64), ref32.astype(np.float64)
    assert np.linalg.norm(a - b) / np.linalg.norm(b) <= 1e-3
    # a row is a weighted mean of V rows of magnitude ~1e4, each held as fp16(code x scale): the error of every channel
    # scales with the magnitude of the row, not with the channel's own value
    row_scale = np.abs(b).max(axis=2, keepdims=True)
    assert (np.abs(a - b) <= 2e-3 * np.maximum(1.0, row_scale)).all(), (np.abs(a - b) / np.maximum(1.0, row_scale)).max()
