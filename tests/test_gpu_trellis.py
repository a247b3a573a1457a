"""Trellis-coded rows on the GPU against the oracle: payload words, scales, projection coefficients, the encoder's
reconstruction and the decoder's rows, all bit for bit.  Synthetic profile blobs (see tests/test_oracle_trellis.py)."""
import numpy as np
import pytest

from yasakani_amd import kvqp

pytestmark = pytest.mark.gpu


def _rows(seed, n):
    rng = np.random.default_rng(seed)
    y = (rng.standard_normal((n, 256)) * rng.uniform(0.05, 6, (n, 1))).astype(np.float32)
    y[:, [5, 77, 130, 201]] *= 8
    y[3] = 0                                                       # rms 0 -> 1, scale from the multiplier alone
    y[4, 1:] = 0
    return y


def _same(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint32), np.ascontiguousarray(b).view(np.uint32))


@pytest.mark.parametrize("kk,mu,dirs,flat", [(5, False, 0, ()), (4, False, 0, ()), (3, False, 0, ()), (5, True, 2, ()), (4, True, 1, (1, 6))])
def test_rows_bit_exact(native, oracle, kk, mu, dirs, flat):
    blob = kvqp.synthetic(layers=2, kk=kk, seed=kk + 10 * dirs, mu=mu, dirs=dirs, flat_groups=flat)
    n = 96
    y = _rows(kk, n)
    grp = (np.arange(n) * 5) % 16
    pos = np.arange(n)
    ref = oracle.tb_encode_rows(blob, grp, pos, y, stride_words=40)
    got = native.tb_pack_unpack(blob, y, grp, pos, stride=160)
    assert ref["coded"].all()
    assert np.array_equal(got["words"], ref["words"])
    assert _same(got["scale"], ref["scale"]) and np.array_equal(got["pc"], ref["pc"])
    assert _same(got["x"], ref["x"])
    assert _same(got["dec"], ref["x"])                             # the decoder reproduces the encoder's row
    assert _same(got["dec"], oracle.tb_decode_rows(blob, grp, ref["words"], ref["scale"], ref["pc"]))


@pytest.mark.parametrize("kk", [3, 4, 5])
def test_rows_bit_exact_when_paths_tie(native, oracle, kk):
    """Tables with few distinct values and rows of few distinct values: many paths cost the same, so the rows depend on the
    tie rules (smallest predecessor among equal costs, smallest final state) and on the clamp of the targets."""
    rng = np.random.default_rng(100 + kk)
    coarse = (rng.integers(-3, 4, 256) * 256).astype(np.int16)      # 7 distinct table values
    two = np.where(rng.random(256) < 0.5, -512, 512).astype(np.int16)
    groups = [dict(mode=0, kk=kk, table=g & 1, guard=0, mu=None, dirs=[]) for g in range(8)]
    blob = kvqp.build(1, 4, np.array([0.5, 1.0, 1.0, 2.0], np.float32), [(1.0, coarse), (1.0, two)], groups)
    n = 64
    y = rng.integers(-2, 3, (n, 256)).astype(np.float32)            # values in {-2..2}
    y[0] = 0
    y[1] = 1
    y[2, ::2] = 40; y[2, 1::2] = -40                                # targets far outside the table: clamped
    y[3] = np.where(np.arange(256) % 64 < 32, 3.0, -3.0)
    grp = np.arange(n) % 8
    pos = np.arange(n)
    ref = oracle.tb_encode_rows(blob, grp, pos, y, stride_words=40)
    got = native.tb_pack_unpack(blob, y, grp, pos, stride=160)
    assert np.array_equal(got["words"], ref["words"])
    assert _same(got["scale"], ref["scale"]) and _same(got["x"], ref["x"]) and _same(got["dec"], ref["x"])


def test_guard_rows_and_missing_groups_pass_through(native, oracle):
    blob = kvqp.synthetic(layers=1, kk=5, seed=4, guard=7)
    y = _rows(9, 24)
    grp = np.arange(24) % 8
    grp[20:] = 99                                                  # no such group
    pos = np.arange(24)                                            # rows 0..6 sit below the guard position
    ref = oracle.tb_encode_rows(blob, grp, pos, y)
    got = native.tb_pack_unpack(blob, y, grp, pos)
    assert not ref["coded"][:7].any() and ref["coded"][7:20].all() and not ref["coded"][20:].any()
    assert _same(got["x"], ref["x"]) and _same(got["dec"], ref["x"])
    assert np.array_equal(got["words"], ref["words"])
    assert _same(got["x"][:7], y[:7]) and _same(got["x"][20:], y[20:])


def test_many_rows_cross_the_launch_tile(native, oracle):
    blob = kvqp.synthetic(layers=1, kk=4, seed=1)
    n = 1100                                                       # more than one launch of 1024 rows
    y = _rows(21, n)
    grp = np.arange(n) % 8
    ref = oracle.tb_encode_rows(blob, grp, np.zeros(n, np.int32), y)
    got = native.tb_pack_unpack(blob, y, grp, np.zeros(n, np.int32))
    assert np.array_equal(got["words"], ref["words"]) and _same(got["scale"], ref["scale"]) and _same(got["x"], ref["x"])


def test_bad_blobs_are_refused(native):
    blob = bytearray(kvqp.synthetic())
    y = np.zeros((1, 256), np.float32)
    bad = bytearray(blob); bad[1] = 0
    with pytest.raises(native.YkaError, match="KVQP"):
        native.tb_pack_unpack(bad, y, [0], [0])
    with pytest.raises(native.YkaError, match="KVQP"):
        native.tb_pack_unpack(blob[:-4], y, [0], [0])
    with pytest.raises(native.YkaError, match="stride"):
        native.tb_pack_unpack(blob, y, [0], [0], stride=128)


# ---- the cache: trellis-coded rows behind the ordinary entry points ----
NH, KVH = 24, 4


def _kv_rows(seed, n):
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((n, KVH, 256)).astype(np.float32)
    k[:, :, [5, 77, 130, 201]] *= 4
    v = rng.standard_normal((n, KVH, 256)).astype(np.float32)
    return k, v


def _oracle_rows(oracle, blob, layer, k, v):
    """rows [n, KVH, 256] -> per kv head: coded rows of K and V as the oracle codes them"""
    n = k.shape[0]
    enc = {}
    for kind, x in ((0, k), (1, v)):
        for h in range(KVH):
            g = (layer * KVH + h) * 2 + kind
            enc[kind, h] = oracle.tb_encode_rows(blob, np.full(n, g, np.int32), np.arange(n, dtype=np.int32), x[:, h])
            assert enc[kind, h]["coded"].all()
    return enc


@pytest.mark.parametrize("kk,mu", [(5, False), (4, False), (5, True), (4, True)])
@pytest.mark.parametrize("ctx,M", [(0, 1), (0, 7), (70, 2), (300, 5), (1000, 1), (1500, 16), (2100, 64)])
def test_cache_rows_bit_exact_and_attention_within_the_bars(native, oracle, kk, mu, ctx, M):
    from tolerances import assert_attn_close
    layer = 1
    blob = kvqp.synthetic(layers=2, kk=kk, seed=3 + kk, mu=mu)
    n = ctx + M
    k, v = _kv_rows(ctx * 7 + M + kk, n)
    k16, v16 = k[ctx:].astype(np.float16), v[ctx:].astype(np.float16)
    k[ctx:] = k16; v[ctx:] = v16                                   # the pass's own rows arrive as fp16
    q = np.random.default_rng(n).standard_normal((M, NH, 256)).astype(np.float16)
    max_ctx = ((n + 255) // 256) * 256
    with native.KvCache(n_layers=2, head_dim=256, max_ctx=max_ctx) as kv:
        kv.set_profile(blob)
        assert kv.profile_bits == kk
        for p in range(0, ctx, 64):
            m = min(64, ctx - p)
            kv.append256_f32_host(layer, k[p:p + m], v[p:p + m], p, rotate=False)
        out = kv.layer_call(layer, q, k16, v16, ctx)
        kw, ks, vw, vs = kv.export_rows(layer, 0, n)
    enc = _oracle_rows(oracle, blob, layer, k, v)
    kd = np.empty((KVH, n, 256), np.float32); vd = np.empty_like(kd)
    for h in range(KVH):
        assert np.array_equal(kw[h], enc[0, h]["words"][:, :8 * kk]) and np.array_equal(vw[h], enc[1, h]["words"][:, :8 * kk]), h
        assert _same(ks[h], enc[0, h]["scale"]) and _same(vs[h], enc[1, h]["scale"])
        kd[h] = enc[0, h]["x"]; vd[h] = enc[1, h]["x"]
    assert_attn_close(out, oracle.tb_attend_f64(kd, vd, q, ctx), f"kk={kk} mu={mu} ctx={ctx} M={M}")


def test_depth_table_and_split_counts(native, oracle):
    from tolerances import assert_attn_close
    blob = kvqp.synthetic(layers=1, kk=5, seed=11)
    ctx, M = 700, 6
    k, v = _kv_rows(5, ctx + M)
    q = np.random.default_rng(6).standard_normal((M, NH, 256)).astype(np.float16)
    depth = np.array([0, 1, 1, 2, 2, 3], np.uint8)
    with native.KvCache(head_dim=256, max_ctx=1024) as kv:
        kv.set_profile(blob)
        for p in range(0, ctx + M, 64):
            m = min(64, ctx + M - p)
            kv.append256_f32_host(0, k[p:p + m], v[p:p + m], p, rotate=False)
        outs = []
        for S in (0, 3, 97, 200):
            kv.set_opt(1, S)
            outs.append(kv.layer_call(0, q, None, None, ctx, depth=depth))
    enc = _oracle_rows(oracle, blob, 0, k, v)
    kd = np.stack([enc[0, h]["x"] for h in range(KVH)]); vd = np.stack([enc[1, h]["x"] for h in range(KVH)])
    expect = oracle.tb_attend_f64(kd, vd, q, ctx, depth=depth)
    for o, name in zip(outs, ("default", "3 splits", "97 splits", "200 splits")):
        assert_attn_close(o, expect, name)


def test_profiles_the_packed_cache_cannot_hold_are_refused(native):
    with native.KvCache(head_dim=256, max_ctx=256) as kv:
        for kw in (dict(kk=3), dict(kk=5, dirs=1), dict(kk=5, guard=2), dict(kk=5, flat_groups=(0,))):
            with pytest.raises(native.YkaError, match="packed rows need"):
                kv.set_profile(kvqp.synthetic(layers=1, **kw))
        with pytest.raises(native.YkaError, match="cover"):
            kv.set_profile(kvqp.synthetic(layers=1, kv_heads=2))
        kv.set_profile(kvqp.synthetic(layers=1, kk=4))
        with pytest.raises(native.YkaError, match="already"):
            kv.set_profile(kvqp.synthetic(layers=1, kk=4))
        with pytest.raises(native.YkaError, match="no groups for this layer"):
            kv.set_opt(6, 1)                                   # the multi-stream pass would use the groups of layer 1
            kv.ms_call(np.zeros((1, NH, 256), np.float16), None, None, np.zeros(1, np.int32), np.zeros(1, np.int32))
    with native.KvCache(max_ctx=256) as kv:
        with pytest.raises(native.YkaError, match="256"):
            kv.set_profile(kvqp.synthetic(layers=1))


@pytest.mark.parametrize("kk", [4, 5])
def test_wide_and_narrow_kernels_agree_on_a_window(native, oracle, kk):
    """the same 40-row window through the 128-row workgroups and (option key 3) through row tiles of 2 tokens"""
    from tolerances import assert_attn_close
    blob = kvqp.synthetic(layers=1, kk=kk, seed=21, mu=True)
    ctx, M = 900, 40
    k, v = _kv_rows(kk, ctx + M)
    q = np.random.default_rng(kk).standard_normal((M, NH, 256)).astype(np.float16)
    with native.KvCache(head_dim=256, max_ctx=1024) as kv:
        kv.set_profile(blob)
        for p in range(0, ctx + M, 64):
            m = min(64, ctx + M - p)
            kv.append256_f32_host(0, k[p:p + m], v[p:p + m], p, rotate=False)
        wide = kv.layer_call(0, q, None, None, ctx)
        kv.set_opt(2, 5)
        wide5 = kv.layer_call(0, q, None, None, ctx)
        kv.set_opt(3, 1)
        narrow = kv.layer_call(0, q, None, None, ctx)
    enc = _oracle_rows(oracle, blob, 0, k, v)
    kd = np.stack([enc[0, h]["x"] for h in range(KVH)]); vd = np.stack([enc[1, h]["x"] for h in range(KVH)])
    expect = oracle.tb_attend_f64(kd, vd, q, ctx)
    assert_attn_close(wide, expect, "wide"); assert_attn_close(wide5, expect, "wide, 5 splits"); assert_attn_close(narrow, expect, "narrow")


def test_graph_replay_equals_eager_calls(native):
    """the captured form of a layer call (encoder, attention, combine recorded into a graph and replayed over every
    container) gives the bytes of the eager call, for a decode step and for a window"""
    blob = kvqp.synthetic(layers=3, kk=5, seed=2)
    ctx = 600
    k, v = _kv_rows(31, ctx + 20)
    k16, v16 = k.astype(np.float16), v.astype(np.float16)
    rng = np.random.default_rng(32)
    with native.KvCache(n_layers=3, head_dim=256, max_ctx=768) as kv:
        kv.set_profile(blob)
        for layer in range(3):
            for p in range(0, ctx, 64):
                m = min(64, ctx - p)
                kv.append_host(layer, k16[p:p + m], v16[p:p + m], p)
        for M in (1, 20):
            q = rng.standard_normal((M, NH, 256)).astype(np.float16)
            eager = kv.layer_call(2, q, k16[ctx:ctx + M], v16[ctx:ctx + M], ctx)
            _, replay = kv.bench(q, k16[ctx:ctx + M], v16[ctx:ctx + M], ctx, mode=0, use_graph=True, reps=3)
            assert np.array_equal(eager.view(np.uint16), replay.view(np.uint16)), M


def test_rotated_rows_are_rotated_before_they_are_coded(native, oracle):
    """yka_append256_f32 with rotate = 1 on a handle with a profile: signed Hadamard rotation (kvx_rotate), then the
    trellis encoder - stored words and scales against the oracle's rotation followed by the oracle's encoder"""
    blob = kvqp.synthetic(layers=1, kk=5, seed=17)
    n = 70
    k, v = _kv_rows(77, n)
    with native.KvCache(head_dim=256, max_ctx=256) as kv:
        kv.set_profile(blob)
        kv.append256_f32_host(0, k[:64], v[:64], 0, rotate=True)
        kv.append256_f32_host(0, k[64:], v[64:], 64, rotate=True)
        kw, ks, vw, vs = kv.export_rows(0, 0, n)
    kr = np.stack([oracle.kvx_rotate256(k[:, h]) for h in range(KVH)], 1)
    vr = np.stack([oracle.kvx_rotate256(v[:, h]) for h in range(KVH)], 1)
    enc = _oracle_rows(oracle, blob, 0, kr, vr)
    for h in range(KVH):
        assert np.array_equal(kw[h], enc[0, h]["words"][:, :40]) and np.array_equal(vw[h], enc[1, h]["words"][:, :40]), h
        assert _same(ks[h], enc[0, h]["scale"]) and _same(vs[h], enc[1, h]["scale"])


@pytest.mark.parametrize("rot", [False, True])
def test_attn_post_feeds_the_encoder(native, oracle, rot):
    """yka_attn_post on a handle with a profile: RMS norm + rotary + rotation as on flat rows (Q rows bit-exact), and the
    finished K / V rows coded by the trellis encoder: stored words and scales against the oracle's post step followed by
    the oracle's encoder"""
    blob = kvqp.synthetic(layers=1, kk=5, seed=23)
    rng = np.random.default_rng(24)
    M, rd, pos, ctx = 5, 64, 250, 512
    xq = (rng.standard_normal((M, NH, 256)) * 2).astype(np.float32)
    xk = (rng.standard_normal((M, KVH, 256)) * 0.7).astype(np.float32)
    xk[:, :, [5, 77, 130, 201]] *= 8
    xv = rng.standard_normal((M, KVH, 256)).astype(np.float32)
    qw = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    kw_ = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    rope = oracle.rope_table(ctx, rd)
    q16, k32, v32 = oracle.attn_post256(xq, xk, xv, qw, kw_, 1e-6, rope, rd, pos, int(rot))
    with native.KvCache(head_dim=256, max_ctx=ctx) as kv:
        kv.set_profile(blob)
        got_q = kv.attn_post_host(0, xq, xk, xv, pos, qw, kw_, 1e-6, rope, rd, rotate=rot)
        kw, ks, vw, vs = kv.export_rows(0, pos, M)
    assert np.array_equal(got_q.view(np.uint16), q16)
    for h in range(KVH):
        for kind, x, w, s in ((0, k32, kw, ks), (1, v32, vw, vs)):
            enc = oracle.tb_encode_rows(blob, np.full(M, h * 2 + kind, np.int32), np.arange(pos, pos + M, dtype=np.int32), x[:, h])
            assert np.array_equal(w[h], enc["words"][:, :40]) and _same(s[h], enc["scale"]), (h, kind)


# ---- multi-stream passes over trellis-coded rows: every row names its own container (stream) and position ----
MS_CTX = 1024
MS_LENS = [300, 17, 900, 512, 0]                       # cached tokens per stream; the last stream is empty


def _streams(native, oracle, blob, layer):
    rng = np.random.default_rng(55)
    kv = native.KvCache(n_layers=len(MS_LENS), head_dim=256, max_ctx=MS_CTX, max_rows=64)
    kv.set_profile(blob)
    kv.set_opt(6, layer)
    rows = []
    for s, n in enumerate(MS_LENS):
        k = np.zeros((MS_CTX, KVH, 256), np.float16); v = np.zeros_like(k)
        if n:
            kn = rng.standard_normal((n, KVH, 256)).astype(np.float16); kn[:, :, [5, 77, 130, 201]] *= 4
            vn = rng.standard_normal((n, KVH, 256)).astype(np.float16)
            k[:n] = kn; v[:n] = vn
            # fill through the multi-stream pass itself: rows of stream s at positions 0 .. n-1, 32 at a time
            for p in range(0, n, 32):
                m = min(32, n - p)
                kv.ms_call(np.zeros((m, NH, 256), np.float16), kn[p:p + m], vn[p:p + m], np.arange(p, p + m, dtype=np.int32), np.full(m, s, np.int32))
        rows.append([k, v, n])
    return kv, rows, rng


def _stream_expect(oracle, blob, layer, k, v, n, q, pos):
    """fp64 attention of one row at position pos over the oracle-coded rows [0, pos] of its stream"""
    enc = _oracle_rows(oracle, blob, layer, k[:n].astype(np.float32), v[:n].astype(np.float32))
    kd = np.stack([enc[0, h]["x"] for h in range(KVH)]); vd = np.stack([enc[1, h]["x"] for h in range(KVH)])
    return oracle.tb_attend_f64(kd, vd, q, pos), enc


def test_multi_stream_pass_over_trellis_rows(native, oracle):
    from tolerances import assert_attn_close
    layer = 1
    blob = kvqp.synthetic(layers=2, kk=5, seed=13, mu=True)
    kv, rows, rng = _streams(native, oracle, blob, layer)
    with kv:
        # one new row per stream, in any slot order; plus a row whose slot does not exist and one beyond its container
        slots = np.array([2, 0, 4, 1, 3, 9, 1], np.int32)
        pos = np.array([MS_LENS[s] if s < len(MS_LENS) else 5 for s in slots], np.int32)
        pos[6] = MS_CTX
        M = len(slots)
        q = rng.standard_normal((M, NH, 256)).astype(np.float16)
        kn = rng.standard_normal((M, KVH, 256)).astype(np.float16); vn = rng.standard_normal((M, KVH, 256)).astype(np.float16)
        out = kv.ms_call(q, kn, vn, pos, slots)
        assert not out[5:7].view(np.uint16).any()                       # rejected rows yield zeros
        for t in range(5):
            s = int(slots[t]); k, v, n = rows[s]
            k[n] = kn[t]; v[n] = vn[t]
            expect, enc = _stream_expect(oracle, blob, layer, k, v, n + 1, q[t:t + 1], n)
            assert_attn_close(out[t:t + 1], expect, f"row {t} stream {s}")
            kw, ks, vw, vs = kv.export_rows(s, n, 1)
            for h in range(KVH):                                          # the row the pass stored for this stream: bit-exact
                assert np.array_equal(kw[h, 0], enc[0, h]["words"][n, :40]) and np.array_equal(vw[h, 0], enc[1, h]["words"][n, :40])
                assert _same(ks[h, 0:1], enc[0, h]["scale"][n:n + 1]) and _same(vs[h, 0:1], enc[1, h]["scale"][n:n + 1])
        # rows of one stream that follow each other see each other's keys; attend only for the rest
        slots = np.array([0, 0, 0, 2], np.int32); pos = np.array([301, 302, 303, 900], np.int32)
        q = rng.standard_normal((4, NH, 256)).astype(np.float16)
        kn = rng.standard_normal((4, KVH, 256)).astype(np.float16); vn = rng.standard_normal((4, KVH, 256)).astype(np.float16)
        out = kv.ms_call(q, kn, vn, pos, slots)
        k, v, _ = rows[0]
        k[301:304] = kn[:3]; v[301:304] = vn[:3]
        for t in range(3):
            expect, _ = _stream_expect(oracle, blob, layer, k, v, 302 + t, q[t:t + 1], 301 + t)
            assert_attn_close(out[t:t + 1], expect, f"stream 0 row {t}")


@pytest.mark.parametrize("kk", [5, 4])
def test_full_length_32768_decode_and_window(native, oracle, kk):
    """32,768 cached tokens (4,096 distinct rows tiled over the context): the rows the GPU stored are decoded by the oracle
    and a decode step, a 3-row window (wide kernel) and the same window on row tiles are checked against fp64 attention."""
    from tolerances import assert_attn_close
    ctx, U, M = 32768, 4096, 3
    blob = kvqp.synthetic(layers=1, kk=kk, seed=61, mu=True)
    rng = np.random.default_rng(62 + kk)
    k = rng.standard_normal((U + M, KVH, 256)).astype(np.float16); k[:, :, [5, 77, 130, 201]] *= 4
    v = rng.standard_normal((U + M, KVH, 256)).astype(np.float16)
    q = rng.standard_normal((M, NH, 256)).astype(np.float16)
    with native.KvCache(head_dim=256, max_ctx=ctx + 256) as kv:
        kv.set_profile(blob)
        for p in range(0, ctx, 64):
            s0 = p % U
            kv.append_host(0, k[s0:s0 + 64], v[s0:s0 + 64], p)
        dec1 = kv.layer_call(0, q[:1], k[U:U + 1], v[U:U + 1], ctx)
        win = kv.layer_call(0, q, k[U:], v[U:], ctx)
        kv.set_opt(3, 1)
        win_tiles = kv.layer_call(0, q, None, None, ctx)
        kw, ks, vw, vs = kv.export_rows(0, 0, U)
        kw2, ks2, vw2, vs2 = kv.export_rows(0, ctx, M)
        tail = kv.export_rows(0, ctx - U, U)
    assert np.array_equal(tail[0], kw) and np.array_equal(tail[2], vw)          # the tiling repeats bit for bit
    kd = np.empty((KVH, ctx + M, 256), np.float32); vd = np.empty_like(kd)
    for h in range(KVH):
        for kind, w, s, w2, s2, dst in ((0, kw, ks, kw2, ks2, kd), (1, vw, vs, vw2, vs2, vd)):
            g = np.full(U + M, h * 2 + kind, np.int32)
            words = np.zeros((U + M, 40), np.uint32)
            words[:U, :8 * kk] = w[h]; words[U:, :8 * kk] = w2[h]
            rows = oracle.tb_decode_rows(blob, g, words, np.concatenate([s[h], s2[h]]), np.zeros(U + M, np.uint32))
            dst[h, :ctx] = np.tile(rows[:U], (ctx // U, 1)); dst[h, ctx:] = rows[U:]
    expect = oracle.tb_attend_f64(kd, vd, q, ctx)
    assert_attn_close(dec1, expect[:1], f"decode kk={kk}")
    assert_attn_close(win, expect, f"window kk={kk}")
    assert_attn_close(win_tiles, expect, f"window on row tiles kk={kk}")
    assert np.abs(win.astype(np.float64) - expect).max() <= 2e-3                # the plain absolute bar at the measured size


def test_pass_wider_than_a_slice(native, oracle):
    """200 rows in one call: the encoder runs in tiles of 128 tokens, attention in 64-row slices, later rows see the keys
    of earlier rows of the same pass"""
    from tolerances import assert_attn_close
    blob = kvqp.synthetic(layers=1, kk=4, seed=33)
    ctx, M = 300, 200
    k, v = _kv_rows(34, ctx + M)
    k16, v16 = k[ctx:].astype(np.float16), v[ctx:].astype(np.float16)
    k[ctx:] = k16; v[ctx:] = v16
    q = np.random.default_rng(35).standard_normal((M, NH, 256)).astype(np.float16)
    with native.KvCache(head_dim=256, max_ctx=512, max_rows=256) as kv:
        kv.set_profile(blob)
        for p in range(0, ctx, 64):
            m = min(64, ctx - p)
            kv.append256_f32_host(0, k[p:p + m], v[p:p + m], p, rotate=False)
        out = kv.layer_call(0, q, k16, v16, ctx)
        kw, ks, vw, vs = kv.export_rows(0, 0, ctx + M)
    enc = _oracle_rows(oracle, blob, 0, k, v)
    for h in range(KVH):
        assert np.array_equal(kw[h], enc[0, h]["words"][:, :32]) and np.array_equal(vw[h], enc[1, h]["words"][:, :32]), h
        assert _same(ks[h], enc[0, h]["scale"]) and _same(vs[h], enc[1, h]["scale"])
    kd = np.stack([enc[0, h]["x"] for h in range(KVH)]); vd = np.stack([enc[1, h]["x"] for h in range(KVH)])
    assert_attn_close(out, oracle.tb_attend_f64(kd, vd, q, ctx), "200-row pass")


def test_engine_shaped_sequence_post_attend_unrotate(native, oracle):
    """the sequence a caller with the engine's head size runs on packed rows: yka_attn_post with rotation (norm, rotary,
    rotation, trellis encoder), attention over the rotated rows, outputs rotated back by the combiner (option key 4)"""
    from tolerances import assert_attn_close
    blob = kvqp.synthetic(layers=1, kk=5, seed=29)
    rng = np.random.default_rng(30)
    ctx, M, rd = 400, 4, 64
    n = ctx + M
    xq = rng.standard_normal((M, NH, 256)).astype(np.float32)
    xk = (rng.standard_normal((n, KVH, 256)) * 0.8).astype(np.float32); xk[:, :, [5, 77, 130, 201]] *= 6
    xv = rng.standard_normal((n, KVH, 256)).astype(np.float32)
    qw = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    kw_ = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    rope = oracle.rope_table(512, rd)
    zq = np.zeros((64, NH, 256), np.float32)
    with native.KvCache(head_dim=256, max_ctx=512) as kv:
        kv.set_profile(blob)
        kv.set_opt(4, 1)
        for p in range(0, ctx, 64):                              # cached rows: the same step, their Q rows are not needed
            m = min(64, ctx - p)
            kv.attn_post_host(0, zq[:m], xk[p:p + m], xv[p:p + m], p, qw, kw_, 1e-6, rope, rd, rotate=True)
        q16 = kv.attn_post_host(0, xq, xk[ctx:], xv[ctx:], ctx, qw, kw_, 1e-6, rope, rd, rotate=True)
        out = kv.layer_call(0, q16, None, None, ctx)
    # oracle: the post step row by row position, the encoder, fp64 attention in the rotated basis, inverse rotation
    k32 = np.empty((n, KVH, 256), np.float32); v32 = np.empty_like(k32)
    for p in range(0, n, 64):
        m = min(64, n - p)
        _, k32[p:p + m], v32[p:p + m] = oracle.attn_post256(np.zeros((m, NH, 256), np.float32), xk[p:p + m], xv[p:p + m], qw, kw_, 1e-6, rope, rd, p, 1)
    ref_q, _, _ = oracle.attn_post256(xq, xk[ctx:], xv[ctx:], qw, kw_, 1e-6, rope, rd, ctx, 1)
    assert np.array_equal(q16.view(np.uint16), ref_q)
    enc = _oracle_rows(oracle, blob, 0, k32, v32)
    kd = np.stack([enc[0, h]["x"] for h in range(KVH)]); vd = np.stack([enc[1, h]["x"] for h in range(KVH)])
    rotated = oracle.tb_attend_f64(kd, vd, ref_q, ctx)
    expect = oracle.kvx_rotate256(rotated.reshape(-1, 256).astype(np.float32), inverse=True).reshape(M, NH, 256)
    assert_attn_close(out, expect, "post -> encoder -> attention -> inverse rotation")
