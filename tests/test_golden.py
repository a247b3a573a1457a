"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the pinned oracle).

CPU part: the oracle still reproduces them bit for bit.  GPU part: the HIP path reproduces the codec fixture bit for
bit and the attention fixtures within the attention bar, without running the oracle.
"""
import os

import numpy as np
import pytest

from tests.tolerances import assert_attn_close

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ("decode_ctx100", "window5_ctx70", "window6_depth")


def _load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def test_oracle_reproduces_codec_fixture(oracle):
    g = _load("codec_v1.npz")
    codes, scales = oracle.quant_rows(g["x16"].view(np.float16))
    assert (codes == g["codes"]).all() and (scales == g["scales"]).all()
    assert (oracle.dequant_rows(codes, scales).view(np.uint32) == g["dequant_bits"]).all()


@pytest.mark.parametrize("case", CASES)
def test_oracle_reproduces_attention_fixture(oracle, case):
    g = _load("attention_v1.npz")
    ctx = int(g[f"{case}.ctx"]); q = g[f"{case}.q"].view(np.float16); M = q.shape[0]
    c = oracle.Cache(512)
    n = ctx + M
    c.kc[:, :n], c.ks[:, :n], c.vc[:, :n], c.vs[:, :n] = g[f"{case}.kc"], g[f"{case}.ks"], g[f"{case}.vc"], g[f"{case}.vs"]
    dep = g[f"{case}.depth"]; dep = dep if dep.size else None
    o16 = c.attend_f32(q, ctx, dep)
    assert (o16.view(np.uint16) == g[f"{case}.out16"]).all()
    # the appended rows of the fixture are what quantizing k_new / v_new gives
    c2 = oracle.Cache(512)
    c2.append(g[f"{case}.k_new"].view(np.float16), g[f"{case}.v_new"].view(np.float16), ctx)
    assert (c2.kc[:, ctx:n] == g[f"{case}.kc"][:, ctx:n]).all() and (c2.vs[:, ctx:n] == g[f"{case}.vs"][:, ctx:n]).all()


@pytest.mark.gpu
def test_gpu_reproduces_codec_fixture(native):
    g = _load("codec_v1.npz")
    codes, scales, y = native.codec_probe(g["x16"].view(np.float16))
    assert (codes == g["codes"]).all() and (scales == g["scales"]).all()
    assert (y.view(np.uint32) == g["dequant_bits"]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_gpu_reproduces_attention_fixture(native, case):
    g = _load("attention_v1.npz")
    ctx = int(g[f"{case}.ctx"]); q = g[f"{case}.q"].view(np.float16); M = q.shape[0]
    dep = g[f"{case}.depth"]; dep = dep if dep.size else None
    with native.KvCache(max_ctx=512) as kv:
        kv.import_rows(0, 0, g[f"{case}.kc"][:, :ctx], g[f"{case}.ks"][:, :ctx], g[f"{case}.vc"][:, :ctx], g[f"{case}.vs"][:, :ctx])
        out = kv.layer_call(0, q, g[f"{case}.k_new"].view(np.float16), g[f"{case}.v_new"].view(np.float16), ctx, depth=dep)
        got = kv.export_rows(0, ctx, M)
    assert (got[0] == g[f"{case}.kc"][:, ctx:]).all() and (got[1] == g[f"{case}.ks"][:, ctx:]).all()
    assert (got[2] == g[f"{case}.vc"][:, ctx:]).all() and (got[3] == g[f"{case}.vs"][:, ctx:]).all()
    assert_attn_close(out, g[f"{case}.out32"], case)


# ---- the reference's own 256-channel row format, and the step between the QKV projection and the cache ----

def _check_row256(probe, g):
    for mode in (0, 1):
        for rot in (0, 1):
            q8, words, scales, y = probe(g["x"], mode, rot)
            tag = f"m{mode}r{rot}"
            assert (scales.view(np.uint32) == g[tag + ".scales_bits"]).all(), tag
            assert (y.view(np.uint32) == g[tag + ".y_bits"]).all(), tag
            if mode == 0:
                assert (q8 == g[tag + ".q8"]).all(), tag
            else:
                assert (words == g[tag + ".words"]).all(), tag


def test_oracle_reproduces_row256_fixture(oracle):
    _check_row256(oracle.kvx_probe256, _load("row256_v1.npz"))


@pytest.mark.gpu
def test_gpu_reproduces_row256_fixture(native):
    _check_row256(native.kvx256_probe, _load("row256_v1.npz"))


def test_oracle_reproduces_post_fixture(oracle):
    g = _load("post_v1.npz")
    M, pos, ctx = g["xq"].shape[0], int(g["pos"]), int(g["ctx"])
    for rot in (0, 1):
        q16, k16, v16 = oracle.attn_post(g["xq"], g["xk"], g["xv"], g["qw"], g["kw"], float(g["eps"]), g["rope"], int(g["rd"]), pos, rot)
        c = oracle.Cache(ctx)
        c.append(k16, v16, pos)
        sl = slice(pos, pos + M)
        assert (q16 == g[f"r{rot}.q16"]).all()
        for name, arr in (("kc", c.kc), ("ks", c.ks), ("vc", c.vc), ("vs", c.vs)):
            assert (arr[:, sl] == g[f"r{rot}.{name}"]).all(), name


@pytest.mark.gpu
def test_gpu_reproduces_post_fixture(native):
    g = _load("post_v1.npz")
    M, pos, ctx = g["xq"].shape[0], int(g["pos"]), int(g["ctx"])
    for rot in (0, 1):
        with native.KvCache(max_ctx=ctx) as kv:
            q16 = kv.attn_post_host(0, g["xq"], g["xk"], g["xv"], pos, g["qw"], g["kw"], float(g["eps"]), g["rope"], int(g["rd"]), rotate=bool(rot))
            got = kv.export_rows(0, pos, M)
        assert (q16.view(np.uint16) == g[f"r{rot}.q16"]).all()
        for arr, name in zip(got, ("kc", "ks", "vc", "vs")):
            assert (arr == g[f"r{rot}.{name}"]).all(), name


def test_oracle_reproduces_post256_fixture(oracle):
    g = _load("post256_v1.npz")
    pos = int(g["pos"])
    for rot in (0, 1):
        q16, k32, v32 = oracle.attn_post256(g["xq"], g["xk"], g["xv"], g["qw"], g["kw"], float(g["eps"]), g["rope"], int(g["rd"]), pos, rot)
        assert (q16 == g[f"r{rot}.q16"]).all()
        for h in range(4):
            w, s, _ = oracle.flat4_encode256(k32[:, h])
            assert (w == g[f"r{rot}.kw"][h]).all() and (s.view(np.uint32) == g[f"r{rot}.ks"][h].view(np.uint32)).all()
            w, s, _ = oracle.flat4_encode256(v32[:, h])
            assert (w == g[f"r{rot}.vw"][h]).all() and (s.view(np.uint32) == g[f"r{rot}.vs"][h].view(np.uint32)).all()


@pytest.mark.gpu
def test_gpu_reproduces_post256_fixture(native):
    g = _load("post256_v1.npz")
    M, pos, ctx = g["xq"].shape[0], int(g["pos"]), int(g["ctx"])
    for rot in (0, 1):
        with native.KvCache(head_dim=256, max_ctx=ctx) as kv:
            q16 = kv.attn_post_host(0, g["xq"], g["xk"], g["xv"], pos, g["qw"], g["kw"], float(g["eps"]), g["rope"], int(g["rd"]), rotate=bool(rot))
            kw, ks, vw, vs = kv.export_rows(0, pos, M)
        assert (q16.view(np.uint16) == g[f"r{rot}.q16"]).all()
        assert (kw == g[f"r{rot}.kw"]).all() and (vw == g[f"r{rot}.vw"]).all()
        assert (ks.view(np.uint32) == g[f"r{rot}.ks"].view(np.uint32)).all() and (vs.view(np.uint32) == g[f"r{rot}.vs"].view(np.uint32)).all()


def _check_trellis(code, g, name):
    enc = code(g[f"{name}.blob"].tobytes(), g[f"{name}.grp"], g[f"{name}.pos"], g[f"{name}.y"])
    assert (enc["words"][:, :40] == g[f"{name}.words"][:, :40]).all()
    assert (enc["scale"].view(np.uint32) == g[f"{name}.scale"].view(np.uint32)).all() and (enc["pc"] == g[f"{name}.pc"]).all()
    assert (enc["x"].view(np.uint32) == g[f"{name}.x"].view(np.uint32)).all()
    return enc


@pytest.mark.parametrize("name", ["a", "b"])
def test_oracle_reproduces_trellis_fixture(oracle, name):
    enc = _check_trellis(lambda b, grp, pos, y: oracle.tb_encode_rows(b, grp, pos, y), _load("trellis_v1.npz"), name)
    assert (enc["best_mi"] == _load("trellis_v1.npz")[f"{name}.best_mi"]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["a", "b"])
def test_gpu_reproduces_trellis_fixture(native, name):
    g = _load("trellis_v1.npz")
    enc = _check_trellis(lambda b, grp, pos, y: native.tb_pack_unpack(b, y, grp, pos), g, name)
    assert (enc["dec"].view(np.uint32) == g[f"{name}.x"].view(np.uint32)).all()
