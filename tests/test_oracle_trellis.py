"""Pins the oracle's restatement of the trellis row codec (reference: src/kvq_gpu.cuh:51-147, src/kvq_fast.cuh:63-233,
src/kvq_attn.cuh:46-75) by what the mathematics fixes: exhaustive search over every path on short chunks, numpy bit
unpacking, the state recursion, fp64 forms of the projections and of the multiplier choice.  CPU only.

The tables are synthetic (the reference's profile blob is not in its repository): parity against a real profile is
unpinned, the algorithm is not."""
import itertools

import numpy as np
import pytest

from oracle import yko
from yasakani_amd import kvqp


def _brute(xi, ci, kk):
    """every field sequence of len(xi) elements: the minimum cost, and among equal costs the path whose state tuple read
    from the last element backwards is smallest (what 'smaller predecessor, smaller final state' selects)"""
    T = len(xi)
    best = None
    for fields in itertools.product(range(1 << kk), repeat=T):
        st, states, cost = 0, [], 0
        for t, f in enumerate(fields):
            st = ((st << kk) | f) & 255
            states.append(st)
            cost += (int(xi[t]) - int(ci[st])) ** 2
        key = (cost, tuple(reversed(states)))
        if best is None or key < best[0]:
            best = (key, states)
    return best[0][0], np.array(best[1], np.uint8)


@pytest.mark.parametrize("kk,T", [(3, 4), (4, 3), (5, 3)])
def test_viterbi_is_the_exhaustive_minimum(kk, T):
    rng = np.random.default_rng(kk * 10 + T)
    for trial in range(6):
        ci = rng.integers(-1100, 1101, 256).astype(np.int16)
        xi = rng.integers(-2048, 2049, T).astype(np.int32)
        st, cost = yko.tb_viterbi(xi, ci, kk)
        bc, bs = _brute(xi, ci, kk)
        assert cost == bc and np.array_equal(st, bs), (trial, cost, bc)


@pytest.mark.parametrize("kk,T", [(3, 4), (4, 3)])
def test_viterbi_tie_rules_on_tables_with_repeated_values(kk, T):
    rng = np.random.default_rng(77 + kk)
    for trial in range(6):
        ci = rng.choice(np.array([-300, -100, 100, 300], np.int16), 256)     # many states decode alike: many equal-cost paths
        xi = rng.choice(np.array([-200, 0, 200], np.int32), T)
        st, cost = yko.tb_viterbi(xi, ci, kk)
        bc, bs = _brute(xi, ci, kk)
        assert cost == bc and np.array_equal(st, bs), (trial, st, bs)


def test_viterbi_full_chunk_beats_greedy_and_random_paths_and_is_a_valid_path():
    rng = np.random.default_rng(5)
    ci = kvqp.gaussian_table(3)
    for kk in (3, 4, 5):
        xi = np.clip(np.rint(rng.standard_normal(64) * 256), -2048, 2048).astype(np.int32)
        st, cost = yko.tb_viterbi(xi, ci, kk)
        prev = 0
        for t in range(64):                                   # consecutive states share 8 - kk bits
            assert st[t] >> kk == prev & ((1 << (8 - kk)) - 1)
            prev = int(st[t])
        assert cost == int(((xi - ci[st].astype(np.int64)) ** 2).sum())
        g, gc = 0, 0
        for t in range(64):                                   # greedy: best next state at every step
            cand = [((g << kk) | f) & 255 for f in range(1 << kk)]
            g = min(cand, key=lambda s: (int(xi[t]) - int(ci[s])) ** 2)
            gc += (int(xi[t]) - int(ci[g])) ** 2
        assert cost <= gc
        for _ in range(50):
            f = rng.integers(0, 1 << kk, 64); s = 0; c = 0
            for t in range(64):
                s = ((s << kk) | int(f[t])) & 255; c += (int(xi[t]) - int(ci[s])) ** 2
            assert cost <= c


@pytest.mark.parametrize("kb", [3, 4, 5])
def test_pack_is_an_msb_first_bit_stream(kb):
    rng = np.random.default_rng(kb)
    fields = rng.integers(0, 1 << kb, 256).astype(np.uint8)
    w = yko.tb_pack(fields, kb)
    bits = np.unpackbits(w.astype(">u4").view(np.uint8))
    assert bits.size == 256 * kb
    got = np.zeros(256, np.int64)
    for j in range(kb):
        got = got * 2 + bits[j::kb][:256]
    assert np.array_equal(got, fields)


@pytest.mark.parametrize("kk,mu,dirs", [(5, False, 0), (4, False, 0), (3, False, 0), (5, True, 2), (4, True, 1)])
def test_decode_is_the_state_recursion_and_reproduces_the_encoders_row(kk, mu, dirs):
    blob = kvqp.synthetic(layers=1, kk=kk, seed=kk, mu=mu, dirs=dirs)
    assert yko.tb_check_blob(blob) == 0
    rng = np.random.default_rng(100 + kk)
    y = (rng.standard_normal((24, 256)) * rng.uniform(0.1, 4, (24, 1))).astype(np.float32)
    grp = np.arange(24) % 8
    enc = yko.tb_encode_rows(blob, grp, np.zeros(24, np.int32), y)
    assert enc["coded"].all()
    dec = yko.tb_decode_rows(blob, grp, enc["words"], enc["scale"], enc["pc"])
    assert np.array_equal(dec.view(np.uint32), enc["x"].view(np.uint32))
    # independent decode: unpack bits with numpy, run the state recursion per chunk of 64, look the table up
    P = kvqp.parse(blob)
    import struct
    b = bytes(blob)
    off_t = struct.unpack_from("<I", b, 36)[0]
    for i in range(24):
        G = P["groups"][grp[i]]
        to = struct.unpack_from("<I", b, off_t + 4 * G["table"])[0]
        gain = struct.unpack_from("<f", b, to + 4)[0]
        ci = np.frombuffer(b, "<i2", 256, to + 12)
        bits = np.unpackbits(enc["words"][i, :8 * kk].astype(">u4").view(np.uint8))
        f = np.zeros(256, np.int64)
        for j in range(kk):
            f = f * 2 + bits[j::kk][:256]
        st = np.zeros(256, np.int64); s = 0
        for e in range(256):
            s = (((0 if e % 64 == 0 else s) << kk) | int(f[e])) & 255
            st[e] = s
        x = (ci[st].astype(np.float32) * np.float32(1 / 256) * np.float32(gain)) * enc["scale"][i]
        go = G["offset"] + 8
        if G["has_mu"]:
            muv = np.frombuffer(b, "<f2", 256, go).astype(np.float32); go += 512
        c = np.array([enc["pc"][i] & 0xffff, enc["pc"][i] >> 16], np.uint16).view(np.float16).astype(np.float32)
        for j in range(G["m"]):
            x = x + c[j] * np.frombuffer(b, "<f2", 256, go + 512 * j).astype(np.float32)
        if G["has_mu"]:
            x = x + muv
        assert np.array_equal(x.view(np.uint32), dec[i].view(np.uint32)), i


def test_projections_rms_and_the_kept_multiplier_against_fp64():
    blob = kvqp.synthetic(layers=1, kk=5, seed=9, mu=True, dirs=2)
    P = kvqp.parse(blob)
    b = bytes(blob)
    rng = np.random.default_rng(8)
    y = (rng.standard_normal((12, 256)) * 1.7).astype(np.float32)
    grp = np.arange(12) % 8
    enc = yko.tb_encode_rows(blob, grp, np.zeros(12, np.int32), y)
    import struct
    off_t = struct.unpack_from("<I", b, 36)[0]
    for i in range(12):
        G = P["groups"][grp[i]]
        go = G["offset"] + 8
        mu = np.frombuffer(b, "<f2", 256, go).astype(np.float64)
        U = [np.frombuffer(b, "<f2", 256, go + 512 * (1 + j)).astype(np.float64) for j in range(2)]
        r = y[i].astype(np.float64) - mu
        cs = []
        for j in range(2):
            c = float(np.float16(r @ U[j])); cs.append(c); r = r - c * U[j]
        got_c = np.array([enc["pc"][i] & 0xffff, enc["pc"][i] >> 16], np.uint16).view(np.float16).astype(np.float64)
        assert np.allclose(got_c, cs, rtol=2e-3, atol=1e-4)               # one fp16 step where the fp32 sum sits on a tie
        rms = np.sqrt((r * r).mean())
        mults = np.array(P["multipliers"], np.float64)
        assert np.isclose(enc["scale"][i], rms * mults[enc["best_mi"][i]], rtol=1.5e-3)
        # the kept multiplier has the smallest reconstruction error among all of them (fp64 evaluation of every candidate)
        to = struct.unpack_from("<I", b, off_t + 4 * G["table"])[0]
        gain = struct.unpack_from("<f", b, to + 4)[0]
        ci = np.frombuffer(b, "<i2", 256, to + 12)
        r32 = r.astype(np.float32)
        errs = []
        for mval in mults:
            s = float(np.float16(np.float32(rms) * np.float32(mval)))
            xi = np.clip(np.rint(r32 / np.float32(s) * 256), -2048, 2048).astype(np.int32)
            st = np.concatenate([yko.tb_viterbi(xi[64 * c:64 * c + 64], ci, 5)[0] for c in range(4)])
            errs.append(((r - ci[st] / 256.0 * gain * s) ** 2).sum())
        assert errs[enc["best_mi"][i]] <= min(errs) * (1 + 1e-4)


def test_flat_groups_use_the_flat_row_quantizer_and_guard_rows_pass_through():
    blob = kvqp.synthetic(layers=1, kk=5, seed=2, guard=3, flat_groups=(1, 4))
    rng = np.random.default_rng(3)
    y = rng.standard_normal((8, 256)).astype(np.float32)
    enc = yko.tb_encode_rows(blob, np.arange(8), np.full(8, 3, np.int32), y)
    for g in (1, 4):
        words, scale, xq = yko.flat4_encode256(y[g:g + 1])
        assert np.array_equal(enc["words"][g, :32], words[0]) and enc["scale"][g] == scale[0]
        assert np.array_equal(enc["x"][g].view(np.uint32), xq[0].view(np.uint32))
    low = yko.tb_encode_rows(blob, np.arange(8), np.full(8, 2, np.int32), y)       # below the guard position
    assert not low["coded"].any() and np.array_equal(low["x"], y)
    out = yko.tb_encode_rows(blob, np.full(8, 99, np.int32), np.full(8, 5, np.int32), y)   # no such group
    assert not out["coded"].any() and np.array_equal(out["x"], y)


def test_blob_checks():
    blob = bytearray(kvqp.synthetic())
    assert yko.tb_check_blob(blob) == 0
    bad = bytearray(blob); bad[0] = ord("X")
    assert yko.tb_check_blob(bad) != 0
    assert yko.tb_check_blob(blob[:-1]) != 0
    P = kvqp.parse(blob)
    assert P["dim"] == 256 and len(P["groups"]) == 8 and P["groups"][0]["kk"] == 5
    assert yko.tb_group(blob, 5) == {k: P["groups"][5][k] for k in ("mode", "kk", "table", "guard", "m", "has_mu")}


def test_attention_over_decoded_rows_closed_forms():
    """tb_attend_f64 (textbook softmax(QK^T/16)V in fp64 on decoded rows): uniform V rows give that row; one dominant key
    gives its V row; a row sees exactly the keys up to its own position"""
    rng = np.random.default_rng(12)
    n, M = 40, 3
    k = rng.standard_normal((4, n, 256)).astype(np.float32)
    v = np.tile(rng.standard_normal((4, 1, 256)).astype(np.float32), (1, n, 1))
    q = rng.standard_normal((M, 24, 256)).astype(np.float16)
    out = yko.tb_attend_f64(k, v, q, n - M)
    for h in range(24):
        assert np.allclose(out[:, h], v[h // 6, 0], atol=1e-12)
    v = rng.standard_normal((4, n, 256)).astype(np.float32)
    k2 = k.copy(); k2[:, 7] = 0
    for h in range(4):
        k2[h, 7] = 50 * q[0, 6 * h].astype(np.float32) / np.linalg.norm(q[0, 6 * h].astype(np.float32))
    out = yko.tb_attend_f64(k2, v, q[:1], n - 1)
    for h in range(4):
        assert np.allclose(out[0, 6 * h], v[h, 7], atol=1e-6)
    # causal window: changing a key beyond a row's own position changes nothing for that row
    base = yko.tb_attend_f64(k, v, q, n - M)
    k3 = k.copy(); k3[:, n - 1] += 5
    moved = yko.tb_attend_f64(k3, v, q, n - M)
    assert np.array_equal(base[:M - 1], moved[:M - 1]) and not np.array_equal(base[M - 1], moved[M - 1])
