#!/usr/bin/env python3
"""Writes the committed fixtures in this folder from the CPU oracle (oracle/).

The reference holds no vectors, known-answer tests or data files for the int4-KV attention path, so nothing here
comes from the reference: the fixtures freeze the oracle's outputs on small seeded inputs (after the oracle itself
has been pinned by tests/test_oracle_*.py), so that (i) a later change of the oracle is noticed and (ii) the GPU
tests can compare against committed data.

    python tests/golden/make_golden.py        # rewrites codec_v1.npz, attention_v1.npz, row256_v1.npz, post_v1.npz, post256_v1.npz and trellis_v1.npz
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import yko  # noqa: E402


def codec_fixture():
    rng = np.random.default_rng(20261125)
    x = rng.standard_normal((96, 128)).astype(np.float32)
    x[0] = 0.0
    x[1, :32] = 0.0
    x[2] *= 1e-7
    x[3] *= 6e-5
    x[4] *= 9000
    x[5, 7] = 65504.0
    x[6, :8] = [7, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5]
    x[6, 8:32] = 0
    x[7:40, ::9] *= 8
    x[40:] *= (10.0 ** rng.uniform(-5, 3, (56, 1))).astype(np.float32)
    x16 = x.astype(np.float16)
    codes, scales = yko.quant_rows(x16)
    y = yko.dequant_rows(codes, scales)
    np.savez_compressed(os.path.join(HERE, "codec_v1.npz"), x16=x16.view(np.uint16), codes=codes, scales=scales,
                        dequant_bits=y.view(np.uint32))


def attention_fixture():
    cases = {}
    for name, seed, ctx, M, depth in [("decode_ctx100", 11, 100, 1, None), ("window5_ctx70", 12, 70, 5, None),
                                      ("window6_depth", 13, 60, 6, [0, 1, 1, 2, 2, 3])]:
        q, k, v, kn, vn, ch = yko.make_inputs(seed, ctx, M)
        c = yko.Cache(512)
        c.append(k, v, 0)
        c.append(kn, vn, ctx)
        dep = None if depth is None else np.array(depth, np.uint8)
        o16, o32 = c.attend_f32(q, ctx, dep, want_f32=True)
        n = ctx + M
        cases.update({f"{name}.q": q.view(np.uint16), f"{name}.k_new": kn.view(np.uint16), f"{name}.v_new": vn.view(np.uint16),
                      f"{name}.kc": c.kc[:, :n], f"{name}.ks": c.ks[:, :n], f"{name}.vc": c.vc[:, :n], f"{name}.vs": c.vs[:, :n],
                      f"{name}.ctx": np.int32(ctx), f"{name}.depth": np.array([] if depth is None else depth, np.uint8),
                      f"{name}.out16": o16.view(np.uint16), f"{name}.out32": o32, f"{name}.outliers": ch})
    np.savez_compressed(os.path.join(HERE, "attention_v1.npz"), **cases)


def row256_fixture():
    """The reference's own 256-channel row format: rotation, flat int4 (MSB-first words, fp32 scale) and int8 rows."""
    rng = np.random.default_rng(20261126)
    x = (rng.standard_normal((24, 256)) * (10.0 ** rng.uniform(-3, 2, (24, 1)))).astype(np.float32)
    x[0] = 0.0
    x[1] = 0.0; x[1, 200] = -3.0
    x[2] = np.round(x[2] * 4)
    out = {"x": x}
    for mode in (0, 1):
        for rot in (0, 1):
            q8, words, scales, y = yko.kvx_probe256(x, mode, rot)
            tag = f"m{mode}r{rot}"
            out[tag + ".scales_bits"] = scales.view(np.uint32)
            out[tag + ".y_bits"] = y.view(np.uint32)
            if mode == 0:
                out[tag + ".q8"] = q8
            else:
                out[tag + ".words"] = words
    np.savez_compressed(os.path.join(HERE, "row256_v1.npz"), **out)


def post_fixture():
    """The step between the QKV projection and the cache: fp32 rows in, fp16 Q rows and int4 cache rows out."""
    rng = np.random.default_rng(20261127)
    M, rd, pos, ctx = 6, 32, 250, 512
    xq = (rng.standard_normal((M, 24, 128)) * 2).astype(np.float32)
    xk = (rng.standard_normal((M, 4, 128)) * 0.7).astype(np.float32)
    xk[:, :, [3, 40, 77, 120]] *= 8
    xv = rng.standard_normal((M, 4, 128)).astype(np.float32)
    xq[1] = 0; xk[1] = 0; xv[1] = 0
    qw = (rng.standard_normal(128) * 0.1).astype(np.float16).view(np.uint16)
    kw = (rng.standard_normal(128) * 0.1).astype(np.float16).view(np.uint16)
    rope = yko.rope_table(ctx, rd)
    out = {"xq": xq, "xk": xk, "xv": xv, "qw": qw, "kw": kw, "rope": rope, "rd": np.int32(rd), "pos": np.int32(pos),
           "eps": np.float32(1e-6), "ctx": np.int32(ctx)}
    for rot in (0, 1):
        q16, k16, v16 = yko.attn_post(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot)
        c = yko.Cache(ctx)
        c.append(k16, v16, pos)
        sl = slice(pos, pos + M)
        out.update({f"r{rot}.q16": q16, f"r{rot}.kc": c.kc[:, sl], f"r{rot}.ks": c.ks[:, sl], f"r{rot}.vc": c.vc[:, sl], f"r{rot}.vs": c.vs[:, sl]})
    np.savez_compressed(os.path.join(HERE, "post_v1.npz"), **out)


def post256_fixture():
    """The same step for 256-channel heads: fp32 rows in, fp16 Q rows and the words / fp32 scales of the cache rows out."""
    rng = np.random.default_rng(20261128)
    M, rd, pos, ctx = 4, 64, 252, 512
    xq = (rng.standard_normal((M, 24, 256)) * 2).astype(np.float32)
    xk = (rng.standard_normal((M, 4, 256)) * 0.7).astype(np.float32)
    xk[:, :, [5, 77, 130, 201]] *= 8
    xv = rng.standard_normal((M, 4, 256)).astype(np.float32)
    xq[1] = 0; xk[1] = 0; xv[1] = 0
    qw = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    kw = (rng.standard_normal(256) * 0.1).astype(np.float16).view(np.uint16)
    rope = yko.rope_table(ctx, rd)
    out = {"xq": xq, "xk": xk, "xv": xv, "qw": qw, "kw": kw, "rope": rope, "rd": np.int32(rd), "pos": np.int32(pos),
           "eps": np.float32(1e-6), "ctx": np.int32(ctx)}
    for rot in (0, 1):
        q16, k32, v32 = yko.attn_post256(xq, xk, xv, qw, kw, 1e-6, rope, rd, pos, rot)
        kw_ = np.empty((4, M, 32), np.uint32); vw_ = np.empty_like(kw_); ks_ = np.empty((4, M), np.float32); vs_ = np.empty_like(ks_)
        for h in range(4):
            kw_[h], ks_[h], _ = yko.flat4_encode256(k32[:, h])
            vw_[h], vs_[h], _ = yko.flat4_encode256(v32[:, h])
        out.update({f"r{rot}.q16": q16, f"r{rot}.kw": kw_, f"r{rot}.ks": ks_, f"r{rot}.vw": vw_, f"r{rot}.vs": vs_})
    np.savez_compressed(os.path.join(HERE, "post256_v1.npz"), **out)


def trellis_fixture():
    """Trellis-coded rows under two synthetic profiles (5 bits with mean rows and two directions; 4 bits plain): the blob,
    the rows, and what the oracle codes them to.  The blob is stored so that the fixture does not depend on the generator of
    synthetic profiles staying as it is."""
    from yasakani_amd import kvqp
    rng = np.random.default_rng(20261129)
    out = {}
    for name, blob in (("a", kvqp.synthetic(layers=1, kk=5, seed=41, mu=True, dirs=2, flat_groups=(6,))), ("b", kvqp.synthetic(layers=1, kk=4, seed=42))):
        n = 48
        y = (rng.standard_normal((n, 256)) * rng.uniform(0.1, 5, (n, 1))).astype(np.float32)
        y[:, [5, 77, 130, 201]] *= 8
        y[2] = 0
        grp = (np.arange(n) % 8).astype(np.int32); pos = np.arange(n, dtype=np.int32)
        enc = yko.tb_encode_rows(blob, grp, pos, y)
        out.update({f"{name}.blob": np.frombuffer(blob, np.uint8), f"{name}.y": y, f"{name}.grp": grp, f"{name}.pos": pos,
                    f"{name}.words": enc["words"], f"{name}.scale": enc["scale"], f"{name}.pc": enc["pc"], f"{name}.x": enc["x"],
                    f"{name}.best_mi": enc["best_mi"]})
    np.savez_compressed(os.path.join(HERE, "trellis_v1.npz"), **out)


if __name__ == "__main__":
    codec_fixture()
    attention_fixture()
    row256_fixture()
    post_fixture()
    post256_fixture()
    trellis_fixture()
    for f in ("codec_v1.npz", "attention_v1.npz", "row256_v1.npz", "post_v1.npz", "post256_v1.npz", "trellis_v1.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
