#!/usr/bin/env python3
"""Writes the committed fixtures in this folder from the CPU oracle (oracle/).

The reference holds no vectors, known-answer tests or data files for the int4-KV attention path, so nothing here
comes from the reference: the fixtures freeze the oracle's outputs on small seeded inputs (after the oracle itself
has been pinned by tests/test_oracle_*.py), so that (i) a later change of the oracle is noticed and (ii) the GPU
tests can compare against committed data.

    python tests/golden/make_golden.py        # rewrites codec_v1.npz and attention_v1.npz
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


if __name__ == "__main__":
    codec_fixture()
    attention_fixture()
    for f in ("codec_v1.npz", "attention_v1.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
