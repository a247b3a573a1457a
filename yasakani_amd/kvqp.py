"""Profile blobs of the trellis row codec ("KVQP" version 1), as the reference reads them (src/engine35.cpp:48-52,
src/kvq_fast.hpp:52-76, src/kvq_gpu.cuh:53-62,90-92): little-endian, a 96-byte header, then the scale multipliers, the
table records and the group records.

    header: "KVQP", u16 version 1, u16 header bytes 96, u32 total bytes, u16 @16 row length 256, u16 @18 layers,
            u16 @20 kv heads, u16 @22 tables, u16 @24 multipliers, u32 @28 groups = layers * kv heads * 2,
            u32 @32 offset of the fp32 multipliers, u32 @36 offset of the u32 table offsets, u32 @40 offset of the u32
            group offsets
    table:  u8 state bits 8, u8 0, u8 chunk length 64, u8 8, f32 gain, 4 bytes 0, 256 x i16 values (value = i16/256*gain)
    group:  u8 mode (0 trellis, 1 flat int4), u8 bits per element, u8 table, u8 guard position, u8 m (directions), u8 has_mu,
            2 bytes 0, [256 x fp16 mu], m x [256 x fp16 direction]

The reference's own profiles (kvq_u5.bin) ship with its model folders, not with its source; `synthetic` builds a blob of
the same layout with a Gaussian table so that the codec can be exercised without one."""
import struct

import numpy as np


def build(layers, kv_heads, multipliers, tables, groups):
    """tables: list of (gain, values int16[256]); groups: list (layers*kv_heads*2, order ((layer*kv_heads+kvh)*2+kind)) of
    dicts mode, kk, table, guard, mu (None | fp16[256]), dirs (list of fp16[256], at most 2)."""
    assert len(groups) == layers * kv_heads * 2 and 1 <= len(multipliers) <= 16
    body = bytearray(96)
    off_m = len(body)
    body += np.asarray(multipliers, "<f4").tobytes()
    off_t = len(body)
    body += bytes(4 * len(tables))
    off_g = len(body)
    body += bytes(4 * len(groups))
    for i, (gain, vals) in enumerate(tables):
        vals = np.asarray(vals)
        assert vals.shape == (256,) and np.abs(vals).max() <= 1100
        struct.pack_into("<I", body, off_t + 4 * i, len(body))
        body += struct.pack("<BBBBfI", 8, 0, 64, 8, float(gain), 0) + vals.astype("<i2").tobytes()
    for i, g in enumerate(groups):
        dirs = g.get("dirs") or []
        mu = g.get("mu")
        assert len(dirs) <= 2 and g["mode"] in (0, 1)
        struct.pack_into("<I", body, off_g + 4 * i, len(body))
        body += struct.pack("<BBBBBBH", g["mode"], g.get("kk", 4), g.get("table", 0), g.get("guard", 0), len(dirs), 1 if mu is not None else 0, 0)
        if mu is not None:
            body += np.asarray(mu, "<f2").tobytes()
        for d in dirs:
            body += np.asarray(d, "<f2").tobytes()
    body[0:4] = b"KVQP"
    struct.pack_into("<HHI", body, 4, 1, 96, len(body))
    struct.pack_into("<HHHHH", body, 16, 256, layers, kv_heads, len(tables), len(multipliers))
    struct.pack_into("<IIII", body, 28, len(groups), off_m, off_t, off_g)
    return bytes(body)


def gaussian_table(seed):
    """256 values: the 256-quantiles of N(0,1) x 256, assigned to states by a seeded permutation (neighbouring states of a
    trellis must not decode to neighbouring values)."""
    from statistics import NormalDist
    q = np.array([NormalDist().inv_cdf((i + 0.5) / 256) for i in range(256)])
    vals = np.rint(q * 256).astype(np.int16)
    return vals[np.random.default_rng(seed).permutation(256)]


def synthetic(layers=1, kv_heads=4, kk=5, seed=0, n_mult=9, mu=False, dirs=0, guard=0, flat_groups=()):
    """A blob of the production shape: every group trellis-coded with kk bits (those in flat_groups: flat int4)."""
    rng = np.random.default_rng(seed)
    mult = np.linspace(0.80, 1.25, n_mult).astype(np.float32)
    tables = [(1.0, gaussian_table(seed)), (0.97, gaussian_table(seed + 1))]
    groups = []
    for g in range(layers * kv_heads * 2):
        ds = []
        for _ in range(dirs):
            v = rng.standard_normal(256); ds.append((v / np.linalg.norm(v)).astype(np.float16))
        groups.append(dict(mode=1 if g in flat_groups else 0, kk=kk, table=g & 1, guard=guard,
                           mu=(rng.standard_normal(256) * 0.3).astype(np.float16) if mu else None, dirs=ds))
    return build(layers, kv_heads, mult, tables, groups)


def parse(blob):
    """header fields and the group records of a blob (no arrays)"""
    b = bytes(blob)
    if len(b) < 100 or b[:4] != b"KVQP" or struct.unpack_from("<H", b, 4)[0] != 1 or struct.unpack_from("<I", b, 8)[0] != len(b):
        raise ValueError("not a KVQP v1 blob")
    dim, layers, kvh, nt, nm = struct.unpack_from("<HHHHH", b, 16)
    ngrp, off_m, off_t, off_g = struct.unpack_from("<IIII", b, 28)
    groups = []
    for g in range(ngrp):
        go = struct.unpack_from("<I", b, off_g + 4 * g)[0]
        mode, kk, tix, guard, m, has_mu = struct.unpack_from("<BBBBBB", b, go)
        groups.append(dict(mode=mode, kk=kk, table=tix, guard=guard, m=m, has_mu=has_mu, offset=go))
    return dict(dim=dim, layers=layers, kv_heads=kvh, tables=nt, multipliers=list(np.frombuffer(b, "<f4", nm, off_m)), groups=groups)
