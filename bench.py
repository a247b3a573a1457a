#!/usr/bin/env python3
"""Benchmark of the int4-KV GQA attention path on one MI355X.

A step is one layer call (quantize-on-append of the window's new K/V rows + attention over the cache + split
combine) of the headline workload: a 64-row verify window at 32768 cached tokens, 24 query / 4 KV heads, head_dim 128,
int4 group-32 KV.  Steps rotate over `--layers` distinct KV containers (default 32 x 18.9 MB = 604 MB) so that the
256 MB Infinity Cache cannot hold the working set; they are issued as replays of a captured pass, the way the
reference engine replays its passes from graphs.  Inputs are synthetic (seeded normal values, 4 outlier channels of
K scaled x8) and are resident in HBM before the timed region.

Prints one JSON line: value = algorithmic bytes of a layer call / mean time per call (effective KV GB/s).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

NH, KVH, D = 24, 4, 128
TOKEN_BYTES = KVH * 2 * (D // 2 + 2 * (D // 32))      # 576 B per cached token per layer (codes + fp16 group scales)
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch of the dominant kernel from two `rocprofv3 --pmc` runs (FETCH_SIZE x 2.00 + WRITE_SIZE x 1.00,
# factors from a 256 MiB copy in the same runs).  A cited constant, not something this run measures: each entry names
# the summary it was taken from, and the JSON line carries that name so that a stale figure can be told from a fresh one.
# Keyed by (rows, ctx); any other workload reports null.
MEASURED_TRAFFIC = {
    (64, 32768): (32.3e6, "profiles/attend_wide_kernel_verify64_ctx32768.md"),      # 23.5 MB read + 8.8 MB written
    (8, 32768): (22.8e6, "profiles/attend_mid_kernel_windows_ctx32768.md"),         # 19.6 MB read + 3.2 MB written
    (4, 32768): (20.9e6, "profiles/attend_mid_kernel_windows_ctx32768.md"),         # 19.3 MB read + 1.6 MB written
    (1, 32768): (19.7e6, "profiles/attend_narrow_kernel_decode_ctx32768.md"),       # 19.3 MB read + 0.4 MB written
}


def algorithmic_bytes(ctx, M):
    """KV stream + the window's rows written and read back + fp16 K/V in + Q in + out."""
    return ctx * TOKEN_BYTES + 2 * M * TOKEN_BYTES + M * KVH * 2 * D * 2 + 2 * M * NH * D * 2


def algorithmic_flops(ctx, M):
    """4 * rows * head_dim * keys, rows = M * 24, keys of row t = ctx + t + 1."""
    keys = sum(ctx + t + 1 for t in range(M))
    return 4.0 * NH * D * keys


def synth(seed, ctx, M):
    """Seeded inputs: Q [M,24,128]; K/V [ctx+M,4,128] with 4 fixed channels of K scaled x8; fp16."""
    rng = np.random.default_rng(seed)
    ch = rng.choice(D, 4, replace=False)
    q = rng.standard_normal((M, NH, D), dtype=np.float32).astype(np.float16)
    k = rng.standard_normal((ctx + M, KVH, D), dtype=np.float32)
    k[:, :, ch] *= 8.0
    v = rng.standard_normal((ctx + M, KVH, D), dtype=np.float32)
    return q, k.astype(np.float16), v.astype(np.float16)


def fill_cache(kv, k, v, ctx, chunk=4096):
    for p in range(0, ctx, chunk):
        n = min(chunk, ctx - p)
        kv.append_host(0, k[p:p + n], v[p:p + n], p)
    kv.replicate_layer(0)


def timed_passes(torch, kv, layers, q, kn, vn, ctx, M, steps, warmup, issue="graph", condition_ms=0.0):
    """Exactly `steps` layer calls, issued the same way whatever `steps` is.  issue = "graph": replays of captured passes
    that walk the containers in order (full sweeps over all of them, then one pass over the first steps % L), the way the
    reference engine replays its passes; issue = "eager": one yka_append_attend call per step on the same stream (a
    window of 16+ rows keeps the GPU busier than the host needs to issue the next call, and a short timed region does
    not carry the start-up latency of a graph launch).  Before the timed region every container is swept once and
    `warmup` further calls run.  Timed with events on the stream the work is launched on; the host clock around the
    same region is returned beside it."""
    dev = torch.device("cuda:0")
    dq = torch.from_numpy(q.view(np.int16)).to(dev)
    dk = torch.from_numpy(kn.view(np.int16)).to(dev)
    dv = torch.from_numpy(vn.view(np.int16)).to(dev)
    dout = torch.zeros_like(dq)
    dpos = torch.tensor([ctx], dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream().cuda_stream
    L = len(layers)

    def capture(ls):
        return kv.capture_pass(ls, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), M, dpos.data_ptr(), dout.data_ptr())

    sweep = capture(layers)
    passes = {L: sweep}

    def run(n):
        if issue == "eager":
            for i in range(n):
                kv.append_attend(layers[i % L], dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), M, dpos.data_ptr(), dout.data_ptr(), None, stream)
            return
        for _ in range(n // L):
            sweep.launch(stream)
        if n % L:
            if n % L not in passes:
                passes[n % L] = capture(layers[: n % L])
            passes[n % L].launch(stream)

    run(L)                                   # every container once
    # the GPU's power management takes tens of milliseconds of load to settle on its sustained clocks: a timed region of
    # a millisecond right after start-up measures the ramp, not the kernel (59 against 52 us per layer call here).  The
    # same sweeps are therefore replayed, untimed, for `condition_ms` before the warm-up steps.
    t_c = time.perf_counter()
    while (time.perf_counter() - t_c) * 1e3 < condition_ms:
        run(L)
        torch.cuda.synchronize()
    run(warmup)
    run(steps % L)                           # captures the remainder pass outside the timed region
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    run(steps)
    e1.record()
    torch.cuda.synchronize()
    host_dt = time.perf_counter() - t0
    dt = e0.elapsed_time(e1) * 1e-3
    out = dout.cpu().numpy().view(np.float16)
    for p in passes.values():
        p.close()
    return dt, host_dt, out


def small_decode(native, ctx=4096, L=128):
    """Decode on 4,096 cached tokens, rotating over 128 containers (302 MB, more than the Infinity Cache holds)."""
    q, k, v = synth(4096, ctx, 1)
    kv = native.KvCache(n_layers=L, max_ctx=ctx + 256, max_rows=64)
    fill_cache(kv, k, v, ctx)
    ms, _ = kv.bench(q[:1], k[ctx:ctx + 1], v[ctx:ctx + 1], ctx, mode=0, use_graph=True, reps=20)
    us = float(np.median(ms)) * 1e3 / L
    ms2, _ = kv.bench(q[:1], None, None, ctx, mode=2, use_graph=True, reps=20)
    by = algorithmic_bytes(ctx, 1)
    kv.close()
    return {"us_per_layer": us, "kernel_us": float(np.median(ms2)) * 1e3 / L, "value_GBs": by / (us * 1e-6) / 1e9,
            "hbm_peak_frac": by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}


def r256_figures(native, ctx=32768, L=16):
    """The reference's own rows (head_dim 256, one fp32 scale per row): 1,056 B per token per layer, 16 containers of
    34.6 MB.  One layer call = append + attention (decode: row tiles of 2 tokens; windows: 128-row workgroups) + combine."""
    rng = np.random.default_rng(256)
    D2 = 256
    k = rng.standard_normal((4096 + 64, KVH, D2)).astype(np.float16)
    v = rng.standard_normal((4096 + 64, KVH, D2)).astype(np.float16)
    q = rng.standard_normal((64, NH, D2)).astype(np.float16)
    kv = native.KvCache(n_layers=L, head_dim=D2, max_ctx=ctx + 256, max_rows=64)
    for p in range(0, ctx, 64):                       # 4096 distinct rows tiled over the context
        s0 = p % 4096
        kv.append_host(0, k[s0:s0 + 64], v[s0:s0 + 64], p)
    kv.replicate_layer(0)
    out = {}
    token_bytes = KVH * 2 * (128 + 4)
    for rows in (1, 16, 64):
        ms, _ = kv.bench(q[:rows], k[4096:4096 + rows], v[4096:4096 + rows], ctx, mode=0, use_graph=True, reps=10)
        us = float(np.median(ms)) * 1e3 / L
        ms2, _ = kv.bench(q[:rows], None, None, ctx, mode=2, use_graph=True, reps=10)
        k_us = float(np.median(ms2)) * 1e3 / L
        by = ctx * token_bytes + rows * (2 * token_bytes + 2 * KVH * D2 * 2 + 2 * NH * D2 * 2)
        out[f"rows_{rows}"] = {"us_per_layer": us, "kernel_us": k_us, "value_GBs": by / (us * 1e-6) / 1e9,
                               "kernel_hbm_frac": by / (k_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                               "kernel_tflops": 4.0 * rows * NH * D2 * ctx / (k_us * 1e-6) / 1e12}
    kv.close()
    return out


def trellis_figures(native, ctx=32768, L=16, bits=5, torch=None):
    """Trellis-coded rows (the reference's KV5 / KV4 packed streams) under a synthetic profile of the production shape:
    4 x 2 x (32 * bits + 4) bytes per token per layer.  One layer call = trellis encoder for the new rows (two launches) +
    attention on row tiles of 2 tokens + combine; `encode_us` is what the encoder adds to a layer call."""
    from yasakani_amd import kvqp
    rng = np.random.default_rng(500 + bits)
    D2 = 256
    k = rng.standard_normal((4096 + 64, KVH, D2)).astype(np.float16)
    v = rng.standard_normal((4096 + 64, KVH, D2)).astype(np.float16)
    q = rng.standard_normal((64, NH, D2)).astype(np.float16)
    kv = native.KvCache(n_layers=L, head_dim=D2, max_ctx=ctx + 256, max_rows=64)
    kv.set_profile(kvqp.synthetic(layers=L, kk=bits, seed=7))
    for p in range(0, ctx, 64):                       # 4096 distinct rows tiled over the context
        s0 = p % 4096
        kv.append_host(0, k[s0:s0 + 64], v[s0:s0 + 64], p)
    kv.replicate_layer(0)                             # the synthetic profile gives every layer the same tables
    out = {}
    token_bytes = KVH * 2 * (32 * bits + 4)
    for rows in (1, 16, 64):
        ms, _ = kv.bench(q[:rows], k[4096:4096 + rows], v[4096:4096 + rows], ctx, mode=0, use_graph=True, reps=10)
        us = float(np.median(ms)) * 1e3 / L
        ms1, _ = kv.bench(q[:rows], None, None, ctx, mode=1, use_graph=True, reps=10)
        ms2, _ = kv.bench(q[:rows], None, None, ctx, mode=2, use_graph=True, reps=10)
        k_us = float(np.median(ms2)) * 1e3 / L
        by = ctx * token_bytes + rows * (2 * token_bytes + 2 * KVH * D2 * 2 + 2 * NH * D2 * 2)
        out[f"rows_{rows}"] = {"us_per_layer": us, "encode_us": us - float(np.median(ms1)) * 1e3 / L, "kernel_us": k_us,
                               "value_GBs": by / (us * 1e-6) / 1e9, "kernel_hbm_frac": by / (k_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                               "kernel_tflops": 4.0 * rows * NH * D2 * ctx / (k_us * 1e-6) / 1e12}
    if torch is not None:
        # batched decode: the containers as streams of profile layer 0, one row per stream (encoder + attention + combine)
        kv.set_opt(6, 0)
        out["batched_decode"] = batched_decode(torch, native, kv, ctx, L, k[4096:4097], v[4096:4097], q[:1], calls=100,
                                               row_bytes=ctx * token_bytes + 2 * token_bytes + 2 * KVH * D2 * 2 + 2 * NH * D2 * 2)
    kv.close()
    return out


def prefill_chunk(native, reps=5, opts=()):
    """A 2048-row prefill chunk on 131072 cached tokens: one append launch, then two 1024-token slices through the wide
    kernel (128 rows per workgroup) and their combiner launches.  4 containers x 76.7 MB."""
    ctx, M, L = 131072, 2048, 4
    q, k, v = synth(31, ctx, M)
    kv = native.KvCache(n_layers=L, max_ctx=ctx + M, max_rows=M)
    for key, val in opts:
        kv.set_opt(key, val)
    fill_cache(kv, k, v, ctx, chunk=16384)
    ms, _ = kv.bench(q, k[ctx:], v[ctx:], ctx, mode=0, use_graph=True, reps=reps)
    us = float(np.median(ms)) * 1e3 / L
    keys = sum(ctx + t + 1 for t in range(M))
    fl = 4.0 * NH * D * keys
    kv.close()
    return {"us_per_layer": us, "tflops": fl / (us * 1e-6) / 1e12, "mfma_peak_frac": fl / (us * 1e-6) / 1e12 / MFMA_F16_PEAK_TFLOPS}


def sweep(native, which=("verify", "decode", "paged", "prefill"), reps=8, out=sys.stdout):
    """Launch-geometry sweep: every workload below is timed as whole layer calls (append + attention + combine, replayed
    from a graph over all containers of the handle, median of `reps` sweeps) under each value of the option keys that
    shape its grid.  Key 0 / value 0 is the library's own choice.  Prints a table; returns the rows.  Any error ends the
    sweep at once (the exception propagates): nothing is retried."""
    rows_out = []

    warmed = set()

    def timed(kv, L, q, kn, vn, ctx, opts):
        if id(kv) not in warmed:                             # the first sweeps on a fresh handle run at ramping clocks
            warmed.add(id(kv))
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.2:
                kv.bench(q, kn, vn, ctx, mode=0, use_graph=True, reps=reps)
        for key, val in opts:
            kv.set_opt(key, val)
        ms, _ = kv.bench(q, kn, vn, ctx, mode=0, use_graph=True, reps=reps)
        for key, _ in opts:
            kv.set_opt(key, 0 if key != 8 else 10)           # back to the defaults
        return float(np.median(ms)) * 1e3 / L

    def emit(workload, opts, us, note=""):
        label = " ".join(f"{k}={v}" for k, v in opts) or "defaults"
        rows_out.append({"workload": workload, "options": label, "us_per_layer": us, "note": note})
        print(f"| {workload} | {label} | {us:.2f} | {note} |", file=out, flush=True)

    print("| workload | option keys | us per layer call | note |\n|---|---|---|---|", file=out, flush=True)
    if "verify" in which or "decode" in which:
        ctx, L = 32768, 32
        q, k, v = synth(2026, ctx, 64)
        kv = native.KvCache(n_layers=L, max_ctx=((ctx + 64 + 255) // 256) * 256, max_rows=64)
        fill_cache(kv, k, v, ctx)
        kn, vn = k[ctx:], v[ctx:]
        if "verify" in which:
            for M in (4, 8, 16, 32, 64):
                name = f"verify-{M} at 32768"
                emit(name, (), timed(kv, L, q[:M], kn[:M], vn[:M], ctx, ()))
                if M <= 16:
                    for S in (0, 8, 16, 32, 64):
                        emit(name, ((8, 16), (9, S)), timed(kv, L, q[:M], kn[:M], vn[:M], ctx, ((8, 16), (9, S))), "mid kernel")
                for S in (0, 2, 3, 4, 5, 6, 8, 10, 12, 16, 21, 32, 64):
                    emit(name, ((8, 0), (2, S)), timed(kv, L, q[:M], kn[:M], vn[:M], ctx, ((8, 0), (2, S))), "wide kernel")
        if "decode" in which:
            for M in (1, 2):
                for pos in (4096, 32768):
                    name = f"decode ({M} row{'s' if M > 1 else ''}) at {pos}"
                    for hint in ((0, pos) if pos < ctx else (0,)):
                        for S in (0, 8, 16, 32, 48, 64, 96, 128, 192, 256):
                            for fuse in (0, 1):
                                opts = ((5, hint), (1, S), (7, fuse))
                                emit(name, opts, timed(kv, L, q[:M], kn[:M], vn[:M], pos, opts), "32 containers of 32768 tokens; 4096: the first 4096 of each")
        kv.close()
    if "paged" in which:
        ctx, L = 262144, 3
        q, k, v = synth(32, ctx, 64)
        kv = native.KvCache(n_layers=L, max_ctx=ctx + 256, max_rows=64, paged=True)
        kv.set_page_table(np.random.default_rng(32).permutation((ctx + 256) // 256).astype(np.int32))
        fill_cache(kv, k, v, ctx, chunk=16384)
        for S in (0, 64, 96, 128, 192, 256):
            emit("decode at 262144, shuffled pages", ((1, S),), timed(kv, L, q[:1], k[ctx:ctx + 1], v[ctx:ctx + 1], ctx, ((1, S),)))
        for S in (0, 8, 12, 16, 21, 32, 42, 64):
            emit("verify-64 at 262144, shuffled pages", ((2, S),), timed(kv, L, q, k[ctx:], v[ctx:], ctx, ((2, S),)))
        kv.close()
    if "prefill" in which:
        ctx, M, L = 131072, 2048, 4
        q, k, v = synth(31, ctx, M)
        kv = native.KvCache(n_layers=L, max_ctx=ctx + M, max_rows=M)
        fill_cache(kv, k, v, ctx, chunk=16384)
        for slice_len in (0, 512, 683, 1024, 1366, 2048):
            for S in (0, 1, 2, 3, 4, 6, 8):
                if slice_len * S > 4096 or (slice_len == 0 and 1024 * S > 4096):
                    continue                                  # more (token, split) pairs than the partial workspace holds
                opts = ((10, slice_len), (2, S))
                emit("prefill chunk 2048 rows at 131072", opts, timed(kv, L, q, k[ctx:], v[ctx:], ctx, opts))
        kv.close()
    return rows_out


def big_configs(native):
    """Secondary figures for the two large configurations: the prefill chunk above and decode / verify-64 on 262144 tokens
    in shuffled 256-token pages."""
    out = {"prefill_2048_at_131072": prefill_chunk(native)}
    # 262144 tokens, shuffled pages: 3 containers x 151 MB
    ctx, L = 262144, 3
    q, k, v = synth(32, ctx, 64)
    kv = native.KvCache(n_layers=L, max_ctx=ctx + 256, max_rows=64, paged=True)
    kv.set_page_table(np.random.default_rng(32).permutation((ctx + 256) // 256).astype(np.int32))
    fill_cache(kv, k, v, ctx, chunk=16384)
    for rows in (1, 64):
        ms, _ = kv.bench(q[:rows], k[ctx:ctx + rows], v[ctx:ctx + rows], ctx, mode=0, use_graph=True, reps=10)
        us = float(np.median(ms)) * 1e3 / L
        by = algorithmic_bytes(ctx, rows)
        out[f"paged_262144_rows_{rows}"] = {"us_per_layer": us, "value_GBs": by / (us * 1e-6) / 1e9,
                                            "hbm_peak_frac": by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                                            "tflops": algorithmic_flops(ctx, rows) / (us * 1e-6) / 1e12}
    kv.close()
    return out


def batched_decode(torch, native, kv, ctx, L, k_new, v_new, q, calls=200, row_bytes=None):
    """Multi-stream passes on the containers already filled for the headline run: one row per stream, B streams at `ctx`
    cached tokens each (one pass = append + attention + combine for all B rows; B x 18.9 MB of KV)."""
    dev = torch.device("cuda:0")
    out = {}
    stream = torch.cuda.current_stream().cuda_stream
    for B in (8, 16, 32):
        if B > L:
            continue
        rep = (B + q.shape[0] - 1) // q.shape[0]
        dq = torch.from_numpy(np.tile(q, (rep, 1, 1))[:B].view(np.int16).copy()).to(dev)
        dk = torch.from_numpy(np.tile(k_new, (rep, 1, 1))[:B].view(np.int16).copy()).to(dev)
        dv = torch.from_numpy(np.tile(v_new, (rep, 1, 1))[:B].view(np.int16).copy()).to(dev)
        dout = torch.zeros_like(dq)
        dpos = torch.full((B,), ctx, dtype=torch.int32, device=dev)
        # consecutive passes take different groups of B containers, so that all L containers (more than the 256 MB
        # Infinity Cache holds) are streamed before any is read again
        groups = [torch.arange(g * B, (g + 1) * B, dtype=torch.int32, device=dev) for g in range(L // B)]
        fn = lambda i: kv.append_attend_ms(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, dpos.data_ptr(),
                                           groups[i % len(groups)].data_ptr(), dout.data_ptr(), stream)
        for i in range(10):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(calls):
            fn(i)
        e1.record(); torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / calls
        by = B * (row_bytes if row_bytes else algorithmic_bytes(ctx, 1))
        out[f"streams_{B}"] = {"us_per_pass": us, "us_per_row": us / B, "value_GBs": by / (us * 1e-6) / 1e9,
                               "hbm_peak_frac": by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
    return out


def append_vs_post(torch, native, kv, ctx, rows_list=(1, 64), calls=400):
    """Eager launches on torch's stream: plain quantize-on-append of fp16 rows against the fused norm + rotary + rotation +
    quantize step fed with the projection's fp32 rows (one launch each; us per call, launch cost included)."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(7)
    out = {}
    stream = torch.cuda.current_stream().cuda_stream
    for M in rows_list:
        xq = torch.randn(M, NH, D, generator=g).to(dev); xk = torch.randn(M, KVH, D, generator=g).to(dev)
        xv = torch.randn(M, KVH, D, generator=g).to(dev)
        k16 = xk.half(); v16 = xv.half()
        w = (torch.randn(D, generator=g) * 0.1).half().to(dev)
        rd = 32
        f = torch.arange(ctx + M, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(rd // 2, dtype=torch.float64) / rd))[None, :]
        rope = torch.stack([torch.cos(f), torch.sin(f)], dim=-1).float().contiguous().to(dev)
        q16 = torch.empty(M, NH, D, dtype=torch.float16, device=dev)
        dpos = torch.tensor([ctx], dtype=torch.int32, device=dev)
        P = native.PostParams(w.data_ptr(), w.data_ptr(), 1e-6, rope.data_ptr(), rd, ctx + M, 1)
        res = {}
        for name, fn in (("append", lambda l: kv.append(l, k16.data_ptr(), v16.data_ptr(), M, dpos.data_ptr(), stream)),
                         ("post", lambda l: kv.attn_post(l, xq.data_ptr(), xk.data_ptr(), xv.data_ptr(), M, dpos.data_ptr(), P, q16.data_ptr(), stream))):
            for i in range(20):
                fn(i % kv.cfg.n_layers)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(calls):
                fn(i % kv.cfg.n_layers)
            e1.record(); torch.cuda.synchronize()
            res[name + "_us"] = e0.elapsed_time(e1) * 1e3 / calls
        res["post_bytes"] = M * (NH + 2 * KVH) * D * 4 + M * NH * D * 2 + M * TOKEN_BYTES
        out[f"rows_{M}"] = res
    return out


def cpu_baseline(kv, q, ctx, M, budget_s=10.0):
    """The CPU oracle on the same quantized cache: the reference's token-streaming split-KV loop restated in C, its inner
    loops written so that the compiler vectorises them (AVX2), parallel over (KV head x split) with OpenMP.  Bounded
    sample: whole layer calls are repeated until about `budget_s` seconds of CPU work are spent.  Beside the headline
    figure (all threads) the same call is timed on one thread and on the two decode configurations."""
    from oracle import yko
    threads = min(16, os.cpu_count() or 1)
    oc = yko.Cache(kv.max_ctx)
    n = ctx + M
    oc.kc[:, :n], oc.ks[:, :n], oc.vc[:, :n], oc.vs[:, :n] = kv.export_rows(0, 0, n)

    def sample(qq, pos, thr, budget, least=3):
        calls, t0 = 0, time.perf_counter()
        while True:
            r = oc.attend_f32(qq, pos, threads=thr)
            calls += 1
            el = time.perf_counter() - t0
            if el > budget and calls >= least:
                return el / calls, calls, el, r

    def sample_scalar(qq, pos, budget):
        calls, t0 = 0, time.perf_counter()
        while True:
            oc.attend_f32(qq, pos, threads=1, scalar_build=True)
            calls += 1
            el = time.perf_counter() - t0
            if el > budget:
                return el / calls, calls, el

    per_call, calls, el, ref16 = sample(q, ctx, threads, budget_s)
    base = {"value": algorithmic_bytes(ctx, M) / per_call / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "us_per_layer": per_call * 1e6, "build": yko.BUILD_FLAGS,
            "sample": f"{calls} whole layer calls (attention + combine, no append) of the same workload, {el:.1f} s"}
    other = {}
    one, c1, e1, _ = sample(q, ctx, 1, 3.0, least=1)
    other["headline_one_thread"] = {"us_per_layer": one * 1e6, "value_GBs": algorithmic_bytes(ctx, M) / one / 1e9, "cores": 1,
                                    "build": yko.BUILD_FLAGS, "sample": f"{c1} calls, {e1:.1f} s"}
    # the plain scalar build of the same sources on one thread: what a straightforward CPU port of the path does
    sc, cs, es = sample_scalar(q, ctx, 3.0)
    other["headline_scalar_build_one_thread"] = {"us_per_layer": sc * 1e6, "value_GBs": algorithmic_bytes(ctx, M) / sc / 1e9, "cores": 1,
                                                 "build": yko.BUILD_FLAGS_SCALAR, "sample": f"{cs} calls, {es:.1f} s"}
    sd, cd, ed = sample_scalar(q[:1], min(32768, ctx), 1.0)
    other["decode_32768_scalar_build_one_thread"] = {"us_per_layer": sd * 1e6, "value_GBs": algorithmic_bytes(min(32768, ctx), 1) / sd / 1e9,
                                                     "cores": 1, "build": yko.BUILD_FLAGS_SCALAR, "sample": f"{cd} calls, {ed:.1f} s"}
    for name, pos in (("decode_4096", min(4096, ctx)), ("decode_32768", min(32768, ctx))):
        for thr in (threads, 1):
            t, c, e, _ = sample(q[:1], pos, thr, 1.0)
            other[f"{name}_{thr}_threads"] = {"us_per_layer": t * 1e6, "value_GBs": algorithmic_bytes(pos, 1) / t / 1e9, "cores": thr,
                                              "sample": f"{c} calls, {e:.1f} s"}
    base["other_configs"] = other
    return base, ref16


def machine_figures(native):
    """What this GPU sustains on fixed instruction mixes (yka_machine_probe): dense fp16 MFMA rate, streaming read rate,
    and how far vector instructions hide behind MFMAs of the same wave.  The roofline stays priced at the published
    peaks; these are the ceilings a kernel can actually reach on this box."""
    it = 4000
    out = {}
    for blocks, name in ((256, "one_wave_per_simd"), (512, "two_waves_per_simd")):
        r = native.machine_probe(0, 0, it, blocks, 256)
        out[f"mfma_f16_32x32x16_tflops_{name}"] = blocks * 4 * it * 4 * 32768.0 / (r["ms"] * 1e-3) / 1e12
        out[f"shader_mhz_under_mfma_{name}"] = r.get("shader_mhz")
    r0 = native.machine_probe(0, 0, it, 256, 256)
    r6 = native.machine_probe(0, 6, it, 256, 256)
    out["cycles_per_mfma_alone"] = r0["cycles"] / (it * 4)
    out["cycles_per_mfma_with_6_fma_behind_it"] = r6["cycles"] / (it * 4)
    rf = native.machine_probe(2, 8, it, 256, 256)
    out["cycles_per_v_fma_f32_one_wave"] = rf["cycles"] / (it * 32)
    # one wave of MFMAs and one wave of packed-fp16 multiplies on every SIMD: how far the two pipes run side by side
    rp = native.machine_probe(2, 1, it, 256, 256)
    rx = native.machine_probe(5, 1, it, 256, 512)
    out["cycles_per_v_pk_mul_f16_one_wave"] = rp["cycles"] / (it * 32)
    out["cycles_per_v_pk_mul_f16_beside_an_mfma_wave"] = rx["cycles_b"] / (max(1, it * 2 // 3) * 32)
    out["cycles_per_mfma_beside_a_vector_wave"] = rx["cycles"] / (it * 4)
    for nt in (0, 1):
        r = native.machine_probe(4, nt, 2048, 16384, 256)
        out["read_GBs_nontemporal" if nt else "read_GBs_plain"] = 2048 * 1048576 / (r["ms"] * 1e-3) / 1e9
    out["measured_mfma_peak_tflops"] = max(v for k, v in out.items() if k.startswith("mfma_f16"))
    out["measured_read_GBs"] = max(out["read_GBs_plain"], out["read_GBs_nontemporal"])
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--layers", type=int, default=32, help="distinct KV containers the steps rotate over")
    ap.add_argument("--ctx", type=int, default=32768)
    ap.add_argument("--rows", type=int, default=64, help="query rows of the window (64 = headline; 1 = decode)")
    ap.add_argument("--issue", choices=("auto", "graph", "eager"), default="auto",
                    help="how the timed layer calls are issued: captured-pass replays, eager calls, or auto (eager for windows of 16+ rows)")
    ap.add_argument("--condition-ms", type=float, default=100.0,
                    help="untimed replays of the same workload before the warm-up steps, so that the timed steps run at sustained clocks")
    ap.add_argument("--opt", action="append", default=[], metavar="KEY=VALUE",
                    help="yka_set_opt on the headline handle before anything is timed (e.g. 8=16: windows of up to 16 rows on the mid kernel)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary decode / verify-16 / verify-32 lines")
    ap.add_argument("--batched-only", action="store_true",
                    help="run only the multi-stream (batched decode) passes and print their figures (for profiling that kernel)")
    ap.add_argument("--r256-only", action="store_true",
                    help="run only the passes over the reference's 256-channel rows and print their figures (for profiling those kernels)")
    ap.add_argument("--trellis-only", action="store_true",
                    help="run only the passes over trellis-coded rows (5 and 4 bits per element) and print their figures")
    ap.add_argument("--prefill-only", action="store_true", help="only run the 2048-row prefill chunk on 131072 cached tokens and print it")
    ap.add_argument("--sweep", nargs="?", const="verify,decode,paged,prefill", default=None, metavar="GROUPS",
                    help="time layer calls over the option keys that shape the launch (split counts, kernel choice, slice length, "
                         "context hint) and print a table; GROUPS: comma-separated subset of verify,decode,paged,prefill")
    ap.add_argument("--machine", action="store_true", help="only run the machine probe (MFMA rate, read rate, overlap) and print it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three device-to-device copies of 256 MiB (a kernel of known traffic, for scaling FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (one process, one device); --gpus above 1 is not supported")

    import torch
    import yasakani_amd.native as native
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    if args.machine:
        print(json.dumps({"machine": machine_figures(native)}))
        return
    if args.sweep:
        sweep(native, tuple(args.sweep.split(",")))
        return
    if args.prefill_only:
        print(json.dumps({"prefill_2048_at_131072": prefill_chunk(native, reps=8, opts=[tuple(int(x) for x in o.split("=")) for o in args.opt])}))
        return
    if args.r256_only:
        print(json.dumps({"reference_rows_head_dim_256": r256_figures(native, args.ctx)}))
        return
    if args.trellis_only:
        print(json.dumps({"trellis_rows": {f"bits_{b}": trellis_figures(native, args.ctx, bits=b, torch=torch) for b in (5, 4)}}))
        return
    ctx, M, L = args.ctx, args.rows, args.layers
    max_ctx = ((ctx + 64 + 255) // 256) * 256
    q, k, v = synth(2026, ctx, 64)
    kv = native.KvCache(n_layers=L, max_ctx=max_ctx, max_rows=64)
    for kvp in args.opt:
        key, val = kvp.split("=")
        kv.set_opt(int(key), int(val))
    fill_cache(kv, k, v, ctx)
    layers = list(range(L))
    kn, vn = k[ctx:], v[ctx:]

    def measure(rows, steps, warmup):
        issue = args.issue if args.issue != "auto" else ("eager" if rows >= 16 else "graph")
        dt, host_dt, out = timed_passes(torch, kv, layers, q[:rows], kn[:rows], vn[:rows], ctx, rows, steps, warmup, issue, args.condition_ms)
        us = dt / steps * 1e6
        # the dominant kernel alone, hipEvents on the library's stream, replayed from a graph over all containers
        ms, _, inv = kv.bench(q[:rows], None, None, ctx, mode=2, use_graph=True, reps=20, want_inv=True)
        k_us = float(np.median(ms)) * 1e3 / L
        by, fl = algorithmic_bytes(ctx, rows), algorithmic_flops(ctx, rows)
        hbm_s, mfma_s = by / (HBM_PEAK_GBS * 1e9), fl / (MFMA_F16_PEAK_TFLOPS * 1e12)
        if mfma_s > hbm_s:
            roof = {"bound": "mfma", "achieved": fl / (k_us * 1e-6) / 1e12, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s"}
        else:
            roof = {"bound": "hbm", "achieved": by / (k_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
        roof["frac"] = roof["achieved"] / roof["peak"]
        # the cited traffic belongs to the library's own choice of kernel and split count: none is cited under --opt
        roof["traffic"], roof["traffic_source"] = (None, None) if args.opt else MEASURED_TRAFFIC.get((rows, ctx), (None, None))
        roof["kernel_us"] = k_us
        roof["host_clock_us_per_layer"] = host_dt / steps * 1e6
        roof["issue"] = issue
        # the reference's built-in check (kvx_probe.cu:419-441): the window against one-row passes over the same container
        roof["window_vs_single_rows"] = {"rows_differing": int(inv[0]), "rows": int(inv[1]), "values_differing": int(inv[2]),
                                         "max_distance_fp16_spacings": int(inv[3])}
        roof["hbm_frac"] = by / (k_us * 1e-6) / 1e9 / HBM_PEAK_GBS
        return us, by / (us * 1e-6) / 1e9, roof, out

    if args.batched_only:
        print(json.dumps({"batched_decode": batched_decode(torch, native, kv, ctx, L, kn, vn, q, calls=max(8, args.steps // 8))}))
        kv.close()
        return
    us, gbs, roof, out = measure(M, args.steps, args.warmup)
    line = {
        # the headline workload carries the published metric's text verbatim; `value` is its effective-KV-GB/s component,
        # `us_per_layer` and `hbm_peak_frac` are the other two
        "metric": ("\u00b5s/layer + effective KV GB/s (% HBM peak), int4-KV GQA verify-64 at 32k ctx" if (M, ctx) == (64, 32768) else
                   f"\u00b5s/layer + effective KV GB/s (% HBM peak), int4-KV GQA verify-{M} at {ctx} ctx" if M > 1 else
                   f"\u00b5s/layer + effective KV GB/s (% HBM peak), int4-KV GQA decode at {ctx} ctx"),
        "value": gbs, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "conditioning_ms": args.condition_ms,
        "ms_per_step": us / 1e3, "us_per_layer": us, "hbm_peak_frac": gbs / HBM_PEAK_GBS,
        # value / ms_per_step / us_per_layer come from GPU events on the stream the calls are issued on; the host's clock
        # around the same region (issue + synchronize included) is given beside them
        "clock": "GPU events on the launch stream", "host_clock_us_per_layer": roof["host_clock_us_per_layer"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"verify window of {M} rows over {ctx} cached int4 tokens (one layer call = append + attention + combine)",
                   "n_heads": NH, "n_kv_heads": KVH, "head_dim": D, "kv_format": "int4 group-32, fp16 scales",
                   "containers": L, "container_MB": ctx * TOKEN_BYTES / 1e6,
                   "issue": "captured pass replay" if roof["issue"] == "graph" else "eager yka_append_attend calls on one stream"},
        "roofline": roof,
    }
    if not args.no_extra:
        extra = {}
        for rows in (1, 4, 8, 16, 32):
            if rows == M:
                continue
            u, g, r, _ = measure(rows, max(L, args.steps // 2), args.warmup)
            extra[f"rows_{rows}"] = {"us_per_layer": u, "value_GBs": g, "hbm_peak_frac": g / HBM_PEAK_GBS, "roofline": r}
        line["other_windows"] = extra
        # the same two workloads replayed on ONE container: the 18.9 MB stay in the 256 MB Infinity Cache / L2, so this
        # is the cache-hot figure, not an HBM figure
        hot = {}
        for rows in (64, 1):
            dt, _, _ = timed_passes(torch, kv, [0] * L, q[:rows], kn[:rows], vn[:rows], ctx, rows, L * 8, L)
            hot[f"rows_{rows}"] = {"us_per_layer": dt / (L * 8) * 1e6}
        line["cache_hot_single_container"] = hot
        line["decode_4096"] = small_decode(native)
    if not args.no_cpu:
        base, ref16 = cpu_baseline(kv, q[:M], ctx, M)
        line["cpu_baseline"] = base
        a, b = out.astype(np.float64), ref16.astype(np.float64)
        line["parity_vs_cpu"] = {"max_abs": float(np.abs(a - b).max()), "rel_l2": float(np.linalg.norm(a - b) / np.linalg.norm(b))}
    if not args.no_extra:                       # last: it overwrites the rows the parity check above reads
        line["batched_decode"] = batched_decode(torch, native, kv, ctx, L, kn, vn, q)
        line["append_vs_post"] = append_vs_post(torch, native, kv, ctx)
    kv.close()
    if args.calibrate_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["calibration_copy_bytes"] = 256 << 20
    if not args.no_extra:
        line["machine"] = machine_figures(native)
        mf = line["machine"]
        line["roofline"]["frac_of_measured_ceiling"] = (line["roofline"]["achieved"] / mf["measured_mfma_peak_tflops"] if line["roofline"]["bound"] == "mfma"
                                                         else line["roofline"]["achieved"] / mf["measured_read_GBs"])
        line["other_configs"] = big_configs(native)
        line["reference_rows_head_dim_256"] = r256_figures(native)
        line["trellis_rows"] = {"bits_5": trellis_figures(native, torch=torch)}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
