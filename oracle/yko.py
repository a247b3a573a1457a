"""ctypes wrapper of the CPU oracle libyko.so.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke run and the cpu_baseline leg of the benchmark import this module; the product package
(yasakani_amd) never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libyko.so")
D, GROUP = 128, 32
NG = D // GROUP


_SO_SCALAR = os.path.join(_HERE, "libyko_scalar.so")
BUILD_FLAGS = "gcc -O3 -mavx2 -ffp-contract=off -fopenmp (inner loops written for the vectoriser)"
BUILD_FLAGS_SCALAR = "gcc -O2 -fno-tree-vectorize -fno-tree-slp-vectorize -ffp-contract=off (plain scalar code)"


def build(force=False):
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    p = subprocess.run(["make", "-C", _HERE, "all"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("building libyko.so failed:\n" + p.stdout[-4000:])
    return _SO


class _Cache(C.Structure):
    _fields_ = [("n_heads", C.c_int), ("n_kv_heads", C.c_int), ("head_dim", C.c_int), ("max_ctx", C.c_int),
                ("kc", C.c_void_p), ("ks", C.c_void_p), ("vc", C.c_void_p), ("vs", C.c_void_p), ("fmt", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        vp = C.c_void_p
        L.yko_h2f.restype = C.c_float; L.yko_h2f.argtypes = [C.c_uint16]
        L.yko_f2h.restype = C.c_uint16; L.yko_f2h.argtypes = [C.c_float]
        L.yko_quant_rows.argtypes = [vp, C.c_int, C.c_int, vp, vp]
        L.yko_dequant_rows.argtypes = [vp, vp, C.c_int, C.c_int, vp]
        L.yko_pack_nibbles.argtypes = [vp, C.c_int, vp]
        L.yko_unpack_nibbles.argtypes = [vp, C.c_int, vp]
        L.yko_append.argtypes = [C.POINTER(_Cache), vp, vp, C.c_int, C.c_int]
        L.yko_attend_f32.argtypes = [C.POINTER(_Cache), vp, C.c_int, C.c_int, vp, C.c_int, C.c_int, vp, vp]
        L.yko_attend_f64.argtypes = [C.POINTER(_Cache), vp, C.c_int, C.c_int, vp, vp]
        L.yko_combine.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int, vp]
        L.yko_normal.restype = C.c_double; L.yko_normal.argtypes = [C.c_uint64, C.c_uint64]
        L.yko_splitmix64.restype = C.c_uint64; L.yko_splitmix64.argtypes = [C.c_uint64]
        L.yko_outlier_channels.argtypes = [C.c_uint64, C.c_int, vp]
        L.yko_fill_normal_f16.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, vp, C.c_float, vp]
        L.yko_kvx_sign.restype = C.c_float; L.yko_kvx_sign.argtypes = [C.c_int]
        L.yko_kvx_rotate256.argtypes = [vp, vp, C.c_int]
        L.yko_flat4_encode256.argtypes = [vp, vp, vp, vp]
        L.yko_flat4_decode256.argtypes = [vp, C.c_float, vp]
        L.yko_int8_encode256.argtypes = [vp, vp, vp]
        L.yko_kvx_probe256.argtypes = [vp, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp]
        L.yko_attn_out256.argtypes = [vp, vp, vp, C.c_int, C.c_int, vp, vp]
        L.yko_rotate128.argtypes = [vp, vp, C.c_int, C.c_float]
        L.yko_attn_post.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, vp, C.c_float, vp, C.c_int, C.c_int, C.c_int, vp, vp, vp]
        L.yko_unrotate_out.argtypes = [vp, C.c_int, vp]
        L.yko_attn_post256.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, vp, C.c_float, vp, C.c_int, C.c_int, C.c_int, vp, vp, vp]
        L.yko_tb_check_blob.argtypes = [vp, C.c_size_t]
        L.yko_tb_group.argtypes = [vp, C.c_int, vp]
        L.yko_tb_viterbi.argtypes = [vp, C.c_int, vp, C.c_int, vp]
        L.yko_tb_pack.argtypes = [vp, C.c_int, vp]
        L.yko_tb_decode_row.argtypes = [vp, C.c_int, vp, C.c_float, C.c_uint32, vp]
        L.yko_tb_encode_rows.argtypes = [vp, vp, vp, C.c_int, vp, vp, vp, C.c_int, vp, vp, vp, vp]
        _lib = L
    return _lib


_lib_scalar = None


def scalar_lib():
    """The attention oracle built as plain scalar code (timing baseline only; same sources, same results)."""
    global _lib_scalar
    if _lib_scalar is None:
        if not os.path.exists(_SO_SCALAR):
            build()
        L = C.CDLL(_SO_SCALAR)
        L.yko_attend_f32.argtypes = [C.POINTER(_Cache), C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        _lib_scalar = L
    return _lib_scalar


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _as_u16(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint16) if a.dtype == np.float16 else a.astype(np.uint16, copy=False)


def h2f_all():
    """fp32 value of every fp16 bit pattern (65536 entries)."""
    L = lib()
    return np.array([L.yko_h2f(i) for i in range(65536)], np.float32)


def f2h(x):
    L = lib()
    x = np.asarray(x, np.float32).ravel()
    return np.array([L.yko_f2h(float(v)) for v in x], np.uint16)


def quant_rows(x16, dim=D):
    """x16 [rows, dim] fp16 -> codes [rows, dim/2] u8, scales [rows, dim/32] u16."""
    x = _as_u16(x16).reshape(-1, dim)
    rows = x.shape[0]
    codes = np.empty((rows, dim // 2), np.uint8)
    scales = np.empty((rows, dim // GROUP), np.uint16)
    lib().yko_quant_rows(_p(x), rows, dim, _p(codes), _p(scales))
    return codes, scales


def dequant_rows(codes, scales, dim=D):
    codes = np.ascontiguousarray(codes, np.uint8).reshape(-1, dim // 2)
    scales = _as_u16(scales).reshape(-1, dim // GROUP)
    y = np.empty((codes.shape[0], dim), np.float32)
    lib().yko_dequant_rows(_p(codes), _p(scales), codes.shape[0], dim, _p(y))
    return y


def pack_nibbles(fields):
    f = np.ascontiguousarray(fields, np.uint8)
    out = np.empty(f.size // 2, np.uint8)
    lib().yko_pack_nibbles(_p(f), f.size, _p(out))
    return out


def unpack_nibbles(bytes_):
    b = np.ascontiguousarray(bytes_, np.uint8)
    out = np.empty(b.size * 2, np.uint8)
    lib().yko_unpack_nibbles(_p(b), b.size * 2, _p(out))
    return out


class Cache:
    """Canonical cache image of one layer.  head_dim 128: kc/vc [kvh, max_ctx, 64] u8, ks/vs [kvh, max_ctx, 4] u16
    (int4 in 32-channel groups with fp16 scales).  head_dim 256: the reference's own rows - kc/vc [kvh, max_ctx, 32] u32
    (MSB-first 4-bit fields), ks/vs [kvh, max_ctx] f32, one scale per row."""

    def __init__(self, max_ctx, n_heads=24, n_kv_heads=4, head_dim=D):
        self.n_heads, self.n_kv_heads, self.head_dim, self.max_ctx = n_heads, n_kv_heads, head_dim, max_ctx
        self.fmt = 1 if head_dim == 256 else 0
        if self.fmt:
            self.kc = np.zeros((n_kv_heads, max_ctx, 32), np.uint32)
            self.ks = np.zeros((n_kv_heads, max_ctx), np.float32)
        else:
            self.kc = np.zeros((n_kv_heads, max_ctx, head_dim // 2), np.uint8)
            self.ks = np.zeros((n_kv_heads, max_ctx, head_dim // GROUP), np.uint16)
        self.vc = np.zeros_like(self.kc)
        self.vs = np.zeros_like(self.ks)

    def _c(self):
        return _Cache(self.n_heads, self.n_kv_heads, self.head_dim, self.max_ctx,
                      self.kc.ctypes.data, self.ks.ctypes.data, self.vc.ctypes.data, self.vs.ctypes.data, self.fmt)

    def append(self, k16, v16, pos):
        k = _as_u16(k16); v = _as_u16(v16)
        M = k.shape[0]
        assert k.shape == (M, self.n_kv_heads, self.head_dim) and v.shape == k.shape
        assert pos + M <= self.max_ctx
        c = self._c()
        lib().yko_append(C.byref(c), _p(k), _p(v), M, pos)

    def attend_f32(self, q16, pos, depth=None, splits=0, threads=1, want_f32=False, scalar_build=False):
        q = _as_u16(q16)
        M = q.shape[0]
        assert q.shape == (M, self.n_heads, self.head_dim)
        dep = None if depth is None else np.ascontiguousarray(depth, np.uint8)
        out = np.empty(q.shape, np.uint16)
        o32 = np.empty(q.shape, np.float32) if want_f32 else None
        c = self._c()
        (scalar_lib() if scalar_build else lib()).yko_attend_f32(C.byref(c), _p(q), M, pos, _p(dep), splits, threads, _p(out), _p(o32))
        return (out.view(np.float16), o32) if want_f32 else out.view(np.float16)

    def attend_f64(self, q16, pos, depth=None):
        q = _as_u16(q16)
        M = q.shape[0]
        dep = None if depth is None else np.ascontiguousarray(depth, np.uint8)
        out = np.empty(q.shape, np.float64)
        c = self._c()
        lib().yko_attend_f64(C.byref(c), _p(q), M, pos, _p(dep), _p(out))
        return out


def combine(pm, pl, pacc):
    pm = np.ascontiguousarray(pm, np.float32); pl = np.ascontiguousarray(pl, np.float32)
    pacc = np.ascontiguousarray(pacc, np.float32)
    S, rows = pm.shape
    dim = pacc.shape[-1]
    y = np.empty((rows, dim), np.float32)
    lib().yko_combine(_p(pm), _p(pl), _p(pacc), S, rows, dim, _p(y))
    return y


def outlier_channels(seed, dim=D):
    ch = np.zeros(4, np.int32)
    lib().yko_outlier_channels(seed, dim, _p(ch))
    return ch


def fill_normal_f16(seed, n_rows, dim=D, outliers=None, mult=8.0, first=0):
    """fp16 array [n_rows, dim] of N(0,1); channels in `outliers` (4 ints) multiplied by `mult` before rounding."""
    out = np.empty((n_rows, dim), np.uint16)
    ch = None if outliers is None else np.ascontiguousarray(outliers, np.int32)
    lib().yko_fill_normal_f16(seed, first, n_rows * dim, dim, _p(ch), mult, _p(out))
    return out.view(np.float16)


def make_inputs(seed, ctx, M, n_heads=24, n_kv_heads=4, dim=D):
    """Seeded inputs of the measured configurations: Q [M,NH,D], cached K/V [ctx,KVH,D], new K/V [M,KVH,D], all fp16;
    K carries 4 fixed outlier channels scaled x8."""
    ch = outlier_channels(seed, dim)
    q = fill_normal_f16(seed + 1, M * n_heads, dim).reshape(M, n_heads, dim)
    k = fill_normal_f16(seed + 2, (ctx + M) * n_kv_heads, dim, ch, 8.0).reshape(ctx + M, n_kv_heads, dim)
    v = fill_normal_f16(seed + 3, (ctx + M) * n_kv_heads, dim).reshape(ctx + M, n_kv_heads, dim)
    return q, k[:ctx], v[:ctx], k[ctx:], v[ctx:], ch


# ---- the reference's own 256-channel row codec ----

def kvx_signs():
    return np.array([lib().yko_kvx_sign(d) for d in range(256)], dtype=np.float32)


def kvx_rotate256(x, inverse=False):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 256)
    y = np.empty_like(x)
    for r in range(x.shape[0]):
        lib().yko_kvx_rotate256(_p(x[r]), _p(y[r]), 1 if inverse else 0)
    return y


def flat4_encode256(r):
    r = np.ascontiguousarray(r, dtype=np.float32).reshape(-1, 256)
    n = r.shape[0]
    words = np.empty((n, 32), np.uint32); scale = np.empty(n, np.float32); xq = np.empty_like(r)
    for i in range(n):
        lib().yko_flat4_encode256(_p(r[i]), _p(words[i]), _p(scale[i:i + 1]), _p(xq[i]))
    return words, scale, xq


def flat4_decode256(words, scale):
    words = np.ascontiguousarray(words, dtype=np.uint32).reshape(-1, 32)
    y = np.empty((words.shape[0], 256), np.float32)
    for i in range(words.shape[0]):
        lib().yko_flat4_decode256(_p(words[i]), float(scale[i]), _p(y[i]))
    return y


def int8_encode256(x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 256)
    q = np.empty(x.shape, np.int8); scale = np.empty(x.shape[0], np.float32)
    for i in range(x.shape[0]):
        lib().yko_int8_encode256(_p(x[i]), _p(q[i]), _p(scale[i:i + 1]))
    return q, scale


def kvx_probe256(x, mode, rot):
    """round trip [rotate] -> encode -> decode -> [inverse rotate]; returns (q8 or None, words or None, scales, y)"""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 256)
    n = x.shape[0]
    q8 = np.zeros((n, 256), np.int8); words = np.zeros((n, 32), np.uint32)
    scales = np.empty(n, np.float32); y = np.empty_like(x)
    lib().yko_kvx_probe256(_p(x), n, int(mode), int(rot), _p(q8), _p(words), _p(scales), _p(y))
    return (q8 if mode == 0 else None), (words if mode == 1 else None), scales, y


# ---- between the QKV projection and the cache ----

def rotate128(x, inverse=False, factor=0.125):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 128)
    y = np.empty_like(x)
    for r in range(x.shape[0]):
        lib().yko_rotate128(_p(x[r]), _p(y[r]), 1 if inverse else 0, float(factor))
    return y


def rope_table(n_pos, rd, base=10000.0):
    """(cos, sin) [n_pos][rd/2][2] fp32, frequencies base^(-2i/rd), values rounded to fp16 precision
    (the reference rounds its table to its 16-bit activation type, q35_kernels.cu:1101-1107)."""
    i = np.arange(rd // 2, dtype=np.float64)
    f = np.arange(n_pos, dtype=np.float64)[:, None] * base ** (-2.0 * i / rd)[None, :]
    t = np.stack([np.cos(f), np.sin(f)], axis=-1)
    return np.ascontiguousarray(t.astype(np.float16).astype(np.float32))


def attn_post(xq, xk, xv, qn_w16, kn_w16, eps, rope, rd, pos, rot):
    """fp32 projection rows -> (q16, k16, v16) fp16 bit patterns; xq [M,H,128], xk/xv [M,KVH,128]"""
    xq = np.ascontiguousarray(xq, np.float32); xk = np.ascontiguousarray(xk, np.float32); xv = np.ascontiguousarray(xv, np.float32)
    M, H, _ = xq.shape; KVH = xk.shape[1]
    q16 = np.empty((M, H, 128), np.uint16); k16 = np.empty((M, KVH, 128), np.uint16); v16 = np.empty((M, KVH, 128), np.uint16)
    qw = _as_u16(qn_w16); kw = _as_u16(kn_w16)
    if rd > 0:
        rope = np.ascontiguousarray(rope, np.float32)
        assert rope.shape[0] >= pos + M and rope.shape[1] == rd // 2
    else:
        rope = np.zeros(1, np.float32)             # never read when there is no rotary step
    lib().yko_attn_post(_p(xq), _p(xk), _p(xv), M, H, KVH, _p(qw), _p(kw), float(eps), _p(rope), int(rd), int(pos), int(rot),
                        _p(q16), _p(k16), _p(v16))
    return q16, k16, v16


def attn_post256(xq, xk, xv, qn_w16, kn_w16, eps, rope, rd, pos, rot):
    """256-channel heads: fp32 projection rows -> (q16 fp16 bit patterns [M,H,256], k32, v32 fp32 [M,KVH,256]: the rows
    the row quantizer takes)"""
    xq = np.ascontiguousarray(xq, np.float32); xk = np.ascontiguousarray(xk, np.float32); xv = np.ascontiguousarray(xv, np.float32)
    M, H, _ = xq.shape; KVH = xk.shape[1]
    q16 = np.empty((M, H, 256), np.uint16); k32 = np.empty((M, KVH, 256), np.float32); v32 = np.empty((M, KVH, 256), np.float32)
    qw = _as_u16(qn_w16); kw = _as_u16(kn_w16)
    if rd > 0:
        rope = np.ascontiguousarray(rope, np.float32)
        assert rope.shape[0] >= pos + M and rope.shape[1] == rd // 2
    else:
        rope = np.zeros(1, np.float32)
    lib().yko_attn_post256(_p(xq), _p(xk), _p(xv), M, H, KVH, _p(qw), _p(kw), float(eps), _p(rope), int(rd), int(pos), int(rot),
                           _p(q16), _p(k32), _p(v32))
    return q16, k32, v32


def unrotate_out(y32):
    y32 = np.ascontiguousarray(y32, np.float32)
    out = np.empty(y32.shape, np.uint16)
    lib().yko_unrotate_out(_p(y32), int(y32.size // 128), _p(out))
    return out


def attn_out256(y16, gate16, signs):
    """the step after attention for 256-channel heads: y16, gate16 [M, n_heads, 256] fp16, signs [n_heads*256] int8
    -> (qx [M, n_heads*256] int8, alpha [M, n_heads*256/512] f32)"""
    y = _as_u16(y16); g = _as_u16(gate16)
    M, H, _ = y.shape
    sg = np.ascontiguousarray(signs, np.int8)
    qx = np.empty((M, H * 256), np.int8); alpha = np.empty((M, H * 256 // 512), np.float32)
    lib().yko_attn_out256(_p(y), _p(g), _p(sg), M, H, _p(qx), _p(alpha))
    return qx, alpha


# ---- trellis-coded rows ----
def tb_check_blob(blob):
    b = np.frombuffer(bytes(blob), np.uint8)
    return lib().yko_tb_check_blob(_p(b), b.size)


def tb_group(blob, g):
    b = np.frombuffer(bytes(blob), np.uint8); f = np.zeros(6, np.int32)
    if lib().yko_tb_group(_p(b), int(g), _p(f)) != 0:
        raise IndexError(g)
    return dict(zip(("mode", "kk", "table", "guard", "m", "has_mu"), (int(v) for v in f)))


def tb_viterbi(xi, ci, kk):
    """one chunk: integer targets xi [T <= 64], table ci [256] int16 -> (states [T] uint8, path cost)"""
    xi = np.ascontiguousarray(xi, np.int32); ci = np.ascontiguousarray(ci, np.int16)
    st = np.zeros(xi.size, np.uint8)
    cost = lib().yko_tb_viterbi(_p(xi), int(xi.size), _p(ci), int(kk), _p(st))
    return st, cost


def tb_pack(fields, kb):
    fields = np.ascontiguousarray(fields, np.uint8); w = np.zeros(8 * kb, np.uint32)
    lib().yko_tb_pack(_p(fields), int(kb), _p(w))
    return w


def tb_encode_rows(blob, grp, pos, y, stride_words=40):
    """rows y [n, 256] fp32 of groups grp [n] at positions pos [n] -> dict(x, words [n, stride_words], scale, pc, best_mi, coded)"""
    b = np.frombuffer(bytes(blob), np.uint8)
    y = np.ascontiguousarray(y, np.float32); n = y.shape[0]
    grp = np.ascontiguousarray(grp, np.int32); pos = np.ascontiguousarray(pos, np.int32)
    out = dict(x=np.empty((n, 256), np.float32), words=np.zeros((n, stride_words), np.uint32), scale=np.empty(n, np.float32),
               pc=np.empty(n, np.uint32), best_mi=np.empty(n, np.int32), coded=np.empty(n, np.int32))
    lib().yko_tb_encode_rows(_p(b), _p(grp), _p(pos), n, _p(y), _p(out["x"]), _p(out["words"]), int(stride_words), _p(out["scale"]),
                             _p(out["pc"]), _p(out["best_mi"]), _p(out["coded"]))
    return out


def tb_decode_rows(blob, grp, words, scale, pc):
    b = np.frombuffer(bytes(blob), np.uint8)
    words = np.ascontiguousarray(words, np.uint32); n = words.shape[0]
    y = np.empty((n, 256), np.float32)
    for i in range(n):
        if lib().yko_tb_decode_row(_p(b), int(grp[i]), _p(words[i]), float(scale[i]), int(pc[i]), _p(y[i])) != 0:
            raise IndexError(int(grp[i]))
    return y


def tb_attend_f64(k, v, q16, pos, depth=None):
    """textbook attention in fp64 over decoded rows: k, v [n_kv, rows, 256] fp32 (what tb_decode_rows returns per kv head),
    q16 [M, n_heads, 256] fp16; row t sees keys [0, pos + depth(t) + 1).  Returns [M, n_heads, 256] fp64."""
    q = np.asarray(q16, np.float16).astype(np.float64) if np.asarray(q16).dtype != np.uint16 else np.asarray(q16).view(np.float16).astype(np.float64)
    M, H, Dh = q.shape
    n_kv = k.shape[0]; G = H // n_kv
    out = np.zeros((M, H, Dh))
    for t in range(M):
        n = pos + (int(depth[t]) if depth is not None else t) + 1
        for h in range(H):
            kh = k[h // G, :n].astype(np.float64); vh = v[h // G, :n].astype(np.float64)
            s = kh @ q[t, h] / np.sqrt(Dh)
            p = np.exp(s - s.max()); p /= p.sum()
            out[t, h] = p @ vh
    return out
