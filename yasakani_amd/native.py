"""ctypes binding of libyka.so - one Python method per entry point of include/yka_abi.h.

Mirrors the reference's binding style (python/yasakani/_native.py:1-5): argtypes/restype declared once, every int
return checked, the library's thread-local error string raised as RuntimeError.  Host-pointer hooks take numpy
arrays; launch-path calls take raw device addresses (ints), e.g. torch.Tensor.data_ptr().
"""
import ctypes as C
import os

import numpy as np

from .build import library_path

D = 128          # head_dim
GROUP = 32       # channels per scale group
NG = D // GROUP
PAGE = 256       # tokens per page


class YkaError(RuntimeError):
    pass


class KvConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("n_layers", "n_heads", "n_kv_heads", "head_dim", "max_ctx", "max_rows", "paged", "device")]


class PostParams(C.Structure):
    """yka_post_params: device pointers of the norm weights and of the rotary table, and the switches of the step
    between the QKV projection and the cache."""
    _fields_ = [("d_qn_w16", C.c_void_p), ("d_kn_w16", C.c_void_p), ("eps", C.c_float), ("d_rope", C.c_void_p),
                ("rope_dims", C.c_int32), ("rope_rows", C.c_int32), ("rotate", C.c_int32),
                ("d_xgate", C.c_void_p), ("d_gate16", C.c_void_p)]


def _load():
    path = library_path()
    if not os.path.exists(path):
        raise YkaError(f"{path} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
                       "(there is no CPU fallback for this path)")
    lib = C.CDLL(path)
    vp, i32 = C.c_void_p, C.c_int
    sig = {
        "yka_kv_open": (vp, [C.POINTER(KvConfig)]),
        "yka_kv_close": (None, [vp]),
        "yka_last_error": (C.c_char_p, []),
        "yka_build_info": (C.c_char_p, []),
        "yka_set_opt": (i32, [vp, i32, i32]),
        "yka_kv_set_page_table": (i32, [vp, i32, vp, i32]),
        "yka_append": (i32, [vp, i32, vp, vp, i32, vp, vp]),
        "yka_attend": (i32, [vp, i32, vp, i32, vp, vp, vp, vp]),
        "yka_append_attend": (i32, [vp, i32, vp, vp, vp, i32, vp, vp, vp, vp]),
        "yka_append_attend_static": (i32, [vp, i32, vp, vp, vp, i32, vp, vp, vp, vp]),
        "yka_kv_poison_workspace": (i32, [vp]),
        "yka_codec_probe": (i32, [vp, i32, vp, vp, vp]),
        "yka_kvx256_probe": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "yka_attn_post": (i32, [vp, i32, vp, vp, vp, i32, vp, vp, vp, vp]),
        "yka_tb_pack_unpack": (i32, [vp, C.c_size_t, vp, vp, vp, i32, i32, vp, vp, vp, vp, vp]),
        "yka_kv_set_profile": (i32, [vp, vp, C.c_size_t]),
        "yka_kv_profile_bits": (i32, [vp]),
        "yka_kv_export_rows_tb": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "yka_kv_export_rows256": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "yka_append256_f32": (i32, [vp, i32, vp, vp, i32, vp, i32, vp]),
        "yka_attn_out256": (i32, [vp, vp, vp, i32, i32, vp, vp, vp]),
        "yka_attn_out256_host": (i32, [vp, vp, vp, i32, i32, vp, vp]),
        "yka_attn_out256_lo": (i32, [vp, vp, vp, i32, i32, vp, vp, vp]),
        "yka_attn_out256_lo_host": (i32, [vp, vp, vp, i32, i32, vp, vp]),
        "yka_rotate_q256": (i32, [vp, i32, vp, vp]),
        "yka_append256_f32_host": (i32, [vp, i32, vp, vp, i32, i32, i32]),
        "yka_rotate_q256_host": (i32, [vp, i32, vp]),
        "yka_kv_import_rows256": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "yka_append_attend_ms": (i32, [vp, vp, vp, vp, i32, vp, vp, vp, vp]),
        "yka_ms_call_host": (i32, [vp, vp, vp, vp, i32, vp, vp, vp]),
        "yka_attn_post_host": (i32, [vp, i32, vp, vp, vp, i32, i32, vp, vp, C.c_float, vp, i32, i32, i32, vp, vp, vp]),
        "yka_kv_export_rows": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "yka_kv_import_rows": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "yka_kv_dequant_rows": (i32, [vp, i32, i32, i32, vp, vp]),
        "yka_kv_replicate_layer": (i32, [vp, i32]),
        "yka_layer_call_host": (i32, [vp, i32, vp, vp, vp, i32, i32, vp, vp]),
        "yka_append_host": (i32, [vp, i32, vp, vp, i32, i32]),
        "yka_pass_capture": (vp, [vp, vp, i32, vp, vp, vp, i32, vp, vp, vp, i32]),
        "yka_pass_launch": (i32, [vp, vp]),
        "yka_pass_destroy": (None, [vp]),
        "yka_attn_bench": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp]),
        "yka_machine_probe": (i32, [i32, i32, i32, i32, i32, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


EXPORTS = ("yka_kv_open", "yka_kv_close", "yka_last_error", "yka_build_info", "yka_set_opt", "yka_kv_set_page_table",
           "yka_append", "yka_attend", "yka_append_attend", "yka_append_attend_static", "yka_kv_poison_workspace", "yka_codec_probe", "yka_kvx256_probe", "yka_tb_pack_unpack", "yka_kv_set_profile", "yka_kv_profile_bits", "yka_kv_export_rows_tb", "yka_attn_post", "yka_append_attend_ms", "yka_ms_call_host",
           "yka_attn_post_host", "yka_kv_export_rows", "yka_kv_export_rows256", "yka_kv_import_rows256",
           "yka_attn_out256", "yka_attn_out256_host", "yka_attn_out256_lo", "yka_attn_out256_lo_host", "yka_append256_f32", "yka_rotate_q256", "yka_append256_f32_host", "yka_rotate_q256_host",
           "yka_kv_import_rows", "yka_kv_dequant_rows", "yka_kv_replicate_layer", "yka_layer_call_host",
           "yka_append_host", "yka_pass_capture", "yka_pass_launch", "yka_pass_destroy", "yka_attn_bench", "yka_machine_probe")

_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _chk(rc):
    if rc != 0:
        raise YkaError(lib().yka_last_error().decode("utf-8", "replace"))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _u16(a, shape):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    if a.dtype != np.uint16 or a.shape != tuple(shape):
        raise ValueError(f"expected fp16/uint16 array of shape {tuple(shape)}, got {a.dtype} {a.shape}")
    return a


def bf16_bits(x):
    """fp32 array -> bf16 bit patterns (uint16), round to nearest even (finite values)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + np.uint32(0x7fff) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def bf16_to_f32(b):
    """bf16 bit patterns (uint16) -> fp32."""
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def build_info() -> str:
    return lib().yka_build_info().decode()


def machine_probe(kind, p0=0, iters=1000, blocks=256, threads=256):
    """One launch of a fixed instruction mix (see yka_machine_probe in include/yka_abi.h).  Returns a dict with the
    event time and what the waves measured themselves: shader cycles, wall ticks, and the shader clock they imply."""
    out = np.zeros(6, np.float64)
    _chk(lib().yka_machine_probe(kind, p0, iters, blocks, threads, _ptr(out)))
    r = {"ms": out[0], "cycles": out[1], "wall_ticks": out[2], "cycles_b": out[3], "wall_ticks_b": out[4], "wall_khz": out[5]}
    if out[2] > 0 and out[5] > 0:
        r["shader_mhz"] = out[1] / (out[2] / out[5]) / 1e3
    return r


def codec_probe(x16):
    """x16 [rows,128] fp16 -> (codes [rows,64] u8, scales [rows,4] u16 bit patterns, y [rows,128] f32)."""
    x16 = np.ascontiguousarray(x16)
    rows = x16.shape[0]
    x = _u16(x16, (rows, D))
    codes = np.empty((rows, D // 2), np.uint8)
    scales = np.empty((rows, NG), np.uint16)
    y = np.empty((rows, D), np.float32)
    _chk(lib().yka_codec_probe(_ptr(x), rows, _ptr(codes), _ptr(scales), _ptr(y)))
    return codes, scales, y


def attn_out256(y16, gate16, signs):
    """The step after attention for 256-channel heads: y16, gate16 [M, n_heads, 256] fp16, signs [n_heads*256] int8 ->
    (qx [M, n_heads*256] int8, alpha [M, n_heads*256/512] f32)."""
    y = np.ascontiguousarray(y16); g = np.ascontiguousarray(gate16)
    M, H, _ = y.shape
    y = _u16(y, (M, H, 256)); g = _u16(g, (M, H, 256))
    sg = np.ascontiguousarray(signs, np.int8)
    if sg.shape != (H * 256,):
        raise ValueError("signs needs n_heads * 256 entries")
    qx = np.empty((M, H * 256), np.int8); alpha = np.empty((M, H * 256 // 512), np.float32)
    _chk(lib().yka_attn_out256_host(_ptr(y), _ptr(g), _ptr(sg), M, H, _ptr(qx), _ptr(alpha)))
    return qx, alpha


def attn_out256_lo(y16, gate16, signs):
    """The same step in the reference's interleaved layout for at most 8 tokens: qx [n_heads/2, 4096] int8 (zero where no
    token wrote), alpha [M, n_heads*256/512] f32."""
    y = np.ascontiguousarray(y16); g = np.ascontiguousarray(gate16)
    M, H, _ = y.shape
    y = _u16(y, (M, H, 256)); g = _u16(g, (M, H, 256))
    sg = np.ascontiguousarray(signs, np.int8)
    if sg.shape != (H * 256,):
        raise ValueError("signs needs n_heads * 256 entries")
    qx = np.empty((H // 2, 4096), np.int8); alpha = np.empty((M, H * 256 // 512), np.float32)
    _chk(lib().yka_attn_out256_lo_host(_ptr(y), _ptr(g), _ptr(sg), M, H, _ptr(qx), _ptr(alpha)))
    return qx, alpha


def rotate_q256(x32):
    """Rotated query rows: x32 [..., 256] fp32 -> fp16 of the signed Walsh-Hadamard rotation of every row."""
    x = np.ascontiguousarray(x32, np.float32)
    rows = x.size // 256
    q = np.empty(x.shape, np.uint16)
    _chk(lib().yka_rotate_q256_host(_ptr(x), rows, _ptr(q)))
    return q.view(np.float16)


def kvx256_probe(x, mode, rot):
    """Round trip through the reference's 256-channel row format (kvx_probe.cu:7-36).  x [rows,256] f32;
    mode 0 = int8 rows, 1 = flat int4 (MSB-first words); rot = signed Walsh-Hadamard rotation before and after.
    Returns (q8 [rows,256] i8 or None, words [rows,32] u32 or None, scales [rows] f32, y [rows,256] f32)."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 256)
    rows = x.shape[0]
    q8 = np.empty((rows, 256), np.int8) if mode == 0 else None
    words = np.empty((rows, 32), np.uint32) if mode == 1 else None
    scales = np.empty(rows, np.float32)
    y = np.empty((rows, 256), np.float32)
    _chk(lib().yka_kvx256_probe(_ptr(x), rows, int(mode), int(rot), _ptr(q8) if q8 is not None else None,
                                _ptr(words) if words is not None else None, _ptr(scales), _ptr(y)))
    return q8, words, scales, y


def tb_pack_unpack(blob, x, grp, pos, stride=160):
    """Trellis row codec round trip (kvx_probe.cu:123-188): x [rows,256] f32 with a group and a position per row ->
    dict(x = the encoder's reconstruction, words [rows, stride/4] u32, scale [rows] f32, pc [rows] u32, dec = the decoder's rows)."""
    b = np.frombuffer(bytes(blob), np.uint8)
    x = np.ascontiguousarray(x, np.float32).reshape(-1, 256)
    rows = x.shape[0]
    grp = np.ascontiguousarray(grp, np.int32); pos = np.ascontiguousarray(pos, np.int32)
    assert grp.shape == (rows,) and pos.shape == (rows,)
    y = np.empty((rows, 256), np.float32); dec = np.empty((rows, 256), np.float32)
    pay = np.empty((rows, stride), np.uint8); side = np.empty((rows, 2), np.uint32)
    ms = np.zeros(2, np.float32)
    _chk(lib().yka_tb_pack_unpack(_ptr(b), b.size, _ptr(x), _ptr(grp), _ptr(pos), rows, int(stride), _ptr(y), _ptr(pay), _ptr(side), _ptr(dec), _ptr(ms)))
    return dict(x=y, words=pay.view(np.uint32), scale=side[:, 0].copy().view(np.float32), pc=side[:, 1].copy(), dec=dec, ms=ms)


class KvCache:
    """Owns the int4 KV containers of `n_layers` layers on one GPU (the role Engine35 plays for its KV, engine35.cpp:303-329)."""

    def __init__(self, n_layers=1, n_heads=24, n_kv_heads=4, head_dim=D, max_ctx=4096, max_rows=64, paged=False, device=0):
        self.cfg = KvConfig(n_layers, n_heads, n_kv_heads, head_dim, max_ctx, max_rows, int(bool(paged)), device)
        self._bf16 = False          # option key 11: the boundary's 16-bit rows are bf16 (passed and returned as raw uint16 bit patterns)
        self._h = lib().yka_kv_open(C.byref(self.cfg))
        if not self._h:
            raise YkaError(lib().yka_last_error().decode("utf-8", "replace"))

    # -- lifetime --
    def close(self):
        if getattr(self, "_h", None):
            lib().yka_kv_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def n_heads(self):
        return self.cfg.n_heads

    @property
    def n_kv_heads(self):
        return self.cfg.n_kv_heads

    @property
    def max_ctx(self):
        return self.cfg.max_ctx

    # -- options / layout --
    def set_opt(self, key, value):
        _chk(lib().yka_set_opt(self._h, key, value))
        if key == 11:
            self._bf16 = bool(value)

    def set_page_table(self, table, layer=-1):
        t = np.ascontiguousarray(table, dtype=np.int32)
        _chk(lib().yka_kv_set_page_table(self._h, layer, _ptr(t), t.size))

    # -- launch path: device addresses --
    def append(self, layer, d_k16, d_v16, M, d_pos, stream=0):
        _chk(lib().yka_append(self._h, layer, d_k16, d_v16, M, d_pos, stream))

    def append256_f32_host(self, layer, k32, v32, pos, rotate=False):
        """head_dim 256: quantize fp32 rows k32/v32 [M,n_kv_heads,256] into rows pos..pos+M-1, rotating each row first if asked."""
        M = k32.shape[0]
        k = np.ascontiguousarray(k32, np.float32).reshape(M, self.cfg.n_kv_heads, 256)
        v = np.ascontiguousarray(v32, np.float32).reshape(M, self.cfg.n_kv_heads, 256)
        _chk(lib().yka_append256_f32_host(self._h, layer, _ptr(k), _ptr(v), M, pos, int(bool(rotate))))

    def append_attend_ms(self, d_q16, d_k16, d_v16, M, d_row_pos, d_row_slot, d_out16, stream=0):
        """Multi-stream pass with device pointers: row t uses container d_row_slot[t] at position d_row_pos[t]."""
        _chk(lib().yka_append_attend_ms(self._h, d_q16, d_k16, d_v16, M, d_row_pos, d_row_slot, d_out16, stream))

    def ms_call(self, q16, k16, v16, row_pos, row_slot):
        """Multi-stream pass with host arrays: q16 [M,n_heads,head_dim], k16/v16 [M,n_kv_heads,head_dim] (or None), row_pos/row_slot [M]."""
        M = q16.shape[0]
        D = self.cfg.head_dim
        q = _u16(q16, (M, self.cfg.n_heads, D))
        k = None if k16 is None else _u16(k16, (M, self.cfg.n_kv_heads, D))
        v = None if v16 is None else _u16(v16, (M, self.cfg.n_kv_heads, D))
        rp = np.ascontiguousarray(row_pos, np.int32); rs = np.ascontiguousarray(row_slot, np.int32)
        if rp.shape != (M,) or rs.shape != (M,):
            raise ValueError("row_pos and row_slot need one entry per row")
        out = np.empty((M, self.cfg.n_heads, D), np.uint16)
        _chk(lib().yka_ms_call_host(self._h, _ptr(q), _ptr(k), _ptr(v), M, _ptr(rp), _ptr(rs), _ptr(out)))
        return out.view(np.float16)

    def attn_post(self, layer, d_xq, d_xk, d_xv, M, d_pos, params, d_q16, stream=0):
        """Device-pointer form: projection outputs -> Q rows in d_q16, K/V rows quantized into the cache (params: PostParams)."""
        _chk(lib().yka_attn_post(self._h, layer, d_xq, d_xk, d_xv, M, d_pos, C.byref(params), d_q16, stream))

    def attend(self, layer, d_q16, M, d_pos, d_out16, d_depth=None, stream=0):
        _chk(lib().yka_attend(self._h, layer, d_q16, M, d_pos, d_depth, d_out16, stream))

    def append_attend(self, layer, d_q16, d_k16, d_v16, M, d_pos, d_out16, d_depth=None, stream=0):
        _chk(lib().yka_append_attend(self._h, layer, d_q16, d_k16, d_v16, M, d_pos, d_depth, d_out16, stream))

    def append_attend_static(self, layer, d_q16, d_k16, d_v16, M, d_pos, d_out16, d_depth=None, stream=0):
        """yka_append_attend with the split partials in the library's static device workspace (allocation-free form)."""
        _chk(lib().yka_append_attend_static(self._h, layer, d_q16, d_k16, d_v16, M, d_pos, d_depth, d_out16, stream))

    def poison_workspace(self):
        """test hook: NaN patterns over the handle's own split workspace"""
        _chk(lib().yka_kv_poison_workspace(self._h))

    def set_profile(self, blob):
        """switch a head_dim-256 handle to trellis-coded rows under a KVQP profile blob (see yasakani_amd.kvqp)"""
        b = np.frombuffer(bytes(blob), np.uint8)
        _chk(lib().yka_kv_set_profile(self._h, _ptr(b), b.size))
        self.profile_bits = lib().yka_kv_profile_bits(self._h)

    # -- hooks: host arrays --
    def export_rows(self, layer, pos0, n):
        kvh = self.cfg.n_kv_heads
        bits = getattr(self, "profile_bits", 0)
        if bits:                            # trellis-coded rows: payload words [kvh, n, 8 * bits] u32, row scales [kvh, n] f32
            kw = np.empty((kvh, n, 8 * bits), np.uint32); vw = np.empty_like(kw)
            ks = np.empty((kvh, n), np.float32); vs = np.empty_like(ks)
            _chk(lib().yka_kv_export_rows_tb(self._h, layer, pos0, n, _ptr(kw), _ptr(ks), _ptr(vw), _ptr(vs)))
            return kw, ks, vw, vs
        if self.cfg.head_dim == 256:        # words [kvh, n, 32] u32 and row scales [kvh, n] f32
            kw = np.empty((kvh, n, 32), np.uint32); vw = np.empty_like(kw)
            ks = np.empty((kvh, n), np.float32); vs = np.empty_like(ks)
            _chk(lib().yka_kv_export_rows256(self._h, layer, pos0, n, _ptr(kw), _ptr(ks), _ptr(vw), _ptr(vs)))
            return kw, ks, vw, vs
        kc = np.empty((kvh, n, D // 2), np.uint8); vc = np.empty_like(kc)
        ks = np.empty((kvh, n, NG), np.uint16); vs = np.empty_like(ks)
        _chk(lib().yka_kv_export_rows(self._h, layer, pos0, n, _ptr(kc), _ptr(ks), _ptr(vc), _ptr(vs)))
        return kc, ks, vc, vs

    def import_rows(self, layer, pos0, kc, ks, vc, vs):
        kvh = self.cfg.n_kv_heads
        n = kc.shape[1]
        if self.cfg.head_dim == 256:
            kw = np.ascontiguousarray(kc, np.uint32); vw = np.ascontiguousarray(vc, np.uint32)
            fs = np.ascontiguousarray(ks, np.float32); gs = np.ascontiguousarray(vs, np.float32)
            if kw.shape != (kvh, n, 32) or vw.shape != kw.shape or fs.shape != (kvh, n) or gs.shape != fs.shape:
                raise ValueError("expected words [kvh, n, 32] and scales [kvh, n]")
            _chk(lib().yka_kv_import_rows256(self._h, layer, pos0, n, _ptr(kw), _ptr(fs), _ptr(vw), _ptr(gs)))
            return
        kc = np.ascontiguousarray(kc, np.uint8); vc = np.ascontiguousarray(vc, np.uint8)
        ks = _u16(ks, (kvh, n, NG)); vs = _u16(vs, (kvh, n, NG))
        if kc.shape != (kvh, n, D // 2) or vc.shape != kc.shape:
            raise ValueError("codes must be [n_kv_heads, n, 64]")
        _chk(lib().yka_kv_import_rows(self._h, layer, pos0, n, _ptr(kc), _ptr(ks), _ptr(vc), _ptr(vs)))

    def dequant_rows(self, layer, pos0, n):
        kvh = self.cfg.n_kv_heads
        k = np.empty((kvh, n, D), np.float32); v = np.empty_like(k)
        _chk(lib().yka_kv_dequant_rows(self._h, layer, pos0, n, _ptr(k), _ptr(v)))
        return k, v

    def replicate_layer(self, src=0):
        _chk(lib().yka_kv_replicate_layer(self._h, src))

    def layer_call(self, layer, q16, k16, v16, pos, depth=None):
        """One layer call with host arrays: q16 [M,n_heads,128], k16/v16 [M,n_kv_heads,128] fp16 (or None = attend only)."""
        M = q16.shape[0]
        q = _u16(q16, (M, self.cfg.n_heads, self.cfg.head_dim))
        k = None if k16 is None else _u16(k16, (M, self.cfg.n_kv_heads, self.cfg.head_dim))
        v = None if v16 is None else _u16(v16, (M, self.cfg.n_kv_heads, self.cfg.head_dim))
        dep = None if depth is None else np.ascontiguousarray(depth, np.uint8)
        out = np.empty((M, self.cfg.n_heads, self.cfg.head_dim), np.uint16)
        _chk(lib().yka_layer_call_host(self._h, layer, _ptr(q), _ptr(k), _ptr(v), M, pos, _ptr(dep), _ptr(out)))
        return out if self._bf16 else out.view(np.float16)

    def append_host(self, layer, k16, v16, pos):
        """Quantize host rows k16/v16 [M,n_kv_heads,128] into rows pos..pos+M-1."""
        M = k16.shape[0]
        k = _u16(k16, (M, self.cfg.n_kv_heads, self.cfg.head_dim)); v = _u16(v16, (M, self.cfg.n_kv_heads, self.cfg.head_dim))
        _chk(lib().yka_append_host(self._h, layer, _ptr(k), _ptr(v), M, pos))

    def attn_post_host(self, layer, xq, xk, xv, pos, qn_w16, kn_w16, eps, rope, rope_dims, rotate=False, xgate=None):
        """Projection outputs (fp32; xq [M,n_heads,head_dim], xk/xv [M,n_kv_heads,head_dim]) -> RMS norm, rotary,
        optional rotation; K/V rows are quantized into rows pos..pos+M-1, the Q rows come back as 16-bit rows (fp16; raw
        bf16 bit patterns as uint16 if option key 11 is set).  With xgate (the gate half of the Q projection) the gate rows
        come back too: returns (q, gate)."""
        M = xq.shape[0]
        D = self.cfg.head_dim
        xq = np.ascontiguousarray(xq, np.float32).reshape(M, self.cfg.n_heads, D)
        xk = np.ascontiguousarray(xk, np.float32).reshape(M, self.cfg.n_kv_heads, D)
        xv = np.ascontiguousarray(xv, np.float32).reshape(M, self.cfg.n_kv_heads, D)
        qw = _u16(qn_w16, (D,)); kw = _u16(kn_w16, (D,))
        rows = 0
        if rope_dims > 0:
            rope = np.ascontiguousarray(rope, np.float32).reshape(-1, rope_dims // 2, 2)
            rows = rope.shape[0]
        q16 = np.empty((M, self.cfg.n_heads, D), np.uint16)
        g16 = None
        if xgate is not None:
            xgate = np.ascontiguousarray(xgate, np.float32).reshape(M, self.cfg.n_heads, D)
            g16 = np.empty((M, self.cfg.n_heads, D), np.uint16)
        _chk(lib().yka_attn_post_host(self._h, layer, _ptr(xq), _ptr(xk), _ptr(xv), M, pos, _ptr(qw), _ptr(kw), float(eps),
                                      _ptr(rope) if rope_dims > 0 else None, int(rope_dims), rows, int(bool(rotate)), _ptr(q16),
                                      _ptr(xgate) if xgate is not None else None, _ptr(g16) if g16 is not None else None))
        if self._bf16:
            return q16 if g16 is None else (q16, g16)
        return q16.view(np.float16) if g16 is None else (q16.view(np.float16), g16.view(np.float16))

    def capture_pass(self, layers, d_q16, d_k16, d_v16, M, d_pos, d_out16, d_depth=None, mode=0):
        """Records one layer call per listed layer into a graph (device addresses); returns a Pass."""
        ls = np.ascontiguousarray(layers, np.int32)
        h = lib().yka_pass_capture(self._h, _ptr(ls), ls.size, d_q16, d_k16, d_v16, M, d_pos, d_depth, d_out16, mode)
        if not h:
            raise YkaError(lib().yka_last_error().decode("utf-8", "replace"))
        return Pass(h)

    def bench(self, q16, k16, v16, pos, mode=0, use_graph=True, reps=20, want_inv=False):
        """Timed sweeps over all layers; returns (ms per sweep [reps], out of the last layer call) and, if asked, the
        window-against-single-rows invariant (rows differing, rows compared, values differing, largest fp16-spacing distance)."""
        M = q16.shape[0]
        q = _u16(q16, (M, self.cfg.n_heads, self.cfg.head_dim))
        k = None if k16 is None else _u16(k16, (M, self.cfg.n_kv_heads, self.cfg.head_dim))
        v = None if v16 is None else _u16(v16, (M, self.cfg.n_kv_heads, self.cfg.head_dim))
        ms = np.zeros(reps, np.float32)
        out = np.empty((M, self.cfg.n_heads, self.cfg.head_dim), np.uint16)
        inv = np.zeros(4, np.int32) if want_inv else None
        _chk(lib().yka_attn_bench(self._h, _ptr(q), _ptr(k), _ptr(v), M, pos, mode, int(bool(use_graph)), reps, _ptr(ms), _ptr(out), _ptr(inv)))
        return (ms, out.view(np.float16), inv) if want_inv else (ms, out.view(np.float16))


class Pass:
    """A captured sequence of layer calls (the reference replays captured passes, engine35.cpp:1977-1988)."""

    def __init__(self, handle):
        self._h = handle

    def launch(self, stream=0):
        _chk(lib().yka_pass_launch(self._h, stream))

    def close(self):
        if self._h:
            lib().yka_pass_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
