"""The C-ABI library loads without a GPU and exports every entry point that include/yka_abi.h declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "yka_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"YKA_API[^;(]*?\b(yka_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points(native):
    assert _declared() == sorted(native.EXPORTS)


def test_library_exports_every_declared_symbol(native):
    lib = ctypes.CDLL(native.library_path())
    for name in _declared():
        assert hasattr(lib, name), name


def test_build_info_and_error_string_without_gpu(native):
    info = native.build_info()
    assert "arch=gfx950" in info and "page_tokens=256" in info
    assert native.lib().yka_last_error() is not None


def test_bad_config_is_rejected_with_a_message(native):
    # validation happens before any device call, so this runs without a GPU
    for kw, frag in [(dict(head_dim=64), "head_dim"), (dict(n_heads=28), "n_heads"), (dict(max_ctx=1000), "max_ctx"),
                     (dict(n_layers=0), "n_layers"), (dict(max_rows=0), "max_rows"),
                     (dict(n_layers=1 << 20, max_ctx=1 << 30), "1 TiB"), (dict(n_heads=6 * 2048, n_kv_heads=2048), "n_kv_heads")]:
        with pytest.raises(native.YkaError, match=frag):
            native.KvCache(**kw)


def test_profile_blobs_are_checked_before_any_device_call(native):
    """Every corruption below is refused by the host-side parser of the profile blob (magic, version, length, element
    count, multiplier count, offsets, table geometry, table range, group records), so this runs without a GPU."""
    import struct

    import numpy as np

    from yasakani_amd import kvqp
    good = kvqp.synthetic(layers=1, kk=5, seed=3, mu=True, dirs=1)
    info = kvqp.parse(good)
    y = np.zeros((1, 256), np.float32)

    def refused(blob, frag):
        with pytest.raises(native.YkaError, match=frag):
            native.tb_pack_unpack(bytes(blob), y, [0], [0])

    off_m, off_t, off_g = struct.unpack_from("<III", good, 32)
    (t0,) = struct.unpack_from("<I", good, off_t)
    (g0,) = struct.unpack_from("<I", good, off_g)
    assert info is not None and good[:4] == b"KVQP"
    b = bytearray(good); b[0] = ord("X"); refused(b, "KVQP")
    b = bytearray(good); struct.pack_into("<H", b, 4, 2); refused(b, "KVQP")                      # version
    refused(good[:-1], "KVQP")                                                                     # length field disagrees
    refused(good[:60], "KVQP")                                                                     # shorter than a header
    b = bytearray(good); struct.pack_into("<H", b, 16, 128); refused(b, "256 elements")
    b = bytearray(good); struct.pack_into("<H", b, 24, 0); refused(b, "multiplier count")
    b = bytearray(good); struct.pack_into("<H", b, 24, 17); refused(b, "multiplier count")
    b = bytearray(good); struct.pack_into("<I", b, 40, len(good) - 2); refused(b, "offsets outside")
    for count in (1 << 30, 1 << 31, 0xFFFFFFFF):                                                   # group count (also as a negative int)
        b = bytearray(good); struct.pack_into("<I", b, 28, count); refused(b, "offsets outside")
    b = bytearray(good); b[t0] = 7; refused(b, "8 state bits")
    b = bytearray(good); b[t0 + 2] = 32; refused(b, "chunks of 64")
    b = bytearray(good); struct.pack_into("<h", b, t0 + 12 + 2 * 100, 1101); refused(b, "out of range")
    b = bytearray(good); struct.pack_into("<h", b, t0 + 12 + 2 * 5, -1101); refused(b, "out of range")
    b = bytearray(good); struct.pack_into("<I", b, off_t, len(good) - 100); refused(b, "tables must have|out of range|state bits")
    b = bytearray(good); struct.pack_into("<I", b, off_g, len(good) - 4); refused(b, "group record")
    b = bytearray(good); b[g0] = 2; refused(b, "bad group record")                                 # mode
    b = bytearray(good); b[g0 + 4] = 3; refused(b, "bad group record")                             # directions
    b = bytearray(good); b[g0 + 1] = 6; refused(b, "3..5 bits")
    b = bytearray(good); b[g0 + 1] = 2; refused(b, "3..5 bits")
    b = bytearray(good); b[g0 + 2] = 9; refused(b, "3..5 bits and a table")                        # table index
    with pytest.raises(native.YkaError, match="stride"):
        native.tb_pack_unpack(good, y, [0], [0], stride=128)


def test_probe_entry_points_refuse_bad_arguments_before_any_device_call(native):
    import numpy as np
    L = native.lib()
    x = np.zeros((2, 256), np.float32); y = np.zeros_like(x); sc = np.zeros(2, np.float32)
    q8 = np.zeros((2, 256), np.int8); words = np.zeros((2, 32), np.uint32)
    P = native._ptr

    def refused(rc, frag):
        assert rc != 0 and frag in L.yka_last_error().decode()

    refused(L.yka_kvx256_probe(None, 2, 0, 0, P(q8), None, P(sc), P(y)), "bad argument")
    refused(L.yka_kvx256_probe(P(x), 0, 0, 0, P(q8), None, P(sc), P(y)), "bad argument")
    refused(L.yka_kvx256_probe(P(x), -5, 1, 0, None, P(words), P(sc), P(y)), "bad argument")
    refused(L.yka_kvx256_probe(P(x), 2, 2, 0, P(q8), P(words), P(sc), P(y)), "bad argument")
    refused(L.yka_kvx256_probe(P(x), 2, 0, 0, None, P(words), P(sc), P(y)), "selected mode")
    refused(L.yka_kvx256_probe(P(x), 2, 1, 1, P(q8), None, P(sc), P(y)), "selected mode")
    from yasakani_amd import kvqp
    blob = np.frombuffer(kvqp.synthetic(), np.uint8)
    grp = np.zeros(2, np.int32); pay = np.zeros((2, 160), np.uint8); side = np.zeros((2, 2), np.uint32)
    refused(L.yka_tb_pack_unpack(P(blob), blob.size, None, P(grp), P(grp), 2, 160, P(y), P(pay), P(side), P(x), None), "bad argument")
    refused(L.yka_tb_pack_unpack(P(blob), blob.size, P(x), P(grp), P(grp), 0, 160, P(y), P(pay), P(side), P(x), None), "bad argument")
    refused(L.yka_tb_pack_unpack(P(blob), blob.size, P(x), P(grp), P(grp), 2, 162, P(y), P(pay), P(side), P(x), None), "stride")
    refused(L.yka_tb_pack_unpack(P(blob), blob.size, P(x), P(grp), P(grp), 2, 2048, P(y), P(pay), P(side), P(x), None), "stride")
    refused(L.yka_tb_pack_unpack(None, 0, P(x), P(grp), P(grp), 2, 160, P(y), P(pay), P(side), P(x), None), "KVQP")


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "yasakani_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                src = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in src.replace("no CPU fallback", ""), os.path.join(dirpath, f)
