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
                     (dict(n_layers=0), "n_layers"), (dict(max_rows=0), "max_rows")]:
        with pytest.raises(native.YkaError, match=frag):
            native.KvCache(**kw)


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "yasakani_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                src = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in src.replace("no CPU fallback", ""), os.path.join(dirpath, f)
