"""MI355X-native int4-KV GQA attention (decode / verify windows / chunked prefill + quantize-on-append).

The package is a thin ctypes mirror of the C ABI in include/yka_abi.h, in the way the reference's
python/yasakani/_native.py mirrors include/yskn_abi.h.  All arithmetic lives in libyka.so (HIP, gfx950);
there is no CPU fallback: importing `yasakani_amd.native` raises if the library has not been built.
"""
__version__ = "0.1.0"

from .build import build_library, library_path  # noqa: F401
