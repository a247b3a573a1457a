"""Comparison bars for attention outputs (north star: max-abs 2e-3 and relative L2 1e-3 against the reference's
fp32-accumulated math on the same seeded inputs).  Codes, scales and dequantized values are compared bit-exactly."""
import numpy as np

MAX_ABS = 2e-3
REL_L2 = 1e-3


def attn_errors(out, ref):
    a = np.asarray(out, np.float64)
    b = np.asarray(ref, np.float64)
    return float(np.abs(a - b).max()), float(np.linalg.norm(a - b) / np.linalg.norm(b))


def assert_attn_close(out, ref, what=""):
    ma, rl = attn_errors(out, ref)
    assert ma <= MAX_ABS and rl <= REL_L2, f"{what}: max-abs {ma:.3e} (bar {MAX_ABS}), rel-L2 {rl:.3e} (bar {REL_L2})"
    return ma, rl
