"""bf16 rows at the boundary (option key 11; the reference's activations are bf16, src/q35_kernels.cu:1048,1062) and the
gate rows of the attention-post step.  Inputs are chosen bf16-representable, so the fp16 rows the kernels read are the same
values and the oracle (fed those values) is the reference for both row types."""
import numpy as np
import pytest

from tests.tolerances import assert_attn_close

pytestmark = pytest.mark.gpu


def _bf16_values(x):
    """Values that both 16-bit types hold exactly: bf16-rounded, nothing below 2^-10 in magnitude."""
    from yasakani_amd import native
    y = native.bf16_to_f32(native.bf16_bits(x))
    y[np.abs(y) < 2.0 ** -10] = 0.0
    return y


@pytest.mark.parametrize("M,ctx,head_dim", [(1, 700, 128), (7, 1500, 128), (64, 2000, 128), (150, 300, 128), (1, 500, 256), (16, 900, 256)])
def test_bf16_rows_in_and_out(native, oracle, M, ctx, head_dim):
    rng = np.random.default_rng(9000 + M + ctx)
    D = head_dim
    q = _bf16_values(rng.standard_normal((M, 24, D)).astype(np.float32))
    k = _bf16_values(rng.standard_normal((ctx + M, 4, D)).astype(np.float32))
    v = _bf16_values(rng.standard_normal((ctx + M, 4, D)).astype(np.float32))
    q16, k16, v16 = q.astype(np.float16), k.astype(np.float16), v.astype(np.float16)     # exact: 8 significant bits, |x| < 8
    assert np.array_equal(q16.astype(np.float32), q) and np.array_equal(k16.astype(np.float32), k)
    max_ctx = ((ctx + M + 255) // 256) * 256
    outs = {}
    for bf in (0, 1):
        with native.KvCache(max_ctx=max_ctx, max_rows=max(M, 64), head_dim=D) as kv:
            kv.set_opt(11, bf)
            rows = (lambda a: native.bf16_bits(a.astype(np.float32))) if bf else (lambda a: a)
            for p in range(0, ctx, 512):
                n = min(512, ctx - p)
                kv.append_host(0, rows(k16[p:p + n]), rows(v16[p:p + n]), p)                 # bf16 rows through the append entry too
            outs[bf] = kv.layer_call(0, rows(q16), rows(k16[ctx:]), rows(v16[ctx:]), ctx)
            outs[("cache", bf)] = kv.export_rows(0, 0, ctx + M)
    # the same cache whatever the row type of the inputs
    for a, b in zip(outs[("cache", 0)], outs[("cache", 1)]):
        assert np.array_equal(a, b)
    out16 = outs[0].astype(np.float32)
    outbf = native.bf16_to_f32(outs[1])
    # both round the same fp32 result: bf16(fp16(y)) and bf16(y) differ only where the fp16 rounding lands on a bf16 tie
    # (the 3 bits fp16 keeps beyond bf16 read 100: one value in 8, of which half resolve the other way), and then by one
    # bf16 spacing
    same = native.bf16_bits(out16) == outs[1]
    assert same.mean() > 0.9, same.mean()
    assert (np.abs(outbf - out16) <= 2.0 ** -7 * np.abs(out16) + 2.0 ** -24).all()
    if D == 128:
        oc = oracle.Cache(max_ctx)
        oc.append(k16, v16, 0)
        ref = oc.attend_f32(q16, ctx, threads=8, want_f32=True)[1]
        assert_attn_close(outs[0], ref, f"fp16 rows M={M}")
        err = np.abs(outbf - ref)
        assert (err <= 2e-3 + 2.0 ** -8 * np.abs(ref)).all(), err.max()                      # within the bar plus one bf16 spacing


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("bf", [0, 1])
def test_post_step_writes_gate_rows(native, oracle, head_dim, bf):
    """The gate half of the Q projection leaves as the projection rounded once to the handle's 16-bit row type
    (src/q35_kernels.cu:1030,1048); Q rows in bf16 mode are the same fp32 values rounded to bf16 instead of fp16."""
    rng = np.random.default_rng(9100 + head_dim + bf)
    M, pos, ctx, rd, D = 9, 100, 256, 64, head_dim
    xq = (rng.standard_normal((M, 24, D)) * 2).astype(np.float32)
    xg = (rng.standard_normal((M, 24, D)) * 3).astype(np.float32)
    xk = rng.standard_normal((M, 4, D)).astype(np.float32)
    xv = rng.standard_normal((M, 4, D)).astype(np.float32)
    qw = (rng.standard_normal(D) * 0.1).astype(np.float16)
    kw = (rng.standard_normal(D) * 0.1).astype(np.float16)
    rope = oracle.rope_table(ctx, rd)
    with native.KvCache(max_ctx=ctx, head_dim=D) as kv:
        q_plain = kv.attn_post_host(0, xq, xk, xv, pos, qw, kw, 1e-6, rope, rd, rotate=False)
        rows_plain = kv.export_rows(0, pos, M)
        kv.set_opt(11, bf)
        q, gate = kv.attn_post_host(0, xq, xk, xv, pos, qw, kw, 1e-6, rope, rd, rotate=False, xgate=xg)
        rows = kv.export_rows(0, pos, M)
    if bf:
        assert np.array_equal(gate, native.bf16_bits(xg))
        # Q rows: the value before the final rounding is not visible from outside; it lies within half an fp16 spacing of
        # the fp16 row, so the bf16 row is within one bf16 spacing of it
        qf = native.bf16_to_f32(q)
        assert np.abs(qf - q_plain.astype(np.float32)).max() <= 2.0 ** -8 * np.abs(q_plain.astype(np.float32)).max()
    else:
        assert np.array_equal(gate.view(np.uint16), xg.astype(np.float16).view(np.uint16))
        assert np.array_equal(q.view(np.uint16), q_plain.view(np.uint16))
    for a, b in zip(rows, rows_plain):             # the cache rows do not depend on the row type or on the gate rows
        assert np.array_equal(a, b)
