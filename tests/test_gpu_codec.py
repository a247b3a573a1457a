"""GPU codec vs the oracle: codes, scales and dequantized values must be bit-exact (integer/byte work)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _edge_rows(rng):
    x = rng.standard_normal((512, 128)).astype(np.float32)
    x[0] = 0.0                                           # all-zero groups -> scale 1
    x[1, :32] = 0.0
    x[2] *= 1e-7                                         # fp16 subnormal inputs, scale underflows to 0 -> 1
    x[3] *= 6e-5
    x[4] *= 9000                                         # near fp16 max
    x[5, 7] = 65504.0
    x[6, :8] = [7, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5]   # ties to even at scale 1
    x[6, 8:32] = 0
    x[7:40, ::9] *= 8                                    # outlier channels
    x[40:80] *= (10.0 ** rng.uniform(-5, 3, (40, 1))).astype(np.float32)
    return x.astype(np.float16)


def test_codec_probe_bit_exact(native, oracle):
    rng = np.random.default_rng(21)
    x = _edge_rows(rng)
    codes, scales, y = native.codec_probe(x)
    ocodes, oscales = oracle.quant_rows(x)
    assert (scales == oscales).all()
    assert (codes == ocodes).all()
    assert (y.view(np.uint32) == oracle.dequant_rows(ocodes, oscales).view(np.uint32)).all()


def test_codec_probe_every_fp16_value(native, oracle):
    bits = np.arange(65536, dtype=np.uint16)
    v = bits.view(np.float16)
    v = v[np.isfinite(v)]
    x = np.zeros((v.size // 4, 128), np.float16)
    x.reshape(-1, 32)[:, 0] = v
    x.reshape(-1, 32)[:, 1] = -v / np.float16(3)
    codes, scales, y = native.codec_probe(x)
    ocodes, oscales = oracle.quant_rows(x)
    assert (scales == oscales).all() and (codes == ocodes).all()
    assert (y.view(np.uint32) == oracle.dequant_rows(ocodes, oscales).view(np.uint32)).all()


@pytest.mark.parametrize("paged", [False, True])
def test_append_export_dequant_bit_exact(native, oracle, paged):
    rng = np.random.default_rng(22)
    with native.KvCache(n_layers=2, max_ctx=1024, max_rows=64, paged=paged) as kv:
        if paged:
            kv.set_page_table(np.array([2, 0, 3, 1], np.int32))
        oc = oracle.Cache(1024)
        q = rng.standard_normal((64, 24, 128)).astype(np.float16)
        pos = 0
        for M in (1, 2, 5, 64, 33, 1, 64, 17, 64, 64, 64, 64, 64, 64, 64):   # ragged windows, crossing page boundaries
            k = _edge_rows(rng)[: M * 4].reshape(M, 4, 128)
            v = (rng.standard_normal((M, 4, 128)) * 2).astype(np.float16)
            kv.layer_call(1, q[:M], k, v, pos)
            oc.append(k, v, pos)
            pos += M
        kc, ks, vc, vs = kv.export_rows(1, 0, pos)
        assert (kc == oc.kc[:, :pos]).all() and (ks == oc.ks[:, :pos]).all()
        assert (vc == oc.vc[:, :pos]).all() and (vs == oc.vs[:, :pos]).all()
        kd, vd = kv.dequant_rows(1, 0, pos)
        assert (kd.view(np.uint32) == oracle.dequant_rows(oc.kc[:, :pos], oc.ks[:, :pos]).reshape(kd.shape).view(np.uint32)).all()
        assert (vd.view(np.uint32) == oracle.dequant_rows(oc.vc[:, :pos], oc.vs[:, :pos]).reshape(vd.shape).view(np.uint32)).all()
        # layer 0 was never written
        kc0, ks0, vc0, vs0 = kv.export_rows(0, 0, pos)
        assert not kc0.any() and not ks0.any() and not vc0.any() and not vs0.any()


def test_import_export_round_trip(native, oracle):
    rng = np.random.default_rng(23)
    with native.KvCache(max_ctx=512) as kv:
        kc = rng.integers(0, 256, (4, 300, 64), dtype=np.uint8); vc = rng.integers(0, 256, (4, 300, 64), dtype=np.uint8)
        ks = rng.integers(0, 0x7c00, (4, 300, 4), dtype=np.uint16); vs = rng.integers(0, 0x7c00, (4, 300, 4), dtype=np.uint16)
        kv.import_rows(0, 100, kc, ks, vc, vs)
        a, b, c, d = kv.export_rows(0, 100, 300)
        assert (a == kc).all() and (b == ks).all() and (c == vc).all() and (d == vs).all()
        z = kv.export_rows(0, 0, 100)
        assert not any(t.any() for t in z)


def test_overwrite_rejected_rows(native, oracle):
    # a verify pass writes M rows; after a partial accept the next pass overwrites the rejected ones (engine35.cpp:2414-2425)
    rng = np.random.default_rng(24)
    with native.KvCache(max_ctx=256) as kv:
        oc = oracle.Cache(256)
        q = rng.standard_normal((8, 24, 128)).astype(np.float16)
        k1, v1 = (rng.standard_normal((8, 4, 128)).astype(np.float16) for _ in range(2))
        k2, v2 = (rng.standard_normal((8, 4, 128)).astype(np.float16) for _ in range(2))
        kv.layer_call(0, q, k1, v1, 50); oc.append(k1, v1, 50)
        kv.layer_call(0, q, k2, v2, 53); oc.append(k2, v2, 53)
        got = kv.export_rows(0, 0, 256)
        assert (got[0] == oc.kc).all() and (got[1] == oc.ks).all() and (got[2] == oc.vc).all() and (got[3] == oc.vs).all()


# ---- the reference's own 256-channel row format (rotation, flat int4 MSB-first, int8 rows) ----

@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("rot", [0, 1])
def test_row256_probe_bit_exact(native, oracle, mode, rot):
    yko = oracle
    rng = np.random.default_rng(100 + 2 * mode + rot)
    x = (rng.standard_normal((257, 256)) * rng.uniform(1e-3, 30, size=(257, 1))).astype(np.float32)
    x[7] = 0.0                                           # zero row: scale 1 (int4) / 0 (int8), all codes zero
    x[8, :] = 0.0; x[8, 3] = -5.0                        # a single non-zero element encodes to the extreme code
    x[9] = np.round(x[9])                                # integers: exact butterflies
    q8, words, scales, y = native.kvx256_probe(x, mode, rot)
    rq8, rwords, rscales, ry = yko.kvx_probe256(x, mode, rot)
    assert np.array_equal(scales.view(np.uint32), rscales.view(np.uint32))
    if mode == 0:
        assert np.array_equal(q8, rq8)
    else:
        assert np.array_equal(words, rwords)
    assert np.array_equal(y.view(np.uint32), ry.view(np.uint32))


def test_row256_probe_rejects_bad_arguments(native):
    x = np.zeros((2, 256), np.float32)
    with pytest.raises(native.YkaError):
        native.kvx256_probe(x, 2, 0)
