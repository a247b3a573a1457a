"""Trellis-coded rows on the GPU against the oracle: payload words, scales, projection coefficients, the encoder's
reconstruction and the decoder's rows, all bit for bit.  Synthetic profile blobs (see tests/test_oracle_trellis.py)."""
import numpy as np
import pytest

from yasakani_amd import kvqp

pytestmark = pytest.mark.gpu


def _rows(seed, n):
    rng = np.random.default_rng(seed)
    y = (rng.standard_normal((n, 256)) * rng.uniform(0.05, 6, (n, 1))).astype(np.float32)
    y[:, [5, 77, 130, 201]] *= 8
    y[3] = 0                                                       # rms 0 -> 1, scale from the multiplier alone
    y[4, 1:] = 0
    return y


def _same(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint32), np.ascontiguousarray(b).view(np.uint32))


@pytest.mark.parametrize("kk,mu,dirs,flat", [(5, False, 0, ()), (4, False, 0, ()), (3, False, 0, ()), (5, True, 2, ()), (4, True, 1, (1, 6))])
def test_rows_bit_exact(native, oracle, kk, mu, dirs, flat):
    blob = kvqp.synthetic(layers=2, kk=kk, seed=kk + 10 * dirs, mu=mu, dirs=dirs, flat_groups=flat)
    n = 96
    y = _rows(kk, n)
    grp = (np.arange(n) * 5) % 16
    pos = np.arange(n)
    ref = oracle.tb_encode_rows(blob, grp, pos, y, stride_words=40)
    got = native.tb_pack_unpack(blob, y, grp, pos, stride=160)
    assert ref["coded"].all()
    assert np.array_equal(got["words"], ref["words"])
    assert _same(got["scale"], ref["scale"]) and np.array_equal(got["pc"], ref["pc"])
    assert _same(got["x"], ref["x"])
    assert _same(got["dec"], ref["x"])                             # the decoder reproduces the encoder's row
    assert _same(got["dec"], oracle.tb_decode_rows(blob, grp, ref["words"], ref["scale"], ref["pc"]))


def test_guard_rows_and_missing_groups_pass_through(native, oracle):
    blob = kvqp.synthetic(layers=1, kk=5, seed=4, guard=7)
    y = _rows(9, 24)
    grp = np.arange(24) % 8
    grp[20:] = 99                                                  # no such group
    pos = np.arange(24)                                            # rows 0..6 sit below the guard position
    ref = oracle.tb_encode_rows(blob, grp, pos, y)
    got = native.tb_pack_unpack(blob, y, grp, pos)
    assert not ref["coded"][:7].any() and ref["coded"][7:20].all() and not ref["coded"][20:].any()
    assert _same(got["x"], ref["x"]) and _same(got["dec"], ref["x"])
    assert np.array_equal(got["words"], ref["words"])
    assert _same(got["x"][:7], y[:7]) and _same(got["x"][20:], y[20:])


def test_many_rows_cross_the_launch_tile(native, oracle):
    blob = kvqp.synthetic(layers=1, kk=4, seed=1)
    n = 1100                                                       # more than one launch of 1024 rows
    y = _rows(21, n)
    grp = np.arange(n) % 8
    ref = oracle.tb_encode_rows(blob, grp, np.zeros(n, np.int32), y)
    got = native.tb_pack_unpack(blob, y, grp, np.zeros(n, np.int32))
    assert np.array_equal(got["words"], ref["words"]) and _same(got["scale"], ref["scale"]) and _same(got["x"], ref["x"])


def test_bad_blobs_are_refused(native):
    blob = bytearray(kvqp.synthetic())
    y = np.zeros((1, 256), np.float32)
    bad = bytearray(blob); bad[1] = 0
    with pytest.raises(native.YkaError, match="KVQP"):
        native.tb_pack_unpack(bad, y, [0], [0])
    with pytest.raises(native.YkaError, match="KVQP"):
        native.tb_pack_unpack(blob[:-4], y, [0], [0])
    with pytest.raises(native.YkaError, match="stride"):
        native.tb_pack_unpack(blob, y, [0], [0], stride=128)
