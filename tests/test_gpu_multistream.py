"""Multi-stream passes (batched decode): every row of a pass names its own KV container and position.  Checked against the
oracle run stream by stream on the same rows."""
import numpy as np
import pytest

from tolerances import assert_attn_close

pytestmark = pytest.mark.gpu

CTX = 1024
LENS = [300, 17, 900, 512, 0]                             # cached tokens per stream; the last stream is empty


def _streams(native, oracle, paged, seed=3):
    rng = np.random.default_rng(seed)
    kv = native.KvCache(n_layers=len(LENS), max_ctx=CTX, max_rows=64, paged=paged)
    if paged:
        for s in range(len(LENS)):
            kv.set_page_table(rng.permutation(CTX // 256).astype(np.int32), layer=s)
    refs = []
    for s, n in enumerate(LENS):
        ref = oracle.Cache(CTX)
        if n:
            _, k, v, _, _, _ = oracle.make_inputs(seed * 100 + s, n, 1)
            kv.append_host(s, k, v, 0)
            ref.append(k, v, 0)
        refs.append(ref)
    return kv, refs, rng


def _rows(rng, M):
    q = rng.standard_normal((M, 24, 128)).astype(np.float16)
    k = rng.standard_normal((M, 4, 128)).astype(np.float16)
    v = rng.standard_normal((M, 4, 128)).astype(np.float16)
    return q, k, v


@pytest.mark.parametrize("paged", [False, True])
def test_one_row_per_stream(native, oracle, paged):
    kv, refs, rng = _streams(native, oracle, paged)
    with kv:
        slots = np.array([2, 0, 4, 1, 3], np.int32)       # any order
        pos = np.array([LENS[s] for s in slots], np.int32)
        q, k, v = _rows(rng, len(slots))
        out = kv.ms_call(q, k, v, pos, slots)
        for t, s in enumerate(slots):
            refs[s].append(k[t:t + 1], v[t:t + 1], int(pos[t]))
            expect = refs[s].attend_f32(q[t:t + 1], int(pos[t]))
            assert_attn_close(out[t:t + 1], expect, f"row {t} stream {s}")
            # the appended row is what the single-stream append stores
            got = kv.export_rows(int(s), int(pos[t]), 1)
            assert np.array_equal(got[0], refs[s].kc[:, pos[t]:pos[t] + 1]) and np.array_equal(got[3], refs[s].vs[:, pos[t]:pos[t] + 1])


def test_rows_of_one_stream_follow_each_other(native, oracle):
    kv, refs, rng = _streams(native, oracle, False)
    with kv:
        # stream 0: its last token and two draft tokens; stream 2: one row; stream 0 rows see each other's keys
        slots = np.array([0, 0, 0, 2], np.int32)
        pos = np.array([300, 301, 302, 900], np.int32)
        q, k, v = _rows(rng, 4)
        out = kv.ms_call(q, k, v, pos, slots)
        refs[0].append(k[0:3], v[0:3], 300)
        assert_attn_close(out[0:3], refs[0].attend_f32(q[0:3], 300), "stream 0 window")     # row t sees keys [0, 300 + t]
        refs[2].append(k[3:4], v[3:4], 900)
        assert_attn_close(out[3:4], refs[2].attend_f32(q[3:4], 900), "stream 2")


@pytest.mark.parametrize("merge_in_launch", [0, 1])
def test_more_rows_than_sixteen_and_attend_only(native, oracle, merge_in_launch):
    kv, refs, rng = _streams(native, oracle, False)
    with kv:
        kv.set_opt(7, merge_in_launch)
        M = 24
        slots = (np.arange(M) % 4).astype(np.int32)
        pos = np.array([LENS[s] - 1 - (t // 4) for t, s in enumerate(slots)], np.int32)     # positions inside the cached part
        q, _, _ = _rows(rng, M)
        out = kv.ms_call(q, None, None, pos, slots)
        for t, s in enumerate(slots):
            assert_attn_close(out[t:t + 1], refs[s].attend_f32(q[t:t + 1], int(pos[t])), f"row {t}")


@pytest.mark.parametrize("merge_in_launch", [0, 1])
def test_rejected_rows_yield_zeros_and_touch_nothing(native, oracle, merge_in_launch):
    kv, refs, rng = _streams(native, oracle, False)
    with kv:
        kv.set_opt(7, merge_in_launch)                    # the last workgroup of a column merges the splits / the combiner launch does
        slots = np.array([1, 9, 3, -1, 2], np.int32)
        pos = np.array([17, 5, -4, 5, CTX], np.int32)     # only row 0 is valid
        q, k, v = _rows(rng, 5)
        before = kv.export_rows(2, 0, CTX)
        out = kv.ms_call(q, k, v, pos, slots)
        assert not np.any(out[1:].view(np.uint16) & 0x7fff)
        refs[1].append(k[0:1], v[0:1], 17)
        assert_attn_close(out[0:1], refs[1].attend_f32(q[0:1], 17), "valid row")
        after = kv.export_rows(2, 0, CTX)
        for a, b in zip(before, after):
            assert np.array_equal(a, b)
        with pytest.raises(native.YkaError):
            kv.ms_call(q, k, None, pos, slots)


# ---- the same passes over the reference's own 256-channel rows (handles opened with head_dim = 256) ----

def _streams256(native, oracle, paged, seed=5):
    rng = np.random.default_rng(seed)
    kv = native.KvCache(n_layers=len(LENS), head_dim=256, max_ctx=CTX, max_rows=64, paged=paged)
    if paged:
        for s in range(len(LENS)):
            kv.set_page_table(rng.permutation(CTX // 256).astype(np.int32), layer=s)
    refs = []
    for s, n in enumerate(LENS):
        ref = oracle.Cache(CTX, 24, 4, 256)
        if n:
            k = rng.standard_normal((n, 4, 256)).astype(np.float16)
            k[:, :, [5, 77, 130, 201]] *= 8
            v = rng.standard_normal((n, 4, 256)).astype(np.float16)
            for p in range(0, n, 64):
                kv.append_host(s, k[p:p + 64], v[p:p + 64], p)
            ref.append(k, v, 0)
        refs.append(ref)
    return kv, refs, rng


def _rows256(rng, M):
    return tuple(rng.standard_normal((M, h, 256)).astype(np.float16) for h in (24, 4, 4))


@pytest.mark.parametrize("paged", [False, True])
def test_one_row_per_stream_256(native, oracle, paged):
    kv, refs, rng = _streams256(native, oracle, paged)
    with kv:
        slots = np.array([2, 0, 4, 1, 3], np.int32)
        pos = np.array([LENS[s] for s in slots], np.int32)
        q, k, v = _rows256(rng, len(slots))
        out = kv.ms_call(q, k, v, pos, slots)
        for t, s in enumerate(slots):
            refs[s].append(k[t:t + 1], v[t:t + 1], int(pos[t]))
            assert_attn_close(out[t:t + 1], refs[s].attend_f32(q[t:t + 1], int(pos[t])), f"row {t} stream {s}")
            got = kv.export_rows(int(s), int(pos[t]), 1)
            assert np.array_equal(got[0], refs[s].kc[:, pos[t]:pos[t] + 1]) and np.array_equal(got[2], refs[s].vc[:, pos[t]:pos[t] + 1])
            assert np.array_equal(got[1].view(np.uint32), refs[s].ks[:, pos[t]:pos[t] + 1].view(np.uint32))
            assert np.array_equal(got[3].view(np.uint32), refs[s].vs[:, pos[t]:pos[t] + 1].view(np.uint32))


def test_rows_of_one_stream_and_bad_rows_256(native, oracle):
    kv, refs, rng = _streams256(native, oracle, False)
    with kv:
        # stream 0: its last token and two draft tokens (they see each other's keys); stream 2: one row; a row whose slot
        # does not exist and one whose position lies outside its container yield zeros and write nothing
        slots = np.array([0, 0, 0, 2, 9, 1], np.int32)
        pos = np.array([300, 301, 302, 900, 5, CTX], np.int32)
        q, k, v = _rows256(rng, 6)
        out = kv.ms_call(q, k, v, pos, slots)
        refs[0].append(k[0:3], v[0:3], 300)
        assert_attn_close(out[0:3], refs[0].attend_f32(q[0:3], 300), "stream 0 window")
        refs[2].append(k[3:4], v[3:4], 900)
        assert_attn_close(out[3:4], refs[2].attend_f32(q[3:4], 900), "stream 2")
        assert not out[4:6].view(np.uint16).any()
        # attend only, more rows than the reference's 16-row cap
        M = 20
        slots = np.array([s % 4 for s in range(M)], np.int32)
        pos = np.array([max(0, LENS[s] - 1 - t) for t, s in enumerate(slots)], np.int32)
        q = rng.standard_normal((M, 24, 256)).astype(np.float16)
        out = kv.ms_call(q, None, None, pos, slots)
        for t, s in enumerate(slots):
            if LENS[s] + (3 if s == 0 else 1 if s == 2 else 0) > pos[t]:
                assert_attn_close(out[t:t + 1], refs[s].attend_f32(q[t:t + 1], int(pos[t])), f"attend-only row {t}")
