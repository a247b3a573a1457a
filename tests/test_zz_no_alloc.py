"""The allocation-free layer call (yka_append_attend_static) against yka_append_attend: same kernels, same split
counts, so outputs and appended rows must agree bit for bit.  Two calls in a row share the GPU's one static workspace;
the second is smaller than the first, so stale partials of the first lie next to the ones it writes.  The handle's own
workspace holds NaN patterns while the static calls run (they must not read it), free device memory is the same before
and after them, and the call is also issued under stream capture - where an allocation is refused - and replayed."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


class _Hip:
    def __init__(self):
        self.rt = ctypes.CDLL("libamdhip64.so")
        self.rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        self.rt.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        self.rt.hipFree.argtypes = [ctypes.c_void_p]
        self.rt.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
        self.rt.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.rt.hipStreamDestroy.argtypes = [ctypes.c_void_p]
        self.rt.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
        self.rt.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
        self.rt.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
        self.rt.hipGraphInstantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        self.rt.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.rt.hipGraphExecDestroy.argtypes = [ctypes.c_void_p]
        self.rt.hipGraphDestroy.argtypes = [ctypes.c_void_p]
        self.bufs = []

    def free_bytes(self):
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        self._ok(self.rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)))
        return free.value

    def _ok(self, rc):
        assert rc == 0, f"HIP error {rc}"

    def alloc(self, nbytes):
        p = ctypes.c_void_p()
        self._ok(self.rt.hipMalloc(ctypes.byref(p), nbytes))
        self.bufs.append(p)
        return p.value

    def upload(self, dptr, arr):
        a = np.ascontiguousarray(arr)
        self._ok(self.rt.hipMemcpy(dptr, a.ctypes.data, a.nbytes, 1))

    def download(self, dptr, arr):
        self._ok(self.rt.hipMemcpy(arr.ctypes.data, dptr, arr.nbytes, 2))

    def sync(self):
        self._ok(self.rt.hipDeviceSynchronize())

    def free_all(self):
        for p in self.bufs:
            self.rt.hipFree(p)
        self.bufs = []


def test_static_workspace_call_equals_the_allocating_one(native, oracle):
    hip = _Hip()
    ctx = 2000
    # (rows, offset of the window inside the new rows): each smaller than the one before; 64 and 16 rows run on the wide
    # kernel, 8 on the kernel whose waves own whole tiles, 2 and 1 on the decode kernel
    calls = [(64, 0), (16, 64), (8, 80), (2, 88), (1, 90)]
    total = sum(m for m, _ in calls)
    _, k_cached, v_cached, k_new, v_new, _ = oracle.make_inputs(4242, ctx, total)
    q_all = oracle.fill_normal_f16(4243, total * 24).view(np.float16).reshape(total, 24, 128)
    try:
        # layer 0 takes the allocating calls, layer 1 (a copy) the static ones
        with native.KvCache(n_layers=2, max_ctx=2304, max_rows=64) as kv:
            for p in range(0, ctx, 64):
                n = min(64, ctx - p)
                kv.append_host(0, k_cached[p:p + n], v_cached[p:p + n], p)
            kv.replicate_layer(0)
            nq, nk = 64 * 24 * 128 * 2, 64 * 4 * 128 * 2
            dq, dk, dv, dpos = hip.alloc(nq), hip.alloc(nk), hip.alloc(nk), hip.alloc(4)
            dout_a, dout_b = hip.alloc(nq), hip.alloc(nq)
            pos = ctx
            shrank = 0
            for M, off in calls:
                q = q_all[off:off + M]
                hip.upload(dq, q.view(np.uint16)); hip.upload(dk, k_new[off:off + M].view(np.uint16)); hip.upload(dv, v_new[off:off + M].view(np.uint16))
                hip.upload(dpos, np.array([pos], np.int32))
                kv.append_attend(0, dq, dk, dv, M, dpos, dout_a)
                hip.sync()
                kv.poison_workspace()                    # the handle's own partials: NaN while the static call runs
                free_before = hip.free_bytes()           # the same kernels have just run for the allocating call: their code is loaded
                kv.append_attend_static(1, dq, dk, dv, M, dpos, dout_b)
                hip.sync()
                shrank += max(0, free_before - hip.free_bytes())
                a = np.empty((M, 24, 128), np.uint16); b = np.empty((M, 24, 128), np.uint16)
                hip.download(dout_a, a); hip.download(dout_b, b)
                assert (a == b).all(), f"outputs differ at M={M}"
                for x, y in zip(kv.export_rows(0, pos, M), kv.export_rows(1, pos, M)):
                    assert (x == y).all(), f"appended rows differ at M={M}"
                pos += M
            # free device memory read right before and right after every static call: a workspace allocated behind the caller's
            # back would be 26 MB (the handle's) or 9.7 MB (the static array's size)
            assert shrank == 0, f"free device memory shrank by {shrank} bytes over the static calls"
            # the same call recorded under stream capture (an allocation there is refused) and replayed twice, with eager
            # work in between; layer 1 holds the rows already, the replays store the same rows again
            M, off = calls[1]
            pos_c = ctx + calls[0][0]
            hip.upload(dq, q_all[off:off + M].view(np.uint16)); hip.upload(dk, k_new[off:off + M].view(np.uint16)); hip.upload(dv, v_new[off:off + M].view(np.uint16))
            hip.upload(dpos, np.array([pos_c], np.int32))
            kv.append_attend(0, dq, dk, dv, M, dpos, dout_a)
            hip.sync()
            want = np.empty((M, 24, 128), np.uint16); hip.download(dout_a, want)
            st, graph, gexec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
            hip._ok(hip.rt.hipStreamCreate(ctypes.byref(st)))
            try:
                kv.poison_workspace()
                hip._ok(hip.rt.hipStreamBeginCapture(st, 0))                 # global mode: unsafe calls (allocations) fail
                try:
                    kv.append_attend_static(1, dq, dk, dv, M, dpos, dout_b, None, st.value)
                finally:
                    rc_end = hip.rt.hipStreamEndCapture(st, ctypes.byref(graph))
                hip._ok(rc_end)
                hip._ok(hip.rt.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, 0))
                for replay in range(2):
                    hip.upload(dout_b, np.zeros((M, 24, 128), np.uint16))
                    hip._ok(hip.rt.hipGraphLaunch(gexec, st))
                    hip._ok(hip.rt.hipStreamSynchronize(st))
                    got = np.empty((M, 24, 128), np.uint16); hip.download(dout_b, got)
                    assert (got == want).all(), f"replay {replay} of the captured static call differs"
                    kv.append_attend_static(1, dq, dk, dv, M, dpos, dout_b)      # eager work between the replays
                    hip.sync()
            finally:
                if gexec: hip.rt.hipGraphExecDestroy(gexec)
                if graph: hip.rt.hipGraphDestroy(graph)
                hip.rt.hipStreamDestroy(st)
            # and the allocating call is what the oracle says (so both are)
            from tests.tolerances import assert_attn_close
            oc = oracle.Cache(2304)
            n = pos
            oc.kc[:, :n], oc.ks[:, :n], oc.vc[:, :n], oc.vs[:, :n] = kv.export_rows(1, 0, n)
            M, off = calls[-1]
            assert_attn_close(b.view(np.float16), oc.attend_f32(q_all[off:off + M], pos - M, threads=4, want_f32=True)[1], "last static call")
            # with the merge of the decode splits inside the launch (option key 7) the static call takes its split tickets
            # from the static array too (all zero after every launch): two calls in a row, against the allocating call
            kv.set_opt(7, 1)
            for M, off in ((2, 80), (1, 82), (1, 80)):
                hip.upload(dq, q_all[off:off + M].view(np.uint16)); hip.upload(dk, k_new[off:off + M].view(np.uint16)); hip.upload(dv, v_new[off:off + M].view(np.uint16))
                hip.upload(dpos, np.array([ctx + off], np.int32))
                kv.append_attend(0, dq, dk, dv, M, dpos, dout_a)
                kv.append_attend_static(1, dq, dk, dv, M, dpos, dout_b)
                hip.sync()
                a = np.empty((M, 24, 128), np.uint16); b = np.empty((M, 24, 128), np.uint16)
                hip.download(dout_a, a); hip.download(dout_b, b)
                assert (a == b).all(), f"outputs differ at M={M} with the merge inside the launch"
            kv.set_opt(7, 0)
            # limits are refused with a message, before anything is launched
            with pytest.raises(native.YkaError, match="64 rows"):
                kv.append_attend_static(1, dq, dk, dv, 65, dpos, dout_b)
        with native.KvCache(head_dim=256, max_ctx=512, max_rows=8) as kv256:
            with pytest.raises(native.YkaError, match="head_dim 128"):
                kv256.append_attend_static(0, dq, dk, dv, 1, dpos, dout_b)
    finally:
        hip.sync()
        hip.free_all()
