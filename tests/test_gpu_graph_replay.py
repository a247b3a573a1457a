"""A captured pass replayed several times at advancing positions, with eager layer calls and synchronisations between the
replays: every replay must equal the eager result on twin containers bit for bit (same kernels, same split counts), and
the rows it appended must equal the eager ones.  Device buffers are plain hipMalloc allocations made through ctypes on
the HIP runtime the library itself uses."""
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
        self.bufs = []

    def _ok(self, rc):
        assert rc == 0, f"HIP error {rc}"

    def alloc(self, nbytes):
        p = ctypes.c_void_p()
        self._ok(self.rt.hipMalloc(ctypes.byref(p), nbytes))
        self.bufs.append(p)
        return p.value

    def upload(self, dptr, arr):
        a = np.ascontiguousarray(arr)
        self._ok(self.rt.hipMemcpy(dptr, a.ctypes.data, a.nbytes, 1))     # hipMemcpyHostToDevice (synchronous)

    def download(self, dptr, arr):
        self._ok(self.rt.hipMemcpy(arr.ctypes.data, dptr, arr.nbytes, 2))  # hipMemcpyDeviceToHost

    def sync(self):
        self._ok(self.rt.hipDeviceSynchronize())

    def free_all(self):
        for p in self.bufs:
            self.rt.hipFree(p)
        self.bufs = []


@pytest.mark.parametrize("M", [1, 2, 16])
def test_captured_pass_replays(native, oracle, M):
    hip = _Hip()
    ctx, steps = 900, 4
    _, k_cached, v_cached, k_new, v_new, _ = oracle.make_inputs(500 + M, ctx, steps * M)
    qs = oracle.fill_normal_f16(77 + M, steps * M * 24).view(np.float16).reshape(steps, M, 24, 128)
    with native.KvCache(n_layers=4, max_ctx=1280, max_rows=64) as kv:
        for p in range(0, ctx, 64):
            n = min(64, ctx - p)
            kv.append_host(0, k_cached[p:p + n], v_cached[p:p + n], p)
        kv.replicate_layer(0)
        nq, nk = M * 24 * 128 * 2, M * 4 * 128 * 2
        dq, dk, dv, dout, dpos = hip.alloc(nq), hip.alloc(nk), hip.alloc(nk), hip.alloc(nq), hip.alloc(4)
        graph = kv.capture_pass([0, 1], dq, dk, dv, M, dpos, dout)
        for s in range(steps):
            pos = ctx + s * M
            qh = qs[s]; kh = k_new[s * M:(s + 1) * M]; vh = v_new[s * M:(s + 1) * M]
            hip.upload(dq, qh); hip.upload(dk, kh); hip.upload(dv, vh); hip.upload(dpos, np.array([pos], np.int32))
            graph.launch(0)
            hip.sync()
            got = np.empty((M, 24, 128), np.float16)
            hip.download(dout, got)
            # eager work between the replays, on the twin containers
            kv.layer_call(2, qh, kh, vh, pos)
            eager = kv.layer_call(3, qh, kh, vh, pos)
            assert np.array_equal(got.view(np.uint16), eager.view(np.uint16)), f"replay {s}"
            for a, b in zip(kv.export_rows(1, pos, M), kv.export_rows(3, pos, M)):
                assert np.array_equal(a, b), f"rows of replay {s}"
        graph.close()
        hip.free_all()
        # the last position against the oracle as well
        ref = oracle.Cache(1280)
        ref.append(k_cached, v_cached, 0)
        ref.append(k_new, v_new, ctx)
        from tolerances import assert_attn_close
        assert_attn_close(got, ref.attend_f32(qs[steps - 1], ctx + (steps - 1) * M), "last replay")
