"""The allocation-free attention entry point (lg_hip_attention_noalloc) against the entry point it is a
variant of (lg_hip_attention), through the C ABI: bit-identical outputs on two calls in a row, the second
on a smaller input (the built-in working array keeps the first call's contents), and a shape that does
not fit the array refused.  The test plays the caller: it brings its inputs and its output as device memory,
allocated up front with the HIP runtime the library itself is linked to."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


class DeviceBuffers:
    """hipMalloc / hipMemcpy / hipFree of the already loaded HIP runtime, for the caller's side of the call."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so.7")
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.held = []

    def upload(self, arr):
        p = C.c_void_p()
        assert self.rt.hipMalloc(C.byref(p), max(arr.nbytes, 16)) == 0
        self.held.append(p)
        assert self.rt.hipMemcpy(p, arr.ctypes.data_as(C.c_void_p), arr.nbytes, 1) == 0       # host to device
        return p

    def download(self, p, arr):
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemcpy(arr.ctypes.data_as(C.c_void_p), p, arr.nbytes, 2) == 0       # device to host

    def free(self):
        for p in self.held:
            self.rt.hipFree(p)
        self.held = []


def noalloc(H, mem, q, kc, vc, n_head, n_head_kv, hd, window, pos):
    dq, dk, dv = mem.upload(q), mem.upload(kc), mem.upload(vc)
    out = np.full(q.shape, np.nan, np.float32)
    dout = mem.upload(out)
    H.lg_hip_attention_noalloc.argtypes = [C.c_void_p] * 3 + [C.c_int] * 7 + [C.c_void_p, C.c_void_p]
    rc = H.lg_hip_attention_noalloc(dq, dk, dv, q.shape[0], n_head, n_head_kv, hd, kc.shape[0], window, pos, dout, None)
    mem.download(dout, out)
    mem.free()
    return rc, out


def test_noalloc_attention_equals_the_allocating_entry_point(lg, gpu_required):
    H = lg.hiplib.load_hip()
    mem = DeviceBuffers()
    H.lg_hip_attention_noalloc_limit.restype = C.c_size_t
    assert H.lg_hip_attention_noalloc_limit() == 8 << 20
    rng = np.random.default_rng(77)
    # first call: config-3 shape (ctx 4096 global, 5 rows); second: a smaller sliding one, fewer rows and heads
    for (n_head, n_head_kv, hd, rows, seq, window, pos) in ((8, 2, 256, 5, 4104, 0, 4091), (4, 2, 128, 2, 160, 128, 300)):
        kc = rng.normal(0, 1, (seq, n_head_kv * hd)).astype(np.float16).view(np.uint16)
        vc = rng.normal(0, 1, (seq, n_head_kv * hd)).astype(np.float16).view(np.uint16)
        q = (rng.normal(0, 1, (rows, n_head * hd)) * 0.08).astype(np.float32)
        print(f"noalloc attention H={n_head} KV={n_head_kv} hd={hd} rows={rows} seq={seq} window={window} pos={pos}", flush=True)
        want, _ = lg.hiplib.attention(q, kc, vc, n_head, n_head_kv, hd, window, pos)
        rc, got = noalloc(H, mem, q, kc, vc, n_head, n_head_kv, hd, window, pos)
        assert rc == 0, H.lg_hip_last_error()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # a shape whose tile partials exceed the array is refused, with the sizes in the message
    seq = 16400
    kc = np.zeros((seq, 8 * 256), np.uint16)
    q = np.zeros((8, 16 * 256), np.float32)
    rc, _ = noalloc(H, mem, q, kc, kc, 16, 8, 256, 0, seq - 8)
    assert rc == -2 and b"working memory" in H.lg_hip_last_error()
