"""The allocation-free attention entry point (lg_hip_attention_noalloc) through the C ABI, against the CPU
oracle's attention (lgo_attention_f16, per row and head) and against the entry point it is a variant of
(lg_hip_attention): bit-identical outputs on two calls in a row, the second on a smaller input (the built-in
working array keeps the first call's contents); a shape that does not fit the array refused; and the call
recorded into a HIP graph whose replays, with new queries between them, are each checked like the eager calls.
The test plays the caller: it brings its inputs and its output as device memory, allocated up front with the
HIP runtime the library itself is linked to."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def loaded_hip_runtime():
    """Path of the HIP runtime that this process has mapped (the one the library under test is linked to)."""
    with open("/proc/self/maps") as f:
        for line in f:
            path = line.split()[-1]
            if os.path.basename(path).startswith("libamdhip64.so"):
                return path
    raise RuntimeError("no libamdhip64 is mapped: load the library under test first")


class DeviceBuffers:
    """hipMalloc / hipMemcpy / hipFree of the already loaded HIP runtime, for the caller's side of the call."""

    def __init__(self):
        self.rt = C.CDLL(loaded_hip_runtime())
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


NOALLOC_ARGS = [C.c_void_p] * 3 + [C.c_int] * 7 + [C.c_void_p, C.c_void_p]


def noalloc(H, mem, q, kc, vc, n_head, n_head_kv, hd, window, pos):
    dq, dk, dv = mem.upload(q), mem.upload(kc), mem.upload(vc)
    out = np.full(q.shape, np.nan, np.float32)
    dout = mem.upload(out)
    H.lg_hip_attention_noalloc.argtypes = NOALLOC_ARGS
    rc = H.lg_hip_attention_noalloc(dq, dk, dv, q.shape[0], n_head, n_head_kv, hd, kc.shape[0], window, pos, dout, None)
    mem.download(dout, out)
    mem.free()
    return rc, out


def oracle_attention(ob, q, kc, vc, n_head, n_head_kv, hd, window, pos):
    """The oracle's attention of one (row, head) at a time: row j is the query at position pos + j and sees the
    keys from its window's start up to itself, in the kernels' tile order with the exact exponential."""
    L = ob.lib()
    rows, seq, kd = q.shape[0], kc.shape[0], n_head_kv * hd
    out = np.zeros_like(q)
    for j in range(rows):
        pj = pos + j
        start = max(0, pj - window + 1) if window else 0
        for h in range(n_head):
            o = np.zeros(hd, np.float32)
            L.lgo_attention_f16(o, np.ascontiguousarray(q[j, h * hd:(h + 1) * hd]), kc.reshape(-1), vc.reshape(-1),
                                hd, kd, h // (n_head // n_head_kv), seq, start, pj, 1, 1)
            out[j, h * hd:(h + 1) * hd] = o
    return out


# first call: config-3 shape (ctx 4096 global, 5 rows); second: a smaller sliding one, fewer rows and heads
SHAPES = ((8, 2, 256, 5, 4104, 0, 4091), (4, 2, 128, 2, 160, 128, 300))


def inputs(rng, n_head, n_head_kv, hd, rows, seq):
    kc = rng.normal(0, 1, (seq, n_head_kv * hd)).astype(np.float16).view(np.uint16)
    vc = rng.normal(0, 1, (seq, n_head_kv * hd)).astype(np.float16).view(np.uint16)
    q = (rng.normal(0, 1, (rows, n_head * hd)) * 0.08).astype(np.float32)
    return q, kc, vc


def test_noalloc_attention_equals_the_oracle_and_the_allocating_entry_point(lg, ob, gpu_required):
    H = lg.hiplib.load_hip()
    mem = DeviceBuffers()
    H.lg_hip_attention_noalloc_limit.restype = C.c_size_t
    assert H.lg_hip_attention_noalloc_limit() == 8 << 20
    rng = np.random.default_rng(77)
    for (n_head, n_head_kv, hd, rows, seq, window, pos) in SHAPES:
        q, kc, vc = inputs(rng, n_head, n_head_kv, hd, rows, seq)
        print(f"noalloc attention H={n_head} KV={n_head_kv} hd={hd} rows={rows} seq={seq} window={window} pos={pos}", flush=True)
        rc, got = noalloc(H, mem, q, kc, vc, n_head, n_head_kv, hd, window, pos)
        assert rc == 0, H.lg_hip_last_error()
        want = oracle_attention(ob, q, kc, vc, n_head, n_head_kv, hd, window, pos)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        other, _ = lg.hiplib.attention(q, kc, vc, n_head, n_head_kv, hd, window, pos)
        assert np.array_equal(got.view(np.uint32), other.view(np.uint32))
    # a shape whose tile partials exceed the array is refused, with the sizes in the message
    seq = 16400
    kc = np.zeros((seq, 8 * 256), np.uint16)
    q = np.zeros((8, 16 * 256), np.float32)
    rc, _ = noalloc(H, mem, q, kc, kc, 16, 8, 256, 0, seq - 8)
    assert rc == -2 and b"working memory" in H.lg_hip_last_error()


def test_noalloc_attention_recorded_into_a_graph(lg, ob, gpu_required):
    """After lg_hip_attention_noalloc_init the entry point makes no runtime call but kernel launches, so a stream
    under capture can take it.  The graph is replayed three times; before each replay the caller overwrites the
    queries (an eager copy, with a device synchronisation), and every replay's output is the oracle's."""
    H = lg.hiplib.load_hip()
    mem = DeviceBuffers()
    rt = mem.rt
    assert H.lg_hip_attention_noalloc_init() == 0, H.lg_hip_last_error()
    n_head, n_head_kv, hd, rows, seq, window, pos = 8, 2, 256, 4, 640, 512, 1000
    rng = np.random.default_rng(78)
    q, kc, vc = inputs(rng, n_head, n_head_kv, hd, rows, seq)
    out = np.full(q.shape, np.nan, np.float32)
    dq, dk, dv, dout = mem.upload(q), mem.upload(kc), mem.upload(vc), mem.upload(out)
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert rt.hipStreamCreateWithFlags(C.byref(stream), 1) == 0                       # non-blocking
    H.lg_hip_attention_noalloc.argtypes = NOALLOC_ARGS
    print("noalloc attention under capture", flush=True)
    assert rt.hipStreamBeginCapture(stream, 0) == 0                                   # global mode: the strictest
    rc = H.lg_hip_attention_noalloc(dq, dk, dv, rows, n_head, n_head_kv, hd, seq, window, pos, dout, stream)
    end = rt.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0, H.lg_hip_last_error()
    assert end == 0 and graph.value
    rt.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    assert rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    rt.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    for replay in range(3):
        print(f"replay {replay}", flush=True)
        q = (rng.normal(0, 1, q.shape) * 0.08).astype(np.float32)
        assert rt.hipMemcpy(dq, q.ctypes.data_as(C.c_void_p), q.nbytes, 1) == 0
        assert rt.hipDeviceSynchronize() == 0
        assert rt.hipGraphLaunch(gexec, stream) == 0
        mem.download(dout, out)
        want = oracle_attention(ob, q, kc, vc, n_head, n_head_kv, hd, window, pos)
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    rt.hipGraphExecDestroy.argtypes = [C.c_void_p]
    rt.hipGraphDestroy.argtypes = [C.c_void_p]
    rt.hipStreamDestroy.argtypes = [C.c_void_p]
    rt.hipGraphExecDestroy(gexec); rt.hipGraphDestroy(graph); rt.hipStreamDestroy(stream)
    mem.free()
