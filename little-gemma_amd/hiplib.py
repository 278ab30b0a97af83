"""ctypes bindings of the product libraries:

* csrc/liblg_hip.so        the gfx950 kernels behind the C ABI of include/lg_hip.h
* host/liblg_modelhip.so   the reference's model.h backend interface implemented on that ABI
                           (model-hip.c) plus the session helpers (session.c)

There is no CPU fallback: without the built libraries or without a GPU these calls raise.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
MAX_ROWS = 8
INFO_KEYS = ("n_layer", "n_embd", "n_head", "n_vocab", "ple", "n_kv_start", "window", "n_ff", "n_head_kv",
             "head_dim_swa", "head_dim_full", "n_ctx")

f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")

_hip = None
_backend = None


class HipError(RuntimeError):
    pass


def build():
    """Compile the HIP library for gfx950 and the C backend on top of it."""
    subprocess.run(["make", "-C", CSRC, "-B", "liblg_hip.so"], check=True, stdout=subprocess.DEVNULL,
                   stderr=subprocess.DEVNULL)
    subprocess.run(["make", "-C", HOST, "-B", "liblg_host.so", "liblg_modelhip.so", "run-hip"], check=True,
                   stdout=subprocess.DEVNULL)


def _opt(arr):
    return arr.ctypes.data_as(C.c_void_p) if arr is not None else None


def load_hip():
    global _hip
    if _hip is not None:
        return _hip
    path = os.path.join(CSRC, "liblg_hip.so")
    if not os.path.exists(path):
        raise HipError(f"{path} is not built (run __graft_entry__.build())")
    L = C.CDLL(path)
    L.lg_hip_last_error.restype = C.c_char_p
    L.lg_hip_ring_rows.argtypes = [C.c_int, C.c_int]
    L.lg_hip_repacked_bytes.argtypes = [C.c_int, C.c_int]
    L.lg_hip_repacked_bytes.restype = C.c_size_t
    L.lg_hip_repack_q4_0.argtypes = [u8p, C.c_int, C.c_int, u8p]
    L.lg_hip_matmul_q4q8.argtypes = [u8p, C.c_int, C.c_int, f32p, C.c_int] + [C.c_void_p] * 5 + [C.c_int, C.c_void_p]
    L.lg_hip_attention.argtypes = [f32p, u16p, u16p] + [C.c_int] * 7 + [f32p, C.c_int, C.c_void_p]
    L.lg_hip_matmul_f32w.argtypes = [f32p, C.c_int, C.c_int, f32p, C.c_int, f32p]
    L.lg_hip_rows_norm_q8.argtypes = [f32p] + [C.c_void_p] * 4 + [C.c_int, C.c_int, C.c_float] + [C.c_void_p] * 5
    L.lg_hip_rows_ple_gate.argtypes = [f32p, f32p, f32p, u8p, f32p, C.c_int, C.c_int, C.c_int, C.c_float] + [C.c_void_p] * 4
    i32p_ = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
    L.lg_hip_ple_inputs.argtypes = [f32p, f32p, u8p, C.c_int, i32p_, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, f32p]
    L.lg_hip_kv_layout.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.lg_hip_kv_write.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, u16p]
    L.lg_hip_kv_read.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, u16p]
    L.lg_hip_kv_save_prefix.argtypes = [C.c_void_p, C.c_int]
    L.lg_hip_kv_restore_prefix.argtypes = [C.c_void_p, C.c_int]
    L.lg_hip_forward_spec.argtypes = [C.c_void_p, C.c_void_p, i32p, C.c_int, C.c_int, i32p, C.POINTER(C.c_int32)]
    L.lg_hip_prefill.argtypes = [C.c_void_p, C.c_void_p, i32p, C.c_int, C.c_int]
    L.lg_hip_get_hidden.argtypes = [C.c_void_p, f32p]
    L.lg_hip_get_logits.argtypes = [C.c_void_p, C.c_int, f32p]
    L.lg_hip_set_option.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
    L.lg_hip_tail_stamps.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int]
    L.lg_hip_mtp_rounds.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, i32p, i32p, i32p, C.POINTER(C.c_int32)]
    L.lg_hip_schedule_load.argtypes = [C.c_void_p, i32p, C.c_int, C.c_int, C.c_int]
    L.lg_hip_schedule_run.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
    L.lg_hip_schedule_wait.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int32)]
    L.lg_hip_schedule_time.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_float)]
    L.lg_hip_profile_step.argtypes = [C.c_void_p, C.c_void_p, i32p, C.c_int, C.c_int, C.c_int,
                                      C.POINTER(C.c_char_p), f32p, i32p,
                                      np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS"), C.c_int]
    _hip = L
    return L


def hip_check(rc, what):
    if rc < 0:
        raise HipError(f"{what}: {load_hip().lg_hip_last_error().decode()} (code {rc})")
    return rc


def device_count():
    return load_hip().lg_hip_device_count()


def load_backend():
    global _backend
    if _backend is not None:
        return _backend
    load_hip()
    path = os.path.join(HOST, "liblg_modelhip.so")
    if not os.path.exists(path):
        raise HipError(f"{path} is not built (run __graft_entry__.build())")
    B = C.CDLL(path)
    B.lg_session_open.argtypes = [C.c_char_p]
    B.lg_session_open.restype = C.c_void_p
    B.lg_session_close.argtypes = [C.c_void_p]
    B.lg_session_kv.argtypes = [C.c_void_p, C.c_int]
    B.lg_session_model.argtypes = [C.c_void_p]
    B.lg_session_model.restype = C.c_void_p
    B.lg_session_kvcache.argtypes = [C.c_void_p]
    B.lg_session_kvcache.restype = C.c_void_p
    B.lg_session_info.argtypes = [C.c_void_p, i32p, C.c_int]
    B.lg_session_layer.argtypes = [C.c_void_p, C.c_int, i32p]
    B.lg_session_prefill.argtypes = [C.c_void_p, i32p, C.c_int, C.c_int]
    B.lg_session_forward_next.argtypes = [C.c_void_p, C.c_int, C.c_int]
    B.lg_session_forward.argtypes = [C.c_void_p, C.c_int, C.c_int, f32p]
    B.lg_session_forward_spec.argtypes = [C.c_void_p, i32p, C.c_int, C.c_int, i32p]
    B.lg_session_generate.argtypes = [C.c_void_p, i32p, C.c_int, C.c_int, C.c_int, C.c_void_p, i32p, C.POINTER(C.c_int)]
    B.lg_model_device.argtypes = [C.c_void_p]
    B.lg_model_device.restype = C.c_void_p
    B.lg_model_device_kv.argtypes = [C.c_void_p]
    B.lg_model_device_kv.restype = C.c_void_p
    B.lg_model_last_hidden.argtypes = [C.c_void_p, f32p]
    B.lg_model_release.restype = None
    B.lg_session_mtp_open.argtypes = [C.c_void_p, C.c_char_p]
    B.lg_session_mtp_open.restype = C.c_void_p
    B.lg_session_mtp_close.argtypes = [C.c_void_p]
    B.lg_session_mtp_close.restype = None
    B.lg_session_mtp_draft.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]
    B.lg_session_mtp_hidden.argtypes = [C.c_void_p, C.c_void_p, f32p]
    B.lg_session_mtp_logits.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]
    B.lg_session_generate_mtp.argtypes = [C.c_void_p, C.c_void_p, i32p, C.c_int, C.c_int, C.c_int, i32p] + [C.POINTER(C.c_int)] * 3
    B.lg_session_generate_mtp_rounds.argtypes = [C.c_void_p, C.c_void_p, i32p, C.c_int, C.c_int, C.c_int, C.c_int, i32p] + [C.POINTER(C.c_int)] * 3
    B.lg_mtp_device.argtypes = [C.c_void_p, C.c_void_p]
    B.lg_mtp_device.restype = C.c_void_p
    _backend = B
    return B


class HipBackend:
    """One GGUF model on the GPU through the model.h backend (model-hip.c)."""

    def __init__(self, path, max_seq, max_rows=MAX_ROWS):
        if device_count() < 1:
            raise HipError("no HIP device: the verify step has no CPU path")
        os.environ["LG_HIP_MAX_ROWS"] = str(max_rows)
        self.B = load_backend()
        self.H = load_hip()
        self.s = self.B.lg_session_open(os.fsencode(path))
        if not self.s:
            raise HipError(f"cannot open {path}")
        if self.B.lg_session_kv(self.s, max_seq) != 0:
            raise HipError("kvcache_init failed")
        self.max_seq = max_seq
        v = np.zeros(16, np.int32)
        n = self.B.lg_session_info(self.s, v, 16)
        self.info = dict(zip(INFO_KEYS, (int(x) for x in v[:n])))
        self.layers = []
        for i in range(self.info["n_layer"]):
            o = np.zeros(4, np.int32)
            self.B.lg_session_layer(self.s, i, o)
            self.layers.append(dict(is_local=int(o[0]), head_dim=int(o[1]), n_head_kv=int(o[2]), ffn_len=int(o[3])))
        self.model = self.B.lg_session_model(self.s)
        self.dev = self.B.lg_model_device(self.model)
        self.dkv = self.B.lg_model_device_kv(self.B.lg_session_kvcache(self.s))

    def close(self):
        if self.s:
            self.B.lg_session_close(self.s)
            self.B.lg_model_release()
            self.s = None

    def new_cache(self, max_seq=None):
        self.max_seq = max_seq or self.max_seq
        if self.B.lg_session_kv(self.s, self.max_seq) != 0:
            raise HipError("kvcache_init failed")
        self.dkv = self.B.lg_model_device_kv(self.B.lg_session_kvcache(self.s))

    # --- model.h calls
    def prefill(self, tokens, pos0=0):
        t = np.ascontiguousarray(tokens, np.int32)
        self.B.lg_session_prefill(self.s, t, len(t), pos0)

    def forward_next(self, token, pos):
        return self.B.lg_session_forward_next(self.s, int(token), int(pos))

    def forward(self, token, pos, n_vocab):
        logits = np.zeros(n_vocab, np.float32)
        self.B.lg_session_forward(self.s, int(token), int(pos), logits)
        return logits

    def forward_spec(self, toks, pos):
        t = np.ascontiguousarray(toks, np.int32)
        out = np.full(len(t), -1, np.int32)
        adv = self.B.lg_session_forward_spec(self.s, t, len(t), int(pos), out)
        return adv, out

    def generate(self, prompt, n_gen, rows=1, drafts=None):
        p = np.ascontiguousarray(prompt, np.int32)
        emitted = np.zeros(n_gen, np.int32)
        steps = C.c_int(0)
        d = np.ascontiguousarray(drafts, np.int32) if drafts is not None else None
        n = self.B.lg_session_generate(self.s, p, len(p), n_gen, rows, _opt(d), emitted, C.byref(steps))
        return emitted[:n], steps.value

    # --- draft head (mtp_open / mtp_draft / mtp_draft_chain of the reference interface)
    def mtp_open(self, path):
        t = self.B.lg_session_mtp_open(self.s, os.fsencode(path))
        if not t:
            raise HipError(f"cannot open draft head {path} for this model")
        return t

    def mtp_close(self, t):
        self.B.lg_session_mtp_close(t)

    def mtp_draft(self, t, token, pos, chain=False):
        return self.B.lg_session_mtp_draft(self.s, t, int(token), int(pos), int(chain))

    def mtp_hidden(self, t, n_inner):
        h = np.zeros(n_inner, np.float32)
        hip_check(self.B.lg_session_mtp_hidden(self.s, t, h), "draft hidden")
        return h

    def mtp_store_logits(self, t, on=True):
        hip_check(self.B.lg_session_mtp_logits(self.s, t, int(on), None), "draft store_logits")

    def mtp_logits(self, t, n_vocab):
        out = np.zeros(n_vocab, np.float32)
        hip_check(self.B.lg_session_mtp_logits(self.s, t, 1, out.ctypes.data), "draft logits")
        return out

    def generate_mtp(self, t, prompt, n_gen, rows):
        p = np.ascontiguousarray(prompt, np.int32)
        emitted = np.zeros(n_gen, np.int32)
        steps, nd, na = C.c_int(0), C.c_int(0), C.c_int(0)
        n = self.B.lg_session_generate_mtp(self.s, t, p, len(p), n_gen, rows, emitted, C.byref(steps), C.byref(nd), C.byref(na))
        if n < 0:
            raise HipError("generate_mtp rejected its arguments")
        return emitted[:n], steps.value, nd.value, na.value

    def generate_mtp_rounds(self, t, prompt, n_gen, rows, batch):
        """generate_mtp with `batch` speculative rounds at a time kept on the device."""
        p = np.ascontiguousarray(prompt, np.int32)
        emitted = np.zeros(n_gen, np.int32)
        steps, nd, na = C.c_int(0), C.c_int(0), C.c_int(0)
        n = self.B.lg_session_generate_mtp_rounds(self.s, t, p, len(p), n_gen, rows, batch, emitted, C.byref(steps), C.byref(nd), C.byref(na))
        if n < 0:
            raise HipError("generate_mtp_rounds rejected its arguments")
        return emitted[:n], steps.value, nd.value, na.value

    def mtp_rounds(self, t, token, pos, rows, n_rounds):
        """n_rounds device-resident speculative rounds through the C ABI: (blocks, out, adv, final_pos)."""
        d = self.B.lg_mtp_device(t, self.model)
        if not d:
            raise HipError("the draft head is not on the device")
        blocks = np.zeros((n_rounds, rows), np.int32)
        out = np.zeros((n_rounds, rows), np.int32)
        adv = np.zeros(n_rounds, np.int32)
        fp = C.c_int32(0)
        hip_check(self.H.lg_hip_mtp_rounds(d, self.dkv, int(token), int(pos), rows, n_rounds, blocks, out, adv, C.byref(fp)), "mtp_rounds")
        return blocks, out, adv, fp.value

    def last_hidden(self, n_embd):
        h = np.zeros(n_embd, np.float32)
        hip_check(self.B.lg_model_last_hidden(self.model, h), "get_hidden")
        return h

    # --- C ABI calls on the same device objects
    def set_option(self, name, value):
        hip_check(self.H.lg_hip_set_option(self.dev, name.encode(), int(value)), "set_option")

    def tail_stamps(self, which=0):
        """[64 units][8] wall-clock stamps (100 MHz ticks) of the latest one-XCD launch (option xcd_tail_stamps):
        which = 0 the layer's tail, 1 the attention half's."""
        out = np.zeros((64, 8), np.uint64)
        hip_check(self.H.lg_hip_tail_stamps(self.dev, which,
                                            out.ctypes.data_as(C.c_void_p), out.size), "tail_stamps")
        return out

    def logits_row(self, row, n_vocab):
        out = np.zeros(n_vocab, np.float32)
        hip_check(self.H.lg_hip_get_logits(self.dev, row, out), "get_logits")
        return out

    def kv_layout(self, layer):
        r, w = C.c_int(), C.c_int()
        hip_check(self.H.lg_hip_kv_layout(self.dkv, layer, C.byref(r), C.byref(w)), "kv_layout")
        return r.value, w.value

    def kv_read(self, layer, which):
        rows, width = self.kv_layout(layer)
        out = np.zeros((rows, width), np.uint16)
        hip_check(self.H.lg_hip_kv_read(self.dkv, layer, which, 0, rows, out), "kv_read")
        return out

    def kv_write(self, layer, which, data, row0=0):
        d = np.ascontiguousarray(data, np.uint16)
        hip_check(self.H.lg_hip_kv_write(self.dkv, layer, which, row0, d.shape[0], d), "kv_write")

    def schedule(self, blocks, pos0):
        b = np.ascontiguousarray(blocks, np.int32)
        hip_check(self.H.lg_hip_schedule_load(self.dev, b, b.shape[0], b.shape[1], pos0), "schedule_load")
        self._sched_shape = b.shape

    def schedule_time(self, n_steps):
        ms = C.c_float(0)
        hip_check(self.H.lg_hip_schedule_time(self.dev, self.dkv, n_steps, C.byref(ms)), "schedule_time")
        return ms.value

    def schedule_run(self, n_steps):
        hip_check(self.H.lg_hip_schedule_run(self.dev, self.dkv, n_steps), "schedule_run")

    def schedule_wait(self):
        steps, rows = self._sched_shape
        out = np.zeros((steps, rows), np.int32)
        adv = np.zeros(steps, np.int32)
        pos = C.c_int32(0)
        done = hip_check(self.H.lg_hip_schedule_wait(self.dev, _opt(out), _opt(adv), C.byref(pos)), "schedule_wait")
        return out[:done], adv[:done], pos.value

    def profile_step(self, toks, pos, repeats=3):
        t = np.ascontiguousarray(toks, np.int32)
        cap = 32
        names = (C.c_char_p * cap)()
        ms = np.zeros(cap, np.float32)
        launches = np.zeros(cap, np.int32)
        nbytes = np.zeros(cap, np.float64)
        n = hip_check(self.H.lg_hip_profile_step(self.dev, self.dkv, t, len(t), pos, repeats, names, ms, launches,
                                                 nbytes, cap), "profile_step")
        return [dict(name=names[i].decode(), ms=float(ms[i]), launches=int(launches[i]), bytes=float(nbytes[i]))
                for i in range(n)]


def matmul_q4q8(w_q4_0, k, m, x, want_dots=False, repeats=0):
    """Isolated q4_0 x q8 matmul through the C ABI.  Returns dict(out, dots, xq, xd, xsum, ms)."""
    H = load_hip()
    w = np.ascontiguousarray(w_q4_0, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    rows = x.shape[0]
    nb = k // 32
    out = np.zeros((rows, m), np.float32)
    dots = np.zeros((rows, m, nb), np.int32) if want_dots else None
    xq = np.zeros((rows, k), np.int8)
    xd = np.zeros((rows, nb), np.float32)
    xsum = np.zeros((rows, nb), np.int32)
    ms = C.c_float(0)
    hip_check(H.lg_hip_matmul_q4q8(w, k, m, x, rows, _opt(out), _opt(dots), _opt(xq), _opt(xd), _opt(xsum),
                                   repeats, C.cast(C.byref(ms), C.c_void_p)), "matmul_q4q8")
    return dict(out=out, dots=dots, xq=xq, xd=xd, xsum=xsum, ms=ms.value)


def rows_norm_q8(x, dout=None, w_post=None, out_scale=None, w_pre=None, eps=1e-6):
    """Isolated row kernel through the C ABI.  x, dout: [rows, E] f32; returns dict(x_out, h, xq, xd, xsum)."""
    H = load_hip()
    x = np.ascontiguousarray(x, np.float32)
    rows, E = x.shape
    keep = [np.ascontiguousarray(a, np.float32) if a is not None else None
            for a in (dout, w_post, None if out_scale is None else np.array([out_scale], np.float32), w_pre)]
    x_out = np.zeros_like(x); h = np.zeros_like(x)
    xq = np.zeros((rows, E), np.int8); xd = np.zeros((rows, E // 32), np.float32); xsum = np.zeros((rows, E // 32), np.int32)
    hip_check(H.lg_hip_rows_norm_q8(x, *[_opt(a) for a in keep], rows, E, eps, _opt(x_out), _opt(h), _opt(xq), _opt(xd), _opt(xsum)),
              "rows_norm_q8")
    return dict(x_out=x_out, h=h, xq=xq, xd=xd, xsum=xsum)


def rows_ple_gate(x, dout, w_post, w_gate_q4_0, ipl, eps=1e-6):
    """Isolated rows + per-layer gate kernel through the C ABI.  x, dout: [rows, E]; w_gate_q4_0: ple q4_0 rows of E;
    ipl: [rows, ple].  Returns dict(x_out, pq, pd, psum)."""
    H = load_hip()
    x = np.ascontiguousarray(x, np.float32)
    rows, E = x.shape
    ipl = np.ascontiguousarray(ipl, np.float32)
    ple = ipl.shape[1]
    x_out = np.zeros_like(x)
    pq = np.zeros((rows, ple), np.int8); pd = np.zeros((rows, ple // 32), np.float32); psum = np.zeros((rows, ple // 32), np.int32)
    hip_check(H.lg_hip_rows_ple_gate(x, np.ascontiguousarray(dout, np.float32), np.ascontiguousarray(w_post, np.float32),
                                     np.ascontiguousarray(w_gate_q4_0, np.uint8), ipl, rows, E, ple, eps,
                                     _opt(x_out), _opt(pq), _opt(pd), _opt(psum)), "rows_ple_gate")
    return dict(x_out=x_out, pq=pq, pd=pd, psum=psum)


def down_m(act, down_q4_0, E, repeats=0, join=1):
    """lg_k_down_m in isolation: act [rows][FF] f32, down_q4_0 raw q4_0 rows [E][FF]; returns out [rows][E], kernel ms."""
    H = load_hip()
    rows, FF = act.shape
    H.lg_hip_down_m.argtypes = [f32p, u8p, C.c_int, C.c_int, C.c_int, C.c_int, f32p, C.c_int, C.POINTER(C.c_float)]
    out = np.zeros((rows, E), np.float32)
    ms = C.c_float(0)
    hip_check(H.lg_hip_down_m(np.ascontiguousarray(act, np.float32), down_q4_0, rows, E, FF, int(join), out, repeats, C.byref(ms)), "down_m")
    return out, ms.value


def gate_up_geglu(x, gate_q4_0, up_q4_0, FF, repeats=0):
    """lg_k_geglu_t / lg_k_geglu_m in isolation: x [rows][E] f32, gate / up raw q4_0 rows [FF][E]; returns dict(aq, ad, asum, ms):
    the q8 of gelu(gate) * up in natural order."""
    H = load_hip()
    x = np.ascontiguousarray(x, np.float32)
    rows, E = x.shape
    H.lg_hip_gate_up_geglu.argtypes = [f32p, u8p, u8p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_float)]
    aq = np.zeros((rows, FF), np.int8); ad = np.zeros((rows, FF // 32), np.float32); asum = np.zeros((rows, FF // 32), np.int32)
    ms = C.c_float(0)
    hip_check(H.lg_hip_gate_up_geglu(x, np.ascontiguousarray(gate_q4_0, np.uint8), np.ascontiguousarray(up_q4_0, np.uint8), rows, E, FF,
                                     aq.ctypes.data, ad.ctypes.data, asum.ctypes.data, repeats, C.byref(ms)), "gate_up_geglu")
    return dict(aq=aq, ad=ad, asum=asum, ms=ms.value)


def ffn_xcd(x, dout, w_post, w_pre, gate_q4_0, up_q4_0, down_q4_0, FF, eps=1e-6, repeats=0, flush_mb=0, want_stamps=False, delay_w=0):
    """The XCD-partitioned feed-forward half of a layer through the C ABI.  x, dout: [rows, E] (rows 4..8); gate / up:
    FF q4_0 rows of E, down: E q4_0 rows of FF.  Returns dict(x_out, act [rows, FF], out [rows, E], kernel_ms)."""
    H = load_hip()
    H.lg_hip_ffn_xcd.argtypes = [f32p, f32p, f32p, f32p, u8p, u8p, u8p, C.c_int, C.c_int, C.c_int, C.c_float,
                                 f32p, f32p, f32p, C.c_int, C.POINTER(C.c_float), C.c_int, C.c_int, C.c_void_p]
    x = np.ascontiguousarray(x, np.float32)
    rows, E = x.shape
    x_out = np.zeros_like(x); act = np.zeros((rows, FF), np.float32); out = np.zeros_like(x)
    ms = C.c_float(0)
    stamps = np.zeros((256, 2, 16), np.int64) if want_stamps else None
    hip_check(H.lg_hip_ffn_xcd(x, np.ascontiguousarray(dout, np.float32), np.ascontiguousarray(w_post, np.float32),
                               np.ascontiguousarray(w_pre, np.float32), np.ascontiguousarray(gate_q4_0, np.uint8),
                               np.ascontiguousarray(up_q4_0, np.uint8), np.ascontiguousarray(down_q4_0, np.uint8),
                               rows, E, FF, eps, x_out, act, out, repeats, C.byref(ms), flush_mb, delay_w, _opt(stamps)), "ffn_xcd")
    return dict(x_out=x_out, act=act, out=out, kernel_ms=ms.value, stamps=stamps)


def ple_inputs(pmp, proj_norm, pte_q4_0, n_tok, toks, n_layer, ple, E, eps=1e-6):
    """Isolated per-layer-input kernel through the C ABI.  pmp: [rows, n_layer*ple] raw projection; pte_q4_0: n_tok
    q4_0 rows of n_layer*ple; toks: [rows].  Returns [rows, n_layer*ple]."""
    H = load_hip()
    pmp = np.ascontiguousarray(pmp, np.float32)
    out = np.zeros_like(pmp)
    hip_check(H.lg_hip_ple_inputs(pmp, np.ascontiguousarray(proj_norm, np.float32), np.ascontiguousarray(pte_q4_0, np.uint8),
                                  n_tok, np.ascontiguousarray(toks, np.int32), pmp.shape[0], n_layer, ple, E, eps, out),
              "ple_inputs")
    return out


def matmul_f32w(w, x):
    """Isolated f32-weight matmul through the C ABI.  w: [m, k] f32, x: [rows, k] f32 -> [rows, m]."""
    H = load_hip()
    w = np.ascontiguousarray(w, np.float32)
    x = np.ascontiguousarray(x, np.float32)
    out = np.zeros((x.shape[0], w.shape[0]), np.float32)
    hip_check(H.lg_hip_matmul_f32w(w, w.shape[1], w.shape[0], x, x.shape[0], out), "matmul_f32w")
    return out


def attention(q, kc, vc, n_head, n_head_kv, hd, window, pos, repeats=0):
    """Isolated decode attention through the C ABI.  q: [rows, n_head*hd]; kc, vc: [seq, n_head_kv*hd] uint16."""
    H = load_hip()
    q = np.ascontiguousarray(q, np.float32)
    kc = np.ascontiguousarray(kc, np.uint16)
    vc = np.ascontiguousarray(vc, np.uint16)
    rows = q.shape[0]
    out = np.zeros_like(q)
    ms = C.c_float(0)
    hip_check(H.lg_hip_attention(q, kc, vc, rows, n_head, n_head_kv, hd, kc.shape[0], window, pos, out, repeats,
                                 C.cast(C.byref(ms), C.c_void_p)), "attention")
    return out, ms.value
