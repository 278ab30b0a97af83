"""ctypes bindings of the CPU oracle (liblg_oracle.so) and, where it was built, of the reference's
own CPU backend (oracle/_ref/libref_n<N>.so).

TEST INFRASTRUCTURE ONLY: import this from tests/, from __graft_entry__.smoke() and from the
cpu_baseline leg of bench.py, nowhere else.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF, I8, I8_LIBM, I8_F32 = 0, 1, 2, 3
ORDER_SEG, ORDER_CUDA32 = 0, 1
_lib = None
_ref = {}

c_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
c_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
c_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
c_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
c_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")


def build(with_ref=True):
    """Compile the oracle; also the reference CPU backend when its sources are present."""
    subprocess.run(["make", "-C", HERE, "-B", "liblg_oracle.so"], check=True, stdout=subprocess.DEVNULL)
    if with_ref and os.path.isdir("/root/reference/src"):
        subprocess.run(["make", "-C", HERE, "-B", "ref"], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    path = os.path.join(HERE, "liblg_oracle.so")
    if not os.path.exists(path):
        build(with_ref=False)
    L = C.CDLL(path)
    L.lgo_quant_q8.argtypes = [c_f32p, C.c_int, c_i8p, c_f32p, c_i32p]
    L.lgo_block_dot.argtypes = [c_u8p, c_i8p]
    L.lgo_block_dot.restype = C.c_int32
    L.lgo_matmul_q4q8.argtypes = [c_u8p, C.c_int, C.c_int, c_i8p, c_f32p, C.c_int, c_f32p, C.c_void_p, C.c_int]
    L.lgo_matmul_f32.argtypes = [c_u8p, C.c_uint32, C.c_int, C.c_int, c_f32p, c_f32p]
    L.lgo_matmul_fw.argtypes = [c_u8p, C.c_uint32, C.c_int, C.c_int, c_f32p, c_f32p]
    L.lgo_rmsnorm.argtypes = [c_f32p, c_f32p, C.c_void_p, C.c_int, C.c_float, C.c_int]
    L.lgo_rope.argtypes = [c_f32p, C.c_int, C.c_int, c_f32p, C.c_void_p, C.c_int]
    L.lgo_attention_f16.argtypes = [c_f32p, c_f32p, c_u16p, c_u16p] + [C.c_int] * 8
    L.lgo_accept.argtypes = [c_i32p, c_i32p, C.c_int]
    for f in ("lgo_expf", "lgo_tanhf"):
        getattr(L, f).argtypes = [C.c_float]
        getattr(L, f).restype = C.c_float
    L.lgo_gelu.argtypes = [C.c_float, C.c_int]
    L.lgo_gelu.restype = C.c_float
    L.lgo_sincosf.argtypes = [C.c_float, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.lgo_f32_to_f16.argtypes = [C.c_float]
    L.lgo_f32_to_f16.restype = C.c_uint16
    L.lgo_f16_to_f32.argtypes = [C.c_uint16]
    L.lgo_f16_to_f32.restype = C.c_float
    L.lgo_ring_rows.argtypes = [C.c_int, C.c_int]
    L.lgo_model_open.argtypes = [C.c_char_p]
    L.lgo_model_open.restype = C.c_void_p
    L.lgo_model_close.argtypes = [C.c_void_p]
    L.lgo_model_info.argtypes = [C.c_void_p, c_i32p, C.c_int]
    L.lgo_layer_info.argtypes = [C.c_void_p, C.c_int, c_i32p]
    L.lgo_kv_new.argtypes = [C.c_void_p, C.c_int, C.c_int]
    L.lgo_kv_new.restype = C.c_void_p
    L.lgo_kv_free.argtypes = [C.c_void_p]
    L.lgo_kv_layer.argtypes = [C.c_void_p, C.c_int, C.c_int] + [C.POINTER(C.c_int)] * 3
    L.lgo_kv_layer.restype = C.c_void_p
    L.lgo_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    L.lgo_prefill.argtypes = [C.c_void_p, C.c_void_p, c_i32p, C.c_int, C.c_int, C.c_int]
    L.lgo_forward_spec.argtypes = [C.c_void_p, C.c_void_p, c_i32p, C.c_int, C.c_int, C.c_int, c_i32p, C.c_void_p]
    L.lgo_set_threads.argtypes = [C.c_int]
    L.lgo_forward_spec_all.argtypes = [C.c_void_p, C.c_void_p, c_i32p, C.c_int, C.c_int, C.c_int, c_i32p, C.c_void_p]
    L.lgo_mtp_open.argtypes = [C.c_char_p, C.c_void_p]
    L.lgo_mtp_open.restype = C.c_void_p
    L.lgo_mtp_close.argtypes = [C.c_void_p]
    L.lgo_mtp_info.argtypes = [C.c_void_p, c_i32p, C.c_int]
    L.lgo_mtp_draft.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, c_f32p, C.c_int, C.c_void_p, C.c_void_p]
    L.lgo_mtp_post.argtypes = [C.c_void_p, c_f32p, C.c_int, c_f32p]
    _lib = L
    return L


INFO_KEYS = ("n_layer", "n_embd", "n_head", "n_vocab", "ple", "n_kv_start", "window", "n_ff", "n_head_kv",
             "head_dim_swa", "head_dim_full", "n_ctx")


def _kv_views(get_layer, handle, n_layer):
    """numpy views of every owning layer's K and V storage: {L: (K, V)} with shape [rows, width]."""
    out = {}
    for L in range(n_layer):
        rows, width, f16 = C.c_int(), C.c_int(), C.c_int()
        pair = []
        for which in (0, 1):
            p = get_layer(handle, L, which, C.byref(rows), C.byref(width), C.byref(f16))
            if not p:
                pair = None
                break
            dt = np.uint16 if f16.value else np.float32
            n = rows.value * width.value
            buf = (C.c_uint16 * n if f16.value else C.c_float * n).from_address(p)
            pair.append(np.frombuffer(buf, dtype=dt).reshape(rows.value, width.value))
        if pair:
            out[L] = tuple(pair)
    return out


class Oracle:
    """One GGUF model under the CPU oracle."""

    def __init__(self, path):
        self.L = lib()
        self.h = self.L.lgo_model_open(os.fsencode(path))
        if not self.h:
            raise RuntimeError(f"oracle: cannot open {path}")
        v = np.zeros(16, np.int32)
        n = self.L.lgo_model_info(self.h, v, 16)
        self.info = dict(zip(INFO_KEYS, (int(x) for x in v[:n])))
        self.layers = []
        for i in range(self.info["n_layer"]):
            o = np.zeros(4, np.int32)
            self.L.lgo_layer_info(self.h, i, o)
            self.layers.append(dict(is_local=int(o[0]), head_dim=int(o[1]), n_head_kv=int(o[2]), ffn_len=int(o[3])))

    def close(self):
        if self.h:
            self.L.lgo_model_close(self.h)
            self.h = None

    def kv_new(self, max_seq, mode):
        kv = self.L.lgo_kv_new(self.h, max_seq, mode)
        if not kv:
            raise MemoryError("oracle kv")
        return kv

    def kv_free(self, kv):
        self.L.lgo_kv_free(kv)

    def kv_views(self, kv):
        return _kv_views(self.L.lgo_kv_layer, kv, self.info["n_layer"])

    def forward(self, kv, token, pos, mode, want_logits=True, want_hidden=False):
        logits = np.zeros(self.info["n_vocab"], np.float32) if want_logits else None
        hidden = np.zeros(self.info["n_embd"], np.float32) if want_hidden else None
        best = self.L.lgo_forward(self.h, kv, token, pos, mode,
                                  logits.ctypes.data if want_logits else None,
                                  hidden.ctypes.data if want_hidden else None)
        if best < 0:
            raise ValueError("oracle forward rejected its arguments")
        return best, logits, hidden

    def prefill(self, kv, tokens, pos0, mode):
        t = np.ascontiguousarray(tokens, np.int32)
        self.L.lgo_prefill(self.h, kv, t, len(t), pos0, mode)

    def forward_spec(self, kv, toks, pos, mode, want_hidden=False):
        t = np.ascontiguousarray(toks, np.int32)
        out = np.full(len(t), -1, np.int32)
        hidden = np.zeros(self.info["n_embd"], np.float32) if want_hidden else None
        adv = self.L.lgo_forward_spec(self.h, kv, t, len(t), pos, mode, out,
                                      hidden.ctypes.data if want_hidden else None)
        return adv, out, hidden

    def forward_spec_all(self, kv, toks, pos, mode, want_hidden=False):
        """The verify step as the device runs it: every row forwarded (rejected rows reach the cache too)."""
        t = np.ascontiguousarray(toks, np.int32)
        out = np.full(len(t), -1, np.int32)
        hidden = np.zeros(self.info["n_embd"], np.float32) if want_hidden else None
        adv = self.L.lgo_forward_spec_all(self.h, kv, t, len(t), pos, mode, out,
                                          hidden.ctypes.data if want_hidden else None)
        return adv, out, hidden

    def mtp_open(self, path):
        return OracleDraft(self, path)


MTP_KEYS = ("n_layer", "n_inner", "n_bb", "n_vocab", "n_head", "n_ff", "has_post")


class OracleDraft:
    """A draft-head file under the CPU oracle, attached to its target."""

    def __init__(self, target, path):
        self.L, self.target = target.L, target
        self.h = self.L.lgo_mtp_open(os.fsencode(path), target.h)
        if not self.h:
            raise RuntimeError(f"oracle: cannot open draft head {path} for this target")
        v = np.zeros(8, np.int32)
        n = self.L.lgo_mtp_info(self.h, v, 8)
        self.info = dict(zip(MTP_KEYS, (int(x) for x in v[:n])))

    def close(self):
        if self.h:
            self.L.lgo_mtp_close(self.h)
            self.h = None

    def draft(self, kv, token, pos, h_prev, mode, want_logits=False):
        hidden = np.zeros(self.info["n_inner"], np.float32)
        logits = np.zeros(self.info["n_vocab"], np.float32) if want_logits else None
        tok = self.L.lgo_mtp_draft(self.h, self.target.h, kv, token, pos, np.ascontiguousarray(h_prev, np.float32), mode,
                                   hidden.ctypes.data, logits.ctypes.data if want_logits else None)
        if tok < 0:
            raise ValueError("oracle draft rejected its arguments")
        return tok, hidden, logits

    def post(self, hidden, mode):
        out = np.zeros(self.info["n_bb"], np.float32)
        if self.L.lgo_mtp_post(self.h, np.ascontiguousarray(hidden, np.float32), mode, out) != 0:
            return None
        return out


def ref_available(n=4):
    return os.path.exists(os.path.join(HERE, "_ref", f"libref_n{n}.so"))


class RefConfig(C.Structure):
    _fields_ = [("arch", C.c_char * 32)] + [(k, C.c_int) for k in (
        "n_layer", "n_embd", "n_head", "n_head_kv", "head_dim_swa", "head_dim_full", "n_ff", "n_vocab",
        "n_ctx", "sliding_window", "n_embd_per_layer", "n_kv_start")] + [(k, C.c_float) for k in (
        "rms_eps", "rope_freq_base", "rope_freq_base_swa", "logit_softcap")]


def ref_lib(n=4):
    if n not in _ref:
        R = C.CDLL(os.path.join(HERE, "_ref", f"libref_n{n}.so"))
        R.ref_open.argtypes = [C.c_char_p]
        R.ref_open.restype = C.c_void_p
        R.ref_close.argtypes = [C.c_void_p]
        R.ref_config.argtypes = [C.c_void_p, C.POINTER(RefConfig)]
        R.ref_layer_info.argtypes = [C.c_void_p, C.c_int, c_i32p]
        R.ref_kv_new.argtypes = [C.c_void_p, C.c_int]
        R.ref_kv_new.restype = C.c_void_p
        R.ref_kv_free.argtypes = [C.c_void_p]
        R.ref_kv_layer.argtypes = [C.c_void_p, C.c_int, C.c_int] + [C.POINTER(C.c_int)] * 3
        R.ref_kv_layer.restype = C.c_void_p
        R.ref_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, c_f32p]
        R.ref_forward_next.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        R.ref_prefill.argtypes = [C.c_void_p, C.c_void_p, c_i32p, C.c_int, C.c_int]
        R.ref_forward_spec.argtypes = [C.c_void_p, C.c_void_p, c_i32p, C.c_int, c_i32p]
        R.ref_last_hidden.argtypes = [C.c_void_p, c_f32p]
        R.ref_dequantize.argtypes = [C.c_uint, c_u8p, c_f32p, C.c_longlong]
        for f in ("ref_n_vocab", "ref_n_embd", "ref_n_layer"):
            getattr(R, f).argtypes = [C.c_void_p]
        R.ref_mtp_open.argtypes = [C.c_void_p, C.c_char_p]
        R.ref_mtp_open.restype = C.c_void_p
        R.ref_mtp_free.argtypes = [C.c_void_p]
        R.ref_mtp_draft.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        R.ref_mtp_n_vocab.argtypes = [C.c_void_p]
        R.ref_mtp_n_inner.argtypes = [C.c_void_p]
        R.ref_mtp_logits.argtypes = [C.c_void_p, c_f32p]
        R.ref_mtp_hidden.argtypes = [C.c_void_p, c_f32p]
        _ref[n] = R
    return _ref[n]


class Reference:
    """One GGUF model under the reference's own CPU backend (compiled from its sources)."""

    def __init__(self, path, n=4):
        self.R = ref_lib(n)
        self.n = n
        self.h = self.R.ref_open(os.fsencode(path))
        if not self.h:
            raise RuntimeError(f"reference: cannot open {path}")
        self.n_vocab = self.R.ref_n_vocab(self.h)
        self.n_embd = self.R.ref_n_embd(self.h)
        self.n_layer = self.R.ref_n_layer(self.h)

    def close(self):
        if self.h:
            self.R.ref_close(self.h)
            self.h = None

    def config(self):
        c = RefConfig()
        self.R.ref_config(self.h, C.byref(c))
        return {k: getattr(c, k) for k, _ in RefConfig._fields_}

    def kv_new(self, max_seq):
        return self.R.ref_kv_new(self.h, max_seq)

    def kv_free(self, kv):
        self.R.ref_kv_free(kv)

    def kv_views(self, kv):
        return _kv_views(self.R.ref_kv_layer, kv, self.n_layer)

    def forward(self, kv, token, pos):
        logits = np.zeros(self.n_vocab, np.float32)
        self.R.ref_forward(self.h, kv, token, pos, logits)
        return logits

    def forward_next(self, kv, token, pos):
        return self.R.ref_forward_next(self.h, kv, token, pos)

    def prefill(self, kv, tokens, pos0):
        t = np.ascontiguousarray(tokens, np.int32)
        self.R.ref_prefill(self.h, kv, t, len(t), pos0)

    def forward_spec(self, kv, toks, pos):
        t = np.ascontiguousarray(toks, np.int32)
        assert len(t) == self.n
        out = np.full(self.n, -1, np.int32)
        adv = self.R.ref_forward_spec(self.h, kv, t, pos, out)
        return adv, out

    def last_hidden(self):
        h = np.zeros(self.n_embd, np.float32)
        self.R.ref_last_hidden(self.h, h)
        return h

    # the reference's host draft head (src/mtp.c), h_prev = this model's last_hidden
    def mtp_open(self, path):
        t = self.R.ref_mtp_open(self.h, os.fsencode(path))
        if not t:
            raise RuntimeError(f"reference: cannot open draft head {path}")
        return t

    def mtp_free(self, t):
        self.R.ref_mtp_free(t)

    def mtp_draft(self, t, kv, token, pos):
        tok = self.R.ref_mtp_draft(self.h, t, kv, token, pos)
        logits = np.zeros(self.R.ref_mtp_n_vocab(t), np.float32)
        hidden = np.zeros(self.R.ref_mtp_n_inner(t), np.float32)
        self.R.ref_mtp_logits(t, logits)
        self.R.ref_mtp_hidden(t, hidden)
        return tok, hidden, logits
