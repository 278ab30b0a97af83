"""Seeded synthetic Gemma-4-style GGUF models (host/synth.c) and the shapes the tests and
the benchmark use.  The shapes are the ones the baseline configuration list names."""
import ctypes as C
import os

from . import hostlib


class SynthSpec(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "n_layer", "n_embd", "n_head", "n_head_kv", "head_dim", "head_dim_full", "n_ff", "n_vocab",
        "n_ctx", "sliding_window", "local_period", "ple", "shared_kv_layers", "has_v", "has_rope_freqs", "ple_float")] + [
        (n, C.c_float) for n in ("w_std", "qk_norm", "norm_jitter", "out_scale", "rms_eps", "rope_base",
                                 "rope_base_swa", "softcap")] + [("seed", C.c_uint64)]


DEFAULTS = dict(head_dim_full=0, n_ctx=8192, sliding_window=512, local_period=6, ple=0, shared_kv_layers=0,
                has_v=1, has_rope_freqs=1, ple_float=0, w_std=0.02, qk_norm=0.0, norm_jitter=0.1, out_scale=0.0,
                rms_eps=1e-6, rope_base=1e6, rope_base_swa=1e4, softcap=30.0, seed=1234)

# 4 layers, d 512, 8 x 64 heads, 2 KV heads, FFN 2048, vocab 8192, sliding-128 / global alternating
TINY = dict(DEFAULTS, n_layer=4, n_embd=512, n_head=8, n_head_kv=2, head_dim=64, n_ff=2048, n_vocab=8192,
            sliding_window=128, local_period=2, qk_norm=0.7)
# the same with every optional piece switched on: PLE, shared-KV tail, V-less layers, output scale
TINY_FULL = dict(TINY, n_layer=6, ple=256, shared_kv_layers=2, has_v=0, out_scale=0.9, head_dim_full=128)
# ... and with the per-layer-embedding matrices kept in a float type, as QAT conversions of E4B store them
TINY_FULL_F32 = dict(TINY_FULL, ple_float=1)
TINY_FULL_F16 = dict(TINY_FULL, ple_float=2)
TINY_FULL_BF16 = dict(TINY_FULL, ple_float=3)
# E4B shape: 42 layers, d 2560, 8/2 heads x 256, FFN 10240, PLE 256, vocab 262144; 5 sliding(512) : 1 global
E4B = dict(DEFAULTS, n_layer=42, n_embd=2560, n_head=8, n_head_kv=2, head_dim=256, n_ff=10240, n_vocab=262144,
           ple=256, sliding_window=512, local_period=6, out_scale=1.0)
# 12B shape: 48 layers, d 3840, 16/8 heads x 256, FFN 15360, vocab 262144; 5 sliding(1024) : 1 global, no PLE
G12B = dict(DEFAULTS, n_layer=48, n_embd=3840, n_head=16, n_head_kv=8, head_dim=256, n_ff=15360, n_vocab=262144,
            sliding_window=1024, local_period=6)


def write_model(path, **spec):
    """Write a model file; returns the spec actually used."""
    full = dict(DEFAULTS)
    full.update(spec)
    s = SynthSpec(**full)
    rc = hostlib.lib().lg_synth_write(os.fsencode(path), C.byref(s))
    if rc != 0:
        raise RuntimeError(f"lg_synth_write({path}) failed with {rc}")
    return full


class AssistantSpec(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "n_layer", "n_inner", "n_backbone", "n_head", "n_ff", "n_vocab", "head_dim_swa", "head_dim_full", "n_full",
        "has_post")] + [(n, C.c_float) for n in ("w_std", "qk_norm", "norm_jitter", "out_scale", "rms_eps", "rope_base",
                                                 "rope_base_swa", "softcap")] + [("seed", C.c_uint64)]


ASSISTANT_DEFAULTS = dict(n_layer=4, n_inner=256, n_head=4, n_full=1, has_post=1, w_std=0.02, qk_norm=0.0,
                          norm_jitter=0.1, out_scale=0.0, rms_eps=1e-6, rope_base=1e6, rope_base_swa=1e4,
                          softcap=30.0, seed=4321)


def assistant_for(target, **over):
    """Spec of a draft head ("gemma4-assistant") that fits the target spec: 4 blocks, 256 wide, the last one
    reading the global cache (when the target's head sizes differ; otherwise all read the sliding one)."""
    hd_l = target["head_dim"]
    hd_g = target.get("head_dim_full") or hd_l
    # the head's query heads share the target's KV heads: a multiple of their number
    nkv = target["n_head_kv"]
    heads = -(-ASSISTANT_DEFAULTS["n_head"] // nkv) * nkv
    spec = dict(ASSISTANT_DEFAULTS, n_head=heads, n_backbone=target["n_embd"], n_vocab=target["n_vocab"], head_dim_swa=hd_l,
                head_dim_full=hd_g, n_ff=1024, qk_norm=target.get("qk_norm", 0.0),
                rope_base=target.get("rope_base", 1e6), rope_base_swa=target.get("rope_base_swa", 1e4))
    spec.update(over)
    return spec


def write_assistant(path, **spec):
    s = AssistantSpec(**spec)
    lib = hostlib.lib()
    lib.lg_synth_write_assistant.restype = C.c_int
    rc = lib.lg_synth_write_assistant(os.fsencode(path), C.byref(s))
    if rc != 0:
        raise RuntimeError(f"lg_synth_write_assistant({path}) failed with {rc}")
    return spec
