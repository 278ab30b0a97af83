#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ by running the REFERENCE's own CPU backend
(compiled from /root/reference by `make -C oracle ref`, never copied) on models this repository
generates.  Run it in the build container only; the GPU box never sees the reference.

Outputs (data only):
  q4_0_dequant.npz      random q4_0 blocks and what the reference's dequantize_into makes of them
  ref_<model>.npz       model spec hash, prompt, per-step greedy tokens of the reference `run` path
                        (model_prefill + model_forward_next), full logits of a few steps,
                        last_hidden of the final step, and a model_forward_spec transcript
  ref_draft_<model>.npz the reference's host draft head (src/mtp.c mtp_draft) on a generated
                        gemma4-assistant file: 16 decode steps, after each one the drafted token,
                        the head's post-norm hidden and, for three steps, its full logits

Usage: make_fixtures.py [all | model | draft]
"""
import hashlib
import importlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
lg = importlib.import_module("little-gemma_amd")
from oracle import binding as ob  # noqa: E402

MODELS = {"tiny": lg.synth.TINY, "tiny_full": lg.synth.TINY_FULL}
# the same with the per-layer-embedding matrices kept f32 (model fixtures only: a draft head never reads them)
FLOAT_PLE_MODELS = {"tiny_full_f32": lg.synth.TINY_FULL_F32}
N_PROMPT, N_GEN, LOGIT_STEPS = 128, 64, (0, 1, 31, 63)


def sha256(path):
    h = hashlib.sha256()
    with open(path, "rb") as f:
        for chunk in iter(lambda: f.read(1 << 20), b""):
            h.update(chunk)
    return h.hexdigest()


def main():
    assert ob.ref_available(4), "build the reference first: make -C oracle ref"
    R = ob.ref_lib(4)
    rng = np.random.default_rng(20250101)
    blocks = rng.integers(0, 256, (64, 18), dtype=np.uint8)
    scales = np.concatenate([rng.normal(0, 0.01, 56), [0.0, -0.0, 6.1e-5, -5.96e-8, 65504.0, 1.0, -2.5, 3e-3]]).astype(np.float16)
    blocks[:, 0:2] = scales.view(np.uint8).reshape(64, 2)
    out = np.zeros(64 * 32, np.float32)
    assert R.ref_dequantize(2, blocks.reshape(-1), out, 64 * 32) == 0
    np.savez_compressed(os.path.join(HERE, "q4_0_dequant.npz"), blocks=blocks, values=out.reshape(64, 32))

    for name, spec in {**MODELS, **FLOAT_PLE_MODELS}.items():
        path = f"/tmp/lg_golden_{name}.gguf"
        lg.synth.write_model(path, **spec)
        ref = ob.Reference(path, 4)
        kv = ref.kv_new(N_PROMPT + N_GEN + 8)
        prng = np.random.default_rng(spec["seed"] + 1)
        prompt = prng.integers(0, spec["n_vocab"], N_PROMPT).astype(np.int32)
        ref.prefill(kv, prompt[:-1], 0)
        tok, pos = int(prompt[-1]), N_PROMPT - 1
        tokens, logits = [], {}
        for step in range(N_GEN):
            row = ref.forward(kv, tok, pos)
            best = int(np.argmax(row))              # first maximum, like the reference's scan
            if step in LOGIT_STEPS:
                logits[step] = row.copy()
            tokens.append(best)
            tok, pos = best, pos + 1
        hidden = ref.last_hidden()
        # model_forward_spec transcript on a fresh cache: perfect drafts, then a wrong one at each slot
        kv2 = ref.kv_new(N_PROMPT + N_GEN + 8)
        ref.prefill(kv2, prompt[:-1], 0)
        seq = [int(prompt[-1])] + tokens
        spec_in, spec_out, spec_adv, at, p2 = [], [], [], 0, N_PROMPT - 1
        for i in range(10):
            blk = seq[at:at + 4]
            if i % 4 != 0:
                blk[i % 4] = (blk[i % 4] + 1) % spec["n_vocab"]
            adv, out4 = ref.forward_spec(kv2, blk, p2)
            spec_in.append(blk); spec_out.append(out4.copy()); spec_adv.append(adv)
            at += adv; p2 += adv
        np.savez_compressed(
            os.path.join(HERE, f"ref_{name}.npz"),
            spec_json=np.frombuffer(json.dumps(spec, sort_keys=True).encode(), np.uint8),
            gguf_sha256=np.frombuffer(sha256(path).encode(), np.uint8),
            prompt=prompt, tokens=np.array(tokens, np.int32),
            logit_steps=np.array(sorted(logits), np.int32), logits=np.stack([logits[s] for s in sorted(logits)]),
            last_hidden=hidden, spec_in=np.array(spec_in, np.int32), spec_out=np.array(spec_out, np.int32),
            spec_adv=np.array(spec_adv, np.int32))
        print(name, "tokens", tokens[:16], "distinct", len(set(tokens)), "spec adv", spec_adv)
        ref.kv_free(kv); ref.kv_free(kv2); ref.close()


def draft_fixtures():
    assert ob.ref_available(4), "build the reference first: make -C oracle ref"
    for name, spec in MODELS.items():
        path, head = f"/tmp/lg_golden_{name}.gguf", f"/tmp/lg_golden_{name}_assistant.gguf"
        lg.synth.write_model(path, **spec)
        aspec = lg.synth.assistant_for(spec)
        lg.synth.write_assistant(head, **aspec)
        ref = ob.Reference(path, 4)
        t = ref.mtp_open(head)
        kv = ref.kv_new(N_PROMPT + 32)
        prng = np.random.default_rng(spec["seed"] + 2)
        prompt = prng.integers(0, spec["n_vocab"], N_PROMPT).astype(np.int32)
        ref.prefill(kv, prompt[:-1], 0)
        tok, pos = int(prompt[-1]), N_PROMPT - 1
        chosen, drafts, hiddens, logits = [], [], [], {}
        for step in range(16):
            tok = ref.forward_next(kv, tok, pos)          # chosen token, will sit at pos + 1
            pos += 1
            d, h, row = ref.mtp_draft(t, kv, tok, pos)
            chosen.append(tok); drafts.append(d); hiddens.append(h)
            if step in (0, 7, 15):
                logits[step] = row
        np.savez_compressed(
            os.path.join(HERE, f"ref_draft_{name}.npz"),
            spec_json=np.frombuffer(json.dumps(spec, sort_keys=True).encode(), np.uint8),
            assistant_json=np.frombuffer(json.dumps(aspec, sort_keys=True).encode(), np.uint8),
            gguf_sha256=np.frombuffer(sha256(path).encode(), np.uint8),
            assistant_sha256=np.frombuffer(sha256(head).encode(), np.uint8),
            prompt=prompt, chosen=np.array(chosen, np.int32), drafts=np.array(drafts, np.int32),
            hidden=np.stack(hiddens), logit_steps=np.array(sorted(logits), np.int32),
            logits=np.stack([logits[s] for s in sorted(logits)]))
        print(name, "chosen", chosen[:8], "drafts", drafts[:8], "accepted", sum(int(drafts[i] == chosen[i + 1]) for i in range(15)))
        ref.mtp_free(t); ref.kv_free(kv); ref.close()


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    if what in ("all", "model"):
        main()
    if what in ("all", "draft"):
        draft_fixtures()
