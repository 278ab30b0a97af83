"""GPU parity of the draft head (mtp_draft_device / mtp_draft_chain_device behind the model.h
interface): every drafted token, the head's hidden state and its logits are bit-identical to the
int8-class oracle, through whole speculative rounds (draft, chained drafts, verify) whose cache
contents are mirrored on the CPU; and generation with the head drafting emits exactly the plain
greedy sequence."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def write_head(lg, model_dir, name, spec, **over):
    path = os.path.join(str(model_dir), f"assistant_{name}" + "".join(f"_{k}{v}" for k, v in sorted(over.items())) + ".gguf")
    if not os.path.exists(path):
        lg.synth.write_assistant(path, **lg.synth.assistant_for(spec, **over))
    return path


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("name,rows", [("tiny", 4), ("tiny_full", 5), ("tiny_full", 2)])
def test_speculative_rounds_match_oracle(lg, ob, gpu_required, model_path, model_dir, name, rows):
    """The reference's mtp_step (src/run.c:54-71) for 12 rounds: draft from the target's hidden,
    rows-2 chained drafts, verify.  Device and oracle run the same calls; tokens, hidden states and
    logits of every draft are compared bit for bit, then the verify results."""
    path, spec = model_path(name)
    head = write_head(lg, model_dir, name, spec)
    rng = np.random.default_rng(11)
    prompt = rng.integers(1, spec["n_vocab"], 70).astype(np.int32)
    max_seq = 70 + 12 * rows + 8
    o = ob.Oracle(path)
    od = o.mtp_open(head)
    gpu = lg.hiplib.HipBackend(path, max_seq, max_rows=8)
    t = gpu.mtp_open(head)
    try:
        ni, nv = od.info["n_inner"], od.info["n_vocab"]
        gpu.mtp_store_logits(t, True)
        kv = o.kv_new(max_seq, ob.I8)
        o.prefill(kv, prompt[:-1], 0, ob.I8)
        gpu.prefill(prompt[:-1], 0)
        pos = len(prompt) - 1
        best, _, hid = o.forward(kv, int(prompt[-1]), pos, ob.I8, want_logits=True, want_hidden=True)
        assert gpu.forward_next(int(prompt[-1]), pos) == best
        pos += 1
        for rnd in range(12):
            print(f"{name} rows {rows}: round {rnd} at position {pos}", flush=True)
            toks = [best]
            want, wh, wl = od.draft(kv, best, pos, hid, ob.I8, want_logits=True)
            got = gpu.mtp_draft(t, best, pos, chain=False)
            assert np.array_equal(bits(gpu.mtp_hidden(t, ni)), bits(wh)), f"draft hidden, round {rnd}"
            assert np.array_equal(bits(gpu.mtp_logits(t, nv)), bits(wl)), f"draft logits, round {rnd}"
            assert got == want
            toks.append(got)
            for j in range(2, rows):
                hp = od.post(wh, ob.I8)
                want, wh, wl = od.draft(kv, toks[j - 1], pos + j - 1, hp, ob.I8, want_logits=True)
                got = gpu.mtp_draft(t, toks[j - 1], pos + j - 1, chain=True)
                assert np.array_equal(bits(gpu.mtp_hidden(t, ni)), bits(wh)), f"chained draft {j} hidden, round {rnd}"
                assert np.array_equal(bits(gpu.mtp_logits(t, nv)), bits(wl)), f"chained draft {j} logits, round {rnd}"
                assert got == want
                toks.append(got)
            adv, out, hid = o.forward_spec_all(kv, toks, pos, ob.I8, want_hidden=True)
            gadv, gout = gpu.forward_spec(toks, pos)
            assert gadv == adv and list(gout[:adv]) == list(out[:adv])
            assert np.array_equal(bits(gpu.last_hidden(spec["n_embd"])), bits(hid))
            pos += adv
            best = int(out[adv - 1])
    finally:
        gpu.mtp_close(t); gpu.close(); od.close(); o.close()


@pytest.mark.parametrize("name", ["tiny", "tiny_full"])
def test_generation_with_the_head_equals_plain_greedy(lg, ob, gpu_required, model_path, model_dir, name):
    """docs/mtp.md:16-19 of the reference: output with -mtp is byte-identical to plain decoding."""
    path, spec = model_path(name)
    head = write_head(lg, model_dir, name, spec)
    rng = np.random.default_rng(5)
    prompt = rng.integers(1, spec["n_vocab"], 48).astype(np.int32)
    n_gen = 96
    gpu = lg.hiplib.HipBackend(path, 48 + n_gen + 1, max_rows=8)
    try:
        plain, _ = gpu.generate(prompt, n_gen, rows=1)
        for rows in (2, 4):
            gpu.new_cache()
            t = gpu.mtp_open(head)
            out, steps, nd, na = gpu.generate_mtp(t, prompt, n_gen, rows)
            gpu.mtp_close(t)
            print(f"{name} block {rows}: {steps} steps, {na}/{nd} drafts accepted", flush=True)
            assert list(out) == list(plain)
            assert 0 <= na <= nd <= (rows - 1) * steps
    finally:
        gpu.close()


def test_head_without_post_projection_cannot_chain(lg, gpu_required, model_path, model_dir):
    path, spec = model_path("tiny")
    head = write_head(lg, model_dir, "tiny", spec, has_post=0)
    gpu = lg.hiplib.HipBackend(path, 64, max_rows=4)
    try:
        # the loader of the reference requires both projections (src/mtp.c:163-167): such a file is refused
        with pytest.raises(lg.hiplib.HipError):
            gpu.mtp_open(head)
    finally:
        gpu.close()


def test_e4b_shape_head(lg, ob, gpu_required, model_path, model_dir):
    """A 4-block, 256-wide head on the E4B-shaped target: the 5120-wide pre-projection (32 K segments),
    cross-attention into 256-wide heads and the 262144-row head matmul, against the oracle."""
    path, spec = model_path("e4b")
    head = write_head(lg, model_dir, "e4b", spec, n_ff=2048)
    rng = np.random.default_rng(3)
    prompt = rng.integers(1, spec["n_vocab"], 12).astype(np.int32)
    o = ob.Oracle(path)
    od = o.mtp_open(head)
    gpu = lg.hiplib.HipBackend(path, 64, max_rows=5)
    t = gpu.mtp_open(head)
    try:
        kv = o.kv_new(64, ob.I8)
        o.prefill(kv, prompt[:-1], 0, ob.I8)
        gpu.prefill(prompt[:-1], 0)
        pos = len(prompt) - 1
        best, _, hid = o.forward(kv, int(prompt[-1]), pos, ob.I8, want_logits=True, want_hidden=True)
        assert gpu.forward_next(int(prompt[-1]), pos) == best
        print("e4b head: draft + chained draft", flush=True)
        want, wh, _ = od.draft(kv, best, pos + 1, hid, ob.I8)
        got = gpu.mtp_draft(t, best, pos + 1)
        assert np.array_equal(bits(gpu.mtp_hidden(t, od.info["n_inner"])), bits(wh))
        assert got == want
        want2, wh2, _ = od.draft(kv, want, pos + 2, od.post(wh, ob.I8), ob.I8)
        got2 = gpu.mtp_draft(t, got, pos + 2, chain=True)
        assert np.array_equal(bits(gpu.mtp_hidden(t, od.info["n_inner"])), bits(wh2))
        assert got2 == want2
    finally:
        gpu.mtp_close(t); gpu.close(); od.close(); o.close()
