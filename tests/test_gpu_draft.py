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


@pytest.mark.parametrize("name,rows", [("tiny", 4), ("tiny_full", 5), ("tiny_full", 2)])
def test_device_rounds_equal_host_driven_rounds(lg, gpu_required, model_path, model_dir, name, rows):
    """lg_hip_mtp_rounds keeps draft, chained drafts, verify, accept and the next chosen token on the device; the
    blocks it verified, the successors and the accept counts must be those of the host-driven loop
    (src/run.c:54-71 of the reference), round for round."""
    path, spec = model_path(name)
    head = write_head(lg, model_dir, name, spec)
    rng = np.random.default_rng(9)
    prompt = rng.integers(1, spec["n_vocab"], 40).astype(np.int32)
    n_rounds = 7
    gpu = lg.hiplib.HipBackend(path, 40 + rows * (n_rounds + 1) + 8, max_rows=8)
    t = gpu.mtp_open(head)
    try:
        def start():
            gpu.new_cache()
            gpu.prefill(prompt[:-1], 0)
            return gpu.forward_next(int(prompt[-1]), len(prompt) - 1), len(prompt)
        best, pos = start()
        want_blocks, want_out, want_adv = [], [], []
        for _ in range(n_rounds):
            toks = [best]
            for j in range(1, rows):
                toks.append(gpu.mtp_draft(t, toks[-1], pos + j - 1, chain=j > 1))
            adv, out = gpu.forward_spec(np.array(toks, np.int32), pos)
            want_blocks.append(toks); want_out.append(out.tolist()); want_adv.append(adv)
            pos += adv; best = int(out[adv - 1])
        first, pos0 = start()
        print(f"{name} rows={rows}: {n_rounds} device rounds from pos {pos0}", flush=True)
        blocks, out, adv, final_pos = gpu.mtp_rounds(t, first, pos0, rows, n_rounds)
        assert adv.tolist() == want_adv
        assert blocks.tolist() == want_blocks
        assert out.tolist() == want_out                        # rejected rows included: both loops verified the same blocks
        assert final_pos == pos0 + int(adv.sum()) == pos
        # the captured round replayed for a shorter run from the same state gives the same first rounds
        first, pos0 = start()
        print(f"{name} rows={rows}: replay, 3 rounds", flush=True)
        b2, o2, a2, fp2 = gpu.mtp_rounds(t, first, pos0, rows, 3)
        assert a2.tolist() == want_adv[:3] and b2.tolist() == want_blocks[:3] and o2.tolist() == want_out[:3]
        assert fp2 == pos0 + int(a2.sum())
        # and a verify step from the host continues from there as if the rounds had been host-driven
        nxt = int(o2[2, a2[2] - 1])
        d1 = gpu.mtp_draft(t, nxt, fp2)
        assert d1 == want_blocks[3][1]
    finally:
        gpu.mtp_close(t); gpu.close()


@pytest.mark.parametrize("name", ["tiny", "tiny_full"])
def test_generation_with_device_rounds_equals_plain_greedy(lg, gpu_required, model_path, model_dir, name):
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
            host = gpu.generate_mtp(t, prompt, n_gen, rows)
            for batch in (1, 3, 16):
                gpu.new_cache()
                print(f"{name} block {rows}, {batch} rounds per batch", flush=True)
                out, steps, nd, na = gpu.generate_mtp_rounds(t, prompt, n_gen, rows, batch)
                assert list(out) == list(plain)
                assert (steps, nd, na) == host[1:]             # the same rounds ran, only without the host in between
            gpu.mtp_close(t)
    finally:
        gpu.close()


def test_run_hip_cli_with_a_draft_head(lg, gpu_required, model_path, model_dir):
    """run-hip -mtp assistant.gguf: exit status 0 means the speculative output equalled its own plain greedy run;
    device-resident rounds (-rounds 8) and the host-driven loop (-rounds 0) print the same ids."""
    import subprocess
    from conftest import ROOT
    exe = os.path.join(ROOT, "little-gemma_amd", "host", "run-hip")
    assert os.path.exists(exe), "run-hip is not built (run __graft_entry__.build())"
    path, spec = model_path("tiny_full")
    head = write_head(lg, model_dir, "tiny_full", spec)
    outs = []
    for rounds in ("8", "0"):
        print(f"run-hip -rounds {rounds}", flush=True)
        r = subprocess.run([exe, "-m", path, "-p", "5,17,300,42,7,1000", "-n", "40", "-mtp", head, "-rounds", rounds],
                           capture_output=True, text=True, timeout=100)
        assert r.returncode == 0, r.stderr[-2000:]
        assert "is byte-identical to plain greedy output" in r.stderr
        ids = [int(x) for x in r.stdout.strip().splitlines()[-1].split(",")]
        assert len(ids) == 40
        outs.append(ids)
    assert outs[0] == outs[1]


def test_device_rounds_refuse_what_does_not_fit(lg, gpu_required, model_path, model_dir):
    path, spec = model_path("tiny")
    head = write_head(lg, model_dir, "tiny", spec)
    gpu = lg.hiplib.HipBackend(path, 64, max_rows=4)
    t = gpu.mtp_open(head)
    try:
        gpu.prefill(np.arange(1, 9, dtype=np.int32), 0)
        best = gpu.forward_next(9, 8)
        for rows, n, pos in ((1, 2, 9), (5, 2, 9), (4, 14, 9), (4, 0, 9), (4, 2, 0)):      # width, width, cache, count, position
            with pytest.raises(lg.hiplib.HipError):
                gpu.mtp_rounds(t, best, pos, rows, n)
        with pytest.raises(lg.hiplib.HipError):
            gpu.mtp_rounds(t, spec["n_vocab"], 9, 4, 2)
        blocks, out, adv, fp = gpu.mtp_rounds(t, best, 9, 4, 13)          # 9 + 4*13 = 61 <= 64: fits
        assert fp == 9 + int(adv.sum()) and blocks[0, 0] == best
    finally:
        gpu.mtp_close(t); gpu.close()


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


def test_12b_width_head(lg, ob, gpu_required, model_path, model_dir):
    """A head on a 3840-wide backbone (the 12B width on 6 layers): its pre-projection has 7680 inputs, 240 blocks,
    which is above 128 and no multiple of 32, so it runs in 8 K segments; draft and chained draft against the oracle."""
    path, spec = model_path("g12b", n_layer=6, n_ff=3072, n_vocab=8192)
    head = write_head(lg, model_dir, "g12b_w", spec)
    assert lg.hiplib.load_hip().lg_hip_segments(2 * spec["n_embd"]) == 8
    rng = np.random.default_rng(5)
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
        print("3840-wide head: draft + chained draft", flush=True)
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
