"""The draft head (gemma4-assistant) on the CPU: the oracle's REF mode against the reference's own
host draft (committed fixture, and the live reference build where present), the int8 class against
REF, the device-order verify step, and the host loader's checks."""
import json
import os

import numpy as np
import pytest


def head_path(lg, model_dir, name, spec, **over):
    path = os.path.join(str(model_dir), f"assistant_{name}" + "".join(f"_{k}{v}" for k, v in sorted(over.items())) + ".gguf")
    if not os.path.exists(path):
        lg.synth.write_assistant(path, **lg.synth.assistant_for(spec, **over))
    return path


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("name", ["tiny", "tiny_full"])
def test_ref_draft_reproduces_reference_fixture(lg, ob, model_path, model_dir, golden, name):
    """16 decode steps, a draft after each: tokens, the head's hidden and its logits are the bits the
    reference's mtp_draft (src/mtp.c:258-356) produced on the same two files."""
    g = golden(f"ref_draft_{name}.npz")
    path, spec = model_path(name)
    assert json.loads(bytes(g["spec_json"]).decode()) == json.loads(json.dumps(spec, sort_keys=True))
    aspec = json.loads(bytes(g["assistant_json"]).decode())
    head = os.path.join(str(model_dir), f"fixture_assistant_{name}.gguf")
    lg.synth.write_assistant(head, **aspec)
    o = ob.Oracle(path)
    d = o.mtp_open(head)
    try:
        prompt = g["prompt"]
        kv = o.kv_new(len(prompt) + 32, ob.REF)
        o.prefill(kv, prompt[:-1], 0, ob.REF)
        tok, pos = int(prompt[-1]), len(prompt) - 1
        steps = {int(s): i for i, s in enumerate(g["logit_steps"])}
        for step in range(16):
            tok, _, hid = o.forward(kv, tok, pos, ob.REF, want_logits=True, want_hidden=True)
            pos += 1
            assert tok == int(g["chosen"][step])
            dt, dh, dl = d.draft(kv, tok, pos, hid, ob.REF, want_logits=True)
            assert dt == int(g["drafts"][step]), f"draft token at step {step}"
            assert np.array_equal(bits(dh), bits(g["hidden"][step])), f"draft hidden at step {step}"
            if step in steps:
                assert np.array_equal(bits(dl), bits(g["logits"][steps[step]])), f"draft logits at step {step}"
    finally:
        d.close(); o.close()


@pytest.mark.parametrize("name,over", [("tiny", {}), ("tiny_full", {}), ("tiny_full", dict(n_full=4, out_scale=0.9, seed=99)),
                                       ("tiny_full", dict(n_layer=2, n_full=0))])
def test_ref_draft_against_live_reference(lg, ob, model_path, model_dir, name, over):
    """Where the reference build is present: a sliding-only, a mixed and a global-only head, bit for
    bit.  The global blocks read f16 rows through the reference's private half reader, which halves
    subnormals (src/mtp.c:96-113); REF mode keeps that, or this comparison fails."""
    if not ob.ref_available(4):
        pytest.skip("reference build absent (oracle/_ref)")
    path, spec = model_path(name)
    head = head_path(lg, model_dir, name, spec, **over)
    o, r = ob.Oracle(path), ob.Reference(path, 4)
    d, rt = o.mtp_open(head), r.mtp_open(head)
    try:
        rng = np.random.default_rng(17)
        prompt = rng.integers(0, spec["n_vocab"], 150).astype(np.int32)     # past the 128-row sliding ring
        kvo, kvr = o.kv_new(200, ob.REF), r.kv_new(200)
        o.prefill(kvo, prompt[:-1], 0, ob.REF); r.prefill(kvr, prompt[:-1], 0)
        tok, pos = int(prompt[-1]), 149
        for step in range(6):
            best, _, hid = o.forward(kvo, tok, pos, ob.REF, want_logits=True, want_hidden=True)
            assert r.forward_next(kvr, tok, pos) == best
            pos += 1
            wt, wh, wl = r.mtp_draft(rt, kvr, best, pos)
            gt, gh, gl = d.draft(kvo, best, pos, hid, ob.REF, want_logits=True)
            assert gt == wt and np.array_equal(bits(gh), bits(wh)) and np.array_equal(bits(gl), bits(wl)), f"step {step}"
            tok = best
    finally:
        r.mtp_free(rt); d.close(); o.close(); r.close()


@pytest.mark.parametrize("blocks,limit", [(1, 0.2), (4, 0.6)])
def test_int8_draft_stays_near_ref(lg, ob, model_path, model_dir, blocks, limit):
    """Same inputs (token, h_prev, cache history), q8 activations instead of f32: one block moves the
    logits by the q8 noise of the target path; four random-init blocks amplify it but stay correlated.
    A wrong cache layer, a missing rotation or a shifted key range gives O(1) already for one block."""
    path, spec = model_path("tiny_full")
    head = head_path(lg, model_dir, "tiny_full", spec, n_layer=blocks, n_full=1)
    o = ob.Oracle(path)
    d = o.mtp_open(head)
    try:
        rng = np.random.default_rng(23)
        prompt = rng.integers(0, spec["n_vocab"], 60).astype(np.int32)
        kr, ki = o.kv_new(100, ob.REF), o.kv_new(100, ob.I8)
        o.prefill(kr, prompt[:-1], 0, ob.REF); o.prefill(ki, prompt[:-1], 0, ob.I8)
        tok, pos, gaps = int(prompt[-1]), 59, []
        for _ in range(8):
            best, _, hid = o.forward(kr, tok, pos, ob.REF, want_logits=True, want_hidden=True)
            o.forward(ki, tok, pos, ob.I8)
            pos += 1
            _, _, l0 = d.draft(kr, best, pos, hid, ob.REF, want_logits=True)
            _, _, l1 = d.draft(ki, best, pos, hid, ob.I8, want_logits=True)
            gaps.append(np.linalg.norm(l1 - l0) / np.linalg.norm(l0))
            tok = best
        assert max(gaps) < limit, gaps
    finally:
        d.close(); o.close()


@pytest.mark.parametrize("blocks", [1, 4])
def test_f32_variant_of_the_int8_draft_sequence_matches_ref_to_reorder_noise(lg, ob, model_path, model_dir, blocks):
    """The int8-class draft with its quantization switched off (I8_F32: same op sequence, tile attention over
    keys < pos, this build's norm orders and functions, f32 activations) must sit within float reordering
    noise of the reference host draft: 1e-3 relative L2, same argmax.  The wide band of the q8 test above
    cannot tell a misplaced op from int8 noise; this one can."""
    path, spec = model_path("tiny_full")
    head = head_path(lg, model_dir, "tiny_full", spec, n_layer=blocks, n_full=1)
    o = ob.Oracle(path)
    d = o.mtp_open(head)
    try:
        rng = np.random.default_rng(29)
        prompt = rng.integers(0, spec["n_vocab"], 150).astype(np.int32)       # past the 128-row sliding window
        kr, kf = o.kv_new(200, ob.REF), o.kv_new(200, ob.I8_F32)
        o.prefill(kr, prompt[:-1], 0, ob.REF); o.prefill(kf, prompt[:-1], 0, ob.I8_F32)
        tok, pos, gaps = int(prompt[-1]), 149, []
        for _ in range(8):
            best, _, hid = o.forward(kr, tok, pos, ob.REF, want_logits=True, want_hidden=True)
            o.forward(kf, tok, pos, ob.I8_F32)
            pos += 1
            t0, _, l0 = d.draft(kr, best, pos, hid, ob.REF, want_logits=True)
            t1, _, l1 = d.draft(kf, best, pos, hid, ob.I8_F32, want_logits=True)
            gaps.append(np.linalg.norm(l1 - l0) / np.linalg.norm(l0))
            assert t0 == t1
            tok = best
        assert max(gaps) <= 1e-3, gaps
    finally:
        d.close(); o.close()


def test_draft_sees_only_positions_before_its_own(lg, ob, model_path, model_dir):
    """The cache row at the draft position (and later ones) must not influence the draft: overwrite
    them with noise and the int8-class draft is unchanged; change the row just before and it moves."""
    path, spec = model_path("tiny_full")
    head = head_path(lg, model_dir, "tiny_full", spec)
    o = ob.Oracle(path)
    d = o.mtp_open(head)
    try:
        rng = np.random.default_rng(2)
        prompt = rng.integers(0, spec["n_vocab"], 40).astype(np.int32)
        kv = o.kv_new(96, ob.I8)
        o.prefill(kv, prompt, 0, ob.I8)
        hid = rng.standard_normal(spec["n_embd"]).astype(np.float32)
        base = d.draft(kv, 7, 40, hid, ob.I8, want_logits=True)[2]
        views = o.kv_views(kv)
        for L, (K, V) in views.items():
            for p in (40, 41, 42):
                K[p % K.shape[0]] = rng.integers(0, 0x3C00, K.shape[1]).astype(np.uint16)
                V[p % V.shape[0]] = rng.integers(0, 0x3C00, V.shape[1]).astype(np.uint16)
        assert np.array_equal(bits(d.draft(kv, 7, 40, hid, ob.I8, want_logits=True)[2]), bits(base))
        src = spec["n_layer"] - spec["shared_kv_layers"] - 1          # last owning layer: the global cache the last block reads
        views[src][1][39 % views[src][1].shape[0]] ^= 0x0200
        assert not np.array_equal(bits(d.draft(kv, 7, 40, hid, ob.I8, want_logits=True)[2]), bits(base))
    finally:
        d.close(); o.close()


def test_device_order_verify_equals_sequential_verify(ob, model_path):
    """lgo_forward_spec_all forwards every row (as the device does) and must agree with the
    reference-order lgo_forward_spec on adv and on out[0..adv-1]."""
    path, spec = model_path("tiny")
    o = ob.Oracle(path)
    try:
        rng = np.random.default_rng(9)
        prompt = rng.integers(0, spec["n_vocab"], 24).astype(np.int32)
        a, b = o.kv_new(80, ob.I8), o.kv_new(80, ob.I8)
        o.prefill(a, prompt[:-1], 0, ob.I8); o.prefill(b, prompt[:-1], 0, ob.I8)
        tok, pos = int(prompt[-1]), 23
        for i in range(6):
            blk = [tok] + [int(x) for x in rng.integers(0, spec["n_vocab"], 3)]
            adv1, out1, h1 = o.forward_spec(a, blk, pos, ob.I8, want_hidden=True)
            adv2, out2, h2 = o.forward_spec_all(b, blk, pos, ob.I8, want_hidden=True)
            assert adv1 == adv2 and list(out1[:adv1]) == list(out2[:adv2]) and np.array_equal(bits(h1), bits(h2))
            tok, pos = int(out1[adv1 - 1]), pos + adv1
    finally:
        o.close()


def test_host_loader_checks_the_head_against_the_target(lg, model_path, model_dir):
    """mtp_open (host/mtp.c, restating src/mtp.c:124-215): accepts a fitting file, refuses a head built
    for another backbone width, another head size, or a file of the wrong architecture."""
    path, spec = model_path("tiny_full")
    B = lg.hiplib.load_backend()
    s = B.lg_session_open(os.fsencode(path))
    assert s
    try:
        good = head_path(lg, model_dir, "tiny_full", spec)
        t = B.lg_session_mtp_open(s, os.fsencode(good))
        assert t
        B.lg_session_mtp_close(t)
        assert not B.lg_session_mtp_open(s, os.fsencode(head_path(lg, model_dir, "tiny_full", spec, n_backbone=768)))
        assert not B.lg_session_mtp_open(s, os.fsencode(head_path(lg, model_dir, "tiny_full", spec, head_dim_swa=32, head_dim_full=32)))
        assert not B.lg_session_mtp_open(s, os.fsencode(path))
    finally:
        B.lg_session_close(s)
