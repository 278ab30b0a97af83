"""Whole-forward oracle: the REF mode against the committed reference fixtures and, where its build
is present, against the reference's CPU backend itself; the int8-class mode against REF."""
import numpy as np
import pytest

N_PROMPT, N_GEN = 128, 64


@pytest.mark.parametrize("name", ["tiny", "tiny_full", "tiny_full_f32"])
def test_ref_mode_reproduces_reference_fixture(ob, model_path, golden, name):
    """Greedy tokens, logits rows and last_hidden recorded from the reference's `run` path
    (model_prefill + model_forward; tests/golden/make_fixtures.py) — bit for bit."""
    g = golden(f"ref_{name}.npz")
    path, _ = model_path(name)
    o = ob.Oracle(path)
    try:
        kv = o.kv_new(N_PROMPT + N_GEN + 8, ob.REF)
        prompt = g["prompt"]
        o.prefill(kv, prompt[:-1], 0, ob.REF)
        tok, pos = int(prompt[-1]), N_PROMPT - 1
        steps = {int(s): i for i, s in enumerate(g["logit_steps"])}
        for step in range(N_GEN):
            best, logits, hidden = o.forward(kv, tok, pos, ob.REF, want_hidden=True)
            assert best == int(g["tokens"][step]), f"step {step}"
            if step in steps:
                assert np.array_equal(logits.view(np.uint32), g["logits"][steps[step]].view(np.uint32)), f"logits step {step}"
            tok, pos = best, pos + 1
        assert np.array_equal(hidden.view(np.uint32), g["last_hidden"].view(np.uint32))
        # model_forward_spec transcript (sequential verify, src/cpu/model-cpu.c:51-58)
        kv2 = o.kv_new(N_PROMPT + N_GEN + 8, ob.REF)
        o.prefill(kv2, prompt[:-1], 0, ob.REF)
        p = N_PROMPT - 1
        for blk, want_out, want_adv in zip(g["spec_in"], g["spec_out"], g["spec_adv"]):
            adv, out, _ = o.forward_spec(kv2, blk, p, ob.REF)
            assert adv == int(want_adv) and out[:adv].tolist() == want_out[:adv].tolist()
            p += adv
        o.kv_free(kv); o.kv_free(kv2)
    finally:
        o.close()


FLOAT_PLE = ["tiny_full_f32", "tiny_full_f16", "tiny_full_bf16"]   # per-layer-embedding matrices kept in a float type


@pytest.mark.parametrize("name", ["tiny", "tiny_full"] + FLOAT_PLE)
def test_ref_mode_against_live_reference(ob, model_path, name):
    if not ob.ref_available(4):
        pytest.skip("reference build absent (needs /root/reference; run make -C oracle ref)")
    path, spec = model_path(name)
    o, r = ob.Oracle(path), ob.Reference(path, 4)
    try:
        rng = np.random.default_rng(77)
        prompt = rng.integers(0, spec["n_vocab"], 150).astype(np.int32)   # past the 128-row sliding ring
        okv, rkv = o.kv_new(200, ob.REF), r.kv_new(200)
        o.prefill(okv, prompt[:-1], 0, ob.REF); r.prefill(rkv, prompt[:-1], 0)
        for L, (K, V) in r.kv_views(rkv).items():
            k2, v2 = o.kv_views(okv)[L]
            assert K.dtype == k2.dtype and np.array_equal(K.view(np.uint8), k2.view(np.uint8)) and np.array_equal(V.view(np.uint8), v2.view(np.uint8))
        tok, pos = int(prompt[-1]), 149
        for _ in range(8):
            want = r.forward(rkv, tok, pos)
            best, got, hid = o.forward(okv, tok, pos, ob.REF, want_hidden=True)
            assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
            assert np.array_equal(r.last_hidden().view(np.uint32), hid.view(np.uint32))
            tok, pos = best, pos + 1
    finally:
        o.close(); r.close()


@pytest.mark.parametrize("name", ["tiny", "tiny_full"] + FLOAT_PLE)
def test_int8_class_stays_in_the_q8_noise_band_of_ref(ob, model_path, name):
    """The int8-class forward is the same network with q8 activations: teacher-forced on the REF
    tokens its logits stay within a few 1e-2 relative L2 of REF at every step.  A dropped residual,
    a swapped norm weight or a misplaced quantization point moves this to O(1)."""
    path, spec = model_path(name)
    o = ob.Oracle(path)
    try:
        rng = np.random.default_rng(spec["seed"] + 1)
        prompt = rng.integers(0, spec["n_vocab"], 140).astype(np.int32)
        kvs = {m: o.kv_new(220, m) for m in (ob.REF, ob.I8, ob.I8_LIBM)}
        for m, kv in kvs.items():
            o.prefill(kv, prompt[:-1], 0, m)
        tok, pos = int(prompt[-1]), 139
        gaps, libm_gaps, agree = [], [], 0
        for _ in range(32):
            b0, l0, _ = o.forward(kvs[ob.REF], tok, pos, ob.REF)
            b1, l1, _ = o.forward(kvs[ob.I8], tok, pos, ob.I8)
            _, l2, _ = o.forward(kvs[ob.I8_LIBM], tok, pos, ob.I8_LIBM)
            gaps.append(np.linalg.norm(l1 - l0) / np.linalg.norm(l0))
            libm_gaps.append(np.linalg.norm(l2 - l1) / np.linalg.norm(l1))
            agree += b0 == b1
            tok, pos = b0, pos + 1
        assert max(gaps) < 0.3 and np.median(gaps) < 0.15
        # replacing lg_math.h by libm moves logits by no more than the q8 noise itself
        assert max(libm_gaps) <= 1.5 * max(gaps)
        assert agree >= 20
    finally:
        o.close()


@pytest.mark.parametrize("name", ["tiny", "tiny_full"] + FLOAT_PLE)
def test_f32_variant_of_the_int8_sequence_matches_ref_to_reorder_noise(ob, model_path, name):
    """I8_F32 runs forward_i8's exact op sequence (quantization points, PLE build, residual and scale placement,
    tile attention, this build's norm orders and elementary functions) with the quantization switched off and
    the reference's cache precision (f32 sliding rings).  What is left between it and REF is float reordering:
    teacher-forced on the REF tokens the logits agree to 1e-3 relative L2 at every step and every argmax is the
    same.  Any misplaced op in the shared sequence shows here at O(1e-1), far above the bar."""
    path, spec = model_path(name)
    o = ob.Oracle(path)
    try:
        rng = np.random.default_rng(spec["seed"] + 1)
        prompt = rng.integers(0, spec["n_vocab"], 140).astype(np.int32)
        kr, kf = o.kv_new(220, ob.REF), o.kv_new(220, ob.I8_F32)
        o.prefill(kr, prompt[:-1], 0, ob.REF); o.prefill(kf, prompt[:-1], 0, ob.I8_F32)
        tok, pos, gaps = int(prompt[-1]), 139, []
        for _ in range(32):
            b0, l0, h0 = o.forward(kr, tok, pos, ob.REF, want_hidden=True)
            b1, l1, h1 = o.forward(kf, tok, pos, ob.I8_F32, want_hidden=True)
            gaps.append(np.linalg.norm(l1 - l0) / np.linalg.norm(l0))
            assert b0 == b1
            assert np.linalg.norm(h1 - h0) <= 1e-3 * np.linalg.norm(h0)
            tok, pos = b0, pos + 1
        assert max(gaps) <= 1e-3, gaps
    finally:
        o.close()


def test_int8_class_sequential_spec_equals_plain_decode(ob, model_path):
    """verify == decode by construction in the oracle: the block form is the same forwards."""
    path, spec = model_path("tiny")
    o = ob.Oracle(path)
    try:
        rng = np.random.default_rng(5)
        prompt = rng.integers(0, spec["n_vocab"], 30).astype(np.int32)
        a, b = o.kv_new(80, ob.I8), o.kv_new(80, ob.I8)
        o.prefill(a, prompt[:-1], 0, ob.I8); o.prefill(b, prompt[:-1], 0, ob.I8)
        tok, pos, seq = int(prompt[-1]), 29, []
        for _ in range(12):
            tok = o.forward(a, tok, pos, ob.I8)[0]; seq.append(tok); pos += 1
        chain = [int(prompt[-1])] + seq
        at, pos = 0, 29
        while at + 4 <= 12:
            adv, out, _ = o.forward_spec(b, np.array(chain[at:at + 4], np.int32), pos, ob.I8)
            assert adv == 4 and out.tolist() == chain[at + 1:at + 5]
            at += adv; pos += adv
    finally:
        o.close()


def test_argmax_ties_resolve_to_the_lower_index(lg, ob, model_path, model_dir):
    """A vocabulary whose upper half repeats its lower half makes every logit a tie with its twin V/2 above:
    the greedy token is always the lower one (src/cpu/model-cpu.c:477-478), in REF and in the int8 class."""
    import os
    import shutil
    from conftest import gguf_tensor_span
    src, spec = model_path("tiny")
    path = os.path.join(str(model_dir), "tiny_tied_cpu.gguf")
    shutil.copyfile(src, path)
    off, nbytes, dims = gguf_tensor_span(path, "token_embd.weight")
    with open(path, "r+b") as f:
        f.seek(off); lower = f.read(nbytes // 2); f.seek(off + nbytes // 2); f.write(lower)
    half = dims[1] // 2
    o = ob.Oracle(path)
    try:
        for mode in (ob.REF, ob.I8):
            kv = o.kv_new(32, mode)
            tok = 3
            for pos in range(6):
                best, row, _ = o.forward(kv, tok, pos, mode)
                assert np.array_equal(row[:half].view(np.uint32), row[half:].view(np.uint32))
                assert best < half and row[best] == row.max()
                tok = best
    finally:
        o.close()
