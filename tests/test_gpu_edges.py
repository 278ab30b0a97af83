"""Two edge cases of the reference interface on the GPU: argmax ties (the lower index wins,
src/cuda/model-cuda.cuh:703-720, src/cpu/model-cpu.c:477-478) and the sampling hook model_pick
(include/model.h:105-111, src/cuda/mtp-kernel.cuh:103-118)."""
import ctypes as C
import os
import shutil

import numpy as np
import pytest

from conftest import gguf_tensor_span
from test_gpu_draft import write_head

pytestmark = pytest.mark.gpu


def duplicate_upper_vocabulary(path):
    """Rows V/2 .. V-1 of token_embd become copies of rows 0 .. V/2-1: with the tied head every logit
    then appears twice, V/2 apart, so every argmax is a tie."""
    off, nbytes, dims = gguf_tensor_span(path, "token_embd.weight")
    with open(path, "r+b") as f:
        f.seek(off)
        lower = f.read(nbytes // 2)
        f.seek(off + nbytes // 2)
        f.write(lower)
    return dims[1]


def test_argmax_ties_resolve_to_the_lower_index(lg, ob, gpu_required, model_path, model_dir):
    src, spec = model_path("tiny_full")
    path = os.path.join(str(model_dir), "tiny_full_tied.gguf")
    shutil.copyfile(src, path)
    V = duplicate_upper_vocabulary(path)
    head_src = write_head(lg, model_dir, "tiny_full", spec)
    head = os.path.join(str(model_dir), "assistant_tied.gguf")
    shutil.copyfile(head_src, head)
    assert duplicate_upper_vocabulary(head) == V
    half = V // 2
    rng = np.random.default_rng(41)
    prompt = rng.integers(0, half, 40).astype(np.int32)
    o = ob.Oracle(path)
    od = o.mtp_open(head)
    gpu = lg.hiplib.HipBackend(path, 160, max_rows=5)
    t = gpu.mtp_open(head)
    try:
        kv = o.kv_new(160, ob.I8)
        o.prefill(kv, prompt[:-1], 0, ob.I8)
        gpu.prefill(prompt[:-1], 0)
        gpu.set_option("store_logits", 1)
        print("ties: one-row decode", flush=True)
        tok, pos = int(prompt[-1]), len(prompt) - 1
        for _ in range(6):                                # model_forward_next: argmax on the device
            want, row, hid = o.forward(kv, tok, pos, ob.I8, want_hidden=True)
            got = gpu.forward_next(tok, pos)
            dev = gpu.logits_row(0, V)
            assert np.array_equal(dev[:half].view(np.uint32), dev[half:].view(np.uint32))      # every value is tied
            assert int(np.argmax(dev)) < half and dev[got] == dev.max()
            assert got == want and got < half
            tok, pos = got, pos + 1
        print("ties: draft head", flush=True)
        d_want, d_hid, _ = od.draft(kv, tok, pos, hid, ob.I8, want_logits=True)
        d_got = gpu.mtp_draft(t, tok, pos, chain=False)
        assert d_got == d_want and d_got < half
        print("ties: verify rows", flush=True)
        for step in range(4):                             # verify rows: every row's successor is the lower twin
            blk = np.array([tok] + [int(x) for x in rng.integers(0, half, 4)], np.int32)
            adv, out, _ = o.forward_spec_all(kv, blk, pos, ob.I8, want_hidden=True)
            gadv, gout = gpu.forward_spec(blk, pos)
            assert gadv == adv and gout.tolist() == list(out)
            assert all(int(x) < half for x in gout)
            for j in range(5):
                dev = gpu.logits_row(j, V)
                assert dev[int(gout[j])] == dev.max() == dev[int(gout[j]) + half]
            tok, pos = int(out[adv - 1]), pos + adv
    finally:
        gpu.mtp_close(t); gpu.close(); od.close(); o.close()


PICK = C.CFUNCTYPE(C.c_int, C.POINTER(C.c_float), C.c_int)


def second_best(row):
    """A deterministic rule that is not the argmax: the index of the second largest value (lower index on ties)."""
    order = np.lexsort((np.arange(row.size), -row))
    return int(order[1])


def test_sampling_hook_replaces_the_argmax(lg, ob, gpu_required, model_path):
    """With model_pick set the backend reads every row's logits back, lets the hook choose, accepts while the
    choice agrees with the next draft, and re-points the hidden state at the last accepted row."""
    path, spec = model_path("tiny_full")
    V, E, rows = spec["n_vocab"], spec["n_embd"], 4
    rng = np.random.default_rng(43)
    prompt = rng.integers(0, V, 50).astype(np.int32)
    o = ob.Oracle(path)
    gpu = lg.hiplib.HipBackend(path, 200, max_rows=rows)
    calls = []

    def pick(ptr, n):
        row = np.ctypeslib.as_array(ptr, shape=(n,))
        calls.append(n)
        return second_best(row)

    hook = PICK(pick)
    slot = C.c_void_p.in_dll(gpu.B, "model_pick")
    try:
        kv = o.kv_new(200, ob.I8)
        o.prefill(kv, prompt[:-1], 0, ob.I8)
        gpu.prefill(prompt[:-1], 0)
        slot.value = C.cast(hook, C.c_void_p).value
        tok, pos = int(prompt[-1]), len(prompt) - 1
        seen = set()
        for step in range(10):
            # the oracle's own chain under the same rule gives drafts that hold; plant the first wrong one
            first_bad = int(rng.integers(1, rows + 1))
            blk, picks, hiddens = [tok], [], []
            for j in range(rows):
                _, row, hid = o.forward(kv, blk[j], pos + j, ob.I8, want_hidden=True)
                picks.append(second_best(row)); hiddens.append(hid)
                if j + 1 < rows:
                    nxt = picks[j] if j + 1 < first_bad else (picks[j] + 1 + int(rng.integers(0, V - 1))) % V
                    blk.append(nxt)
            want_adv = 1
            while want_adv < rows and picks[want_adv - 1] == blk[want_adv]:
                want_adv += 1
            print(f"hook step {step} pos {pos} first_bad {first_bad} adv {want_adv}", flush=True)
            calls.clear()
            adv, out = gpu.forward_spec(np.array(blk, np.int32), pos)
            assert len(calls) == rows and all(n == V for n in calls)
            assert adv == want_adv and out.tolist() == picks
            assert np.array_equal(gpu.last_hidden(E).view(np.uint32), hiddens[adv - 1].view(np.uint32))
            seen.add(adv)
            tok, pos = picks[adv - 1], pos + adv
        assert len(seen) >= 2                              # both partial and full acceptance were exercised
    finally:
        slot.value = None
        gpu.close(); o.close()


@pytest.mark.parametrize("rows,name,over", [(2, "tiny_full", {}), (5, "tiny_full", {}), (6, "tiny", {"n_ff": 5120}), (5, "tiny_full", {"n_ff": 5120})])
def test_every_kernel_choice_gives_the_same_bits(lg, gpu_required, model_path, monkeypatch, rows, name, over):
    """The options that pick between kernels for the same arithmetic (row work inside the q/k/v matmul, the
    attention kernels that share a staged tile, the matrix-core lm_head, wide prompt blocks, graph replay, ffn_down
    cut by K quarter: the last case has the long FFN rows and no per-layer embeddings that kernel is for; the
    per-layer inputs built on a second stream beside layer 0) change
    timing only: every combination leaves the same cache rows and the same logits rows of a verify block."""
    monkeypatch.setenv("LG_HIP_MERGE_O", "1")          # (builds the second copy of attn_output that the merge_o option needs)
    monkeypatch.setenv("LG_HIP_XCD_ATTN_TAIL", "1")    # (... and the one the xcd_attn_tail option needs)
    path, spec = model_path(name, **over)
    V = spec["n_vocab"]
    rng = np.random.default_rng(rows)
    prompt = rng.integers(0, V, 300).astype(np.int32)
    blk = rng.integers(0, V, rows).astype(np.int32)

    def run(**opts):
        gpu = lg.hiplib.HipBackend(path, 400, max_rows=8)
        try:
            for k, v in opts.items():
                gpu.set_option(k, v)
            gpu.set_option("store_logits", 1)
            gpu.prefill(prompt, 0)
            adv, out = gpu.forward_spec(blk, 300)
            logits = np.stack([gpu.logits_row(j, V) for j in range(rows)])
            cache = [gpu.kv_read(L, w).copy() for L in range(spec["n_layer"] - spec["shared_kv_layers"]) for w in (0, 1)]
            return adv, out.copy(), logits, cache
        finally:
            gpu.close()

    base = run()
    assert np.isfinite(base[2]).all()                  # (a bitwise comparison would call two rows of NaN equal)
    for opt, val in (("fuse_rows", 0), ("attn_rows", 0), ("attn_rows_fq", 0), ("head_mfma", 0), ("wide_prefill", 0), ("use_graph", 0), ("down_kq", 0),
                     ("fork_ple", 1),        # (the per-layer inputs as a second branch of the graph: off by default)
                     ("xcd_tail", 0), ("xcd_tail", 2), ("xcd_tail_spread", 0), ("rows_geglu", 1),   # (the row work ahead of gate/up inside the gate/up launch: off by default; the per-layer-input block as separate kernels / as one launch also for narrow blocks)
                     ("down_m", 0), ("down_m", 2),                      # (ffn_down of 4..8-row blocks on v_dot4 instead of the matrix cores; the last two cases have the long FFN rows)
                     ("xcd_attn_tail", 0), ("xcd_attn_tail", 2),   # (attention merge + output projection + row work: separate kernels / one launch on one XCD for every width)
                     ("merge_o", 0), ("merge_o", 2), ("merge_o_slices", 8)):   # (attention merge + output projection: separate / one launch for every width / another cut of the rows)
        print(f"rows={rows} option {opt}={val}", flush=True)
        got = run(**{opt: val})
        assert got[0] == base[0] and np.array_equal(got[1], base[1]), opt
        assert np.array_equal(got[2].view(np.uint32), base[2].view(np.uint32)), opt
        for a, b in zip(got[3], base[3]):
            assert np.array_equal(a, b), opt


@pytest.mark.parametrize("rows", [5, 8, 2])
def test_shared_tile_attention_prepares_its_own_rows(lg, ob, gpu_required, model_path, rows):
    """Layers with 256 and more (tile, kv head) pairs take the attention kernel that stages a tile once for all rows
    of a block; it norms and rotates the block's queries and builds the block's K/V rows itself.  A 2048-key window
    on 4 KV heads (66 tiles) and a global context of the same length, layers that own their cache and layers that
    read another's, a block that starts 2 positions before a tile boundary (its rows fall into two tiles) and the
    next one after it: against the oracle, and bit for bit against the same step with lg_k_qkv_post run ahead
    (attn_rows_fq = 0) and with the per-row attention kernel (attn_rows = 0)."""
    path, spec = model_path("tiny_full", n_head_kv=4, sliding_window=2048)
    V, E = spec["n_vocab"], spec["n_embd"]
    rng = np.random.default_rng(90 + rows)
    n0 = 65 * 32 + 30
    prompt = rng.integers(0, V, n0).astype(np.int32)
    first, tail = int(rng.integers(0, V)), rng.integers(0, V, rows).astype(np.int32)
    ctx = n0 + 64

    def run(**opts):
        gpu = lg.hiplib.HipBackend(path, ctx, max_rows=8)
        try:
            for k, v in opts.items():
                gpu.set_option(k, v)
            gpu.set_option("store_logits", 1)
            gpu.prefill(prompt, 0)
            chain = [first]                                # the model's own continuation: a block that is accepted whole
            for i in range(rows):
                chain.append(gpu.forward_next(chain[-1], n0 + i))
            blocks = [np.array(chain[:rows], np.int32), np.concatenate(([chain[rows]], tail[1:])).astype(np.int32)]
            res, pos = [], n0
            for blk in blocks:
                adv, out = gpu.forward_spec(blk, pos)
                res.append((adv, out.copy(), np.stack([gpu.logits_row(j, V) for j in range(rows)]), gpu.last_hidden(E).copy(), blk))
                pos += adv
            cache = [gpu.kv_read(L, w).copy() for L in range(spec["n_layer"] - spec["shared_kv_layers"]) for w in (0, 1)]
            return res, cache
        finally:
            gpu.close()

    print(f"rows={rows}: default kernels", flush=True)
    base, base_cache = run()
    assert all(np.isfinite(r[2]).all() for r in base)
    assert base[0][0] == rows                              # verify == plain decode
    o = ob.Oracle(path)
    try:
        kv = o.kv_new(ctx, ob.I8)
        o.prefill(kv, prompt, 0, ob.I8)
        pos = n0
        for adv, out, _, hid, blk in base:
            oadv, oout, ohid = o.forward_spec(kv, blk, pos, ob.I8, want_hidden=True)
            assert oadv == adv and oout[:adv].tolist() == out[:adv].tolist()
            assert np.array_equal(hid.view(np.uint32), ohid.view(np.uint32))
            pos += adv
    finally:
        o.close()
    for opts in ({"attn_rows_fq": 0}, {"attn_rows": 0}):
        print(f"rows={rows}: {opts}", flush=True)
        got, cache = run(**opts)
        for g, b in zip(got, base):
            assert g[0] == b[0] and np.array_equal(g[1], b[1]), opts
            assert np.array_equal(g[2].view(np.uint32), b[2].view(np.uint32)), opts
        for a, b in zip(cache, base_cache):
            assert np.array_equal(a, b), opts
