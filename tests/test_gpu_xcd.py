"""GPU parity of the XCD-partitioned feed-forward kernel (one launch for row work, gate/up + GeGLU and ffn_down, the
8 XCDs each taking an eighth of the FFN columns) against the oracle's composition of the same steps, bit for bit,
and the placement of workgroups it relies on."""
import numpy as np
import pytest

from conftest import random_q4_0
from test_gpu_kernels import oracle_matmul

pytestmark = pytest.mark.gpu


def test_workgroups_are_dealt_to_the_xcds_in_turn(lg, gpu_required):
    """The workgroups i of a launch with the same i % 8 run on one XCD: what the XCD-partitioned kernel relies on."""
    import ctypes as C
    H = lg.hiplib.load_hip()
    i32a = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
    H.lg_hip_xcd_map.argtypes = [C.c_int] * 4 + [i32a, i32a]
    xcc = np.zeros((3, 256), np.int32); hw = np.zeros((3, 256), np.int32)
    print("xcd map 256 x 512", flush=True)
    lg.hiplib.hip_check(H.lg_hip_xcd_map(256, 512, 64 * 1024, 3, xcc, hw), "xcd_map")
    # consecutive workgroups on consecutive XCDs; where a launch starts depends on what ran before it
    for launch in xcc:
        assert np.array_equal((launch - launch[0]) % 8, np.arange(256) % 8)


def oracle_ffn(ob, x, dout, w_post, w_pre, wg, wu, wd, FF, eps):
    L = ob.lib()
    rows, E = x.shape
    xn = np.zeros_like(x); h = np.zeros_like(x)
    for j in range(rows):
        o = np.zeros(E, np.float32)
        L.lgo_rmsnorm(o, np.ascontiguousarray(dout[j]), w_post.ctypes.data, E, eps, 1)
        xn[j] = x[j] + o
        L.lgo_rmsnorm(h[j], np.ascontiguousarray(xn[j]), w_pre.ctypes.data, E, eps, 1)
    _, _, _, gate, _ = oracle_matmul(ob, wg, E, FF, h)
    _, _, _, up, _ = oracle_matmul(ob, wu, E, FF, h)
    act = np.zeros((rows, FF), np.float32)
    for j in range(rows):
        act[j] = np.array([L.lgo_gelu(float(v), 1) for v in gate[j]], np.float32) * up[j]
    _, _, _, out, _ = oracle_matmul(ob, wd, FF, E, act)
    return xn, act, out


@pytest.mark.parametrize("rows,E,FF", [(4, 512, 2048), (5, 512, 2048), (8, 512, 2048), (5, 2560, 10240), (4, 2560, 10240),
                                       (8, 2560, 10240), (6, 2560, 10240), (7, 512, 2048), (5, 3840, 15360), (8, 3840, 15360)])
def test_ffn_xcd_matches_oracle(lg, ob, gpu_required, rows, E, FF):
    rng = np.random.default_rng(rows * 31 + E + FF)
    x = rng.normal(0, 1, (rows, E)).astype(np.float32)
    dout = rng.normal(0, 3, (rows, E)).astype(np.float32)
    w_post = (1 + 0.1 * rng.normal(0, 1, E)).astype(np.float32)
    w_pre = (1 + 0.1 * rng.normal(0, 1, E)).astype(np.float32)
    wg, wu, wd = random_q4_0(rng, FF, E), random_q4_0(rng, FF, E), random_q4_0(rng, E, FF)
    x[0, :64] = 0.0
    dout[0, :64] = 0.0
    print(f"ffn_xcd rows={rows} E={E} FF={FF}", flush=True)
    r = lg.hiplib.ffn_xcd(x, dout, w_post, w_pre, wg, wu, wd, FF, eps=1e-6, repeats=3)
    xn, act, out = oracle_ffn(ob, x, dout, w_post, w_pre, wg, wu, wd, FF, 1e-6)
    assert np.array_equal(r["x_out"].view(np.uint32), xn.view(np.uint32)), "residual"
    assert np.array_equal(r["act"].view(np.uint32), act.view(np.uint32)), "gelu(gate) * up"
    assert np.array_equal(r["out"].view(np.uint32), out.view(np.uint32)), "ffn_down"
    print(f"  kernel {1e3 * r['kernel_ms']:.2f} us", flush=True)



@pytest.mark.parametrize("name,rows", [("tiny", 4), ("tiny", 5), ("tiny_full", 5), ("tiny_full", 8)])
def test_verify_steps_with_the_xcd_ffn_kernel_match_the_oracle(lg, ob, gpu_required, model_path, monkeypatch, name, rows):
    """Whole verify steps with the feed-forward half running as the one XCD-partitioned launch (asked for at
    commit with LG_HIP_XCD_FFN=1): accept counts, successors, every row's logits and the kept hidden state are the
    oracle's, bit for bit, and the same as with the option switched off again."""
    monkeypatch.setenv("LG_HIP_XCD_FFN", "1")
    path, spec = model_path(name)
    V = spec["n_vocab"]
    rng = np.random.default_rng(rows + 40)
    prompt = rng.integers(0, V, 150).astype(np.int32)
    o = ob.Oracle(path)
    gpu = lg.hiplib.HipBackend(path, 400, max_rows=8)
    try:
        gpu.set_option("xcd_ffn", 1)
        gpu.prefill(prompt[:-1], 0)
        gpu.set_option("store_logits", 1)
        okv = o.kv_new(400, ob.I8)
        o.prefill(okv, prompt[:-1], 0, ob.I8)
        lg.hiplib.hip_check(gpu.H.lg_hip_kv_save_prefix(gpu.dkv, 149), "save")
        pos = 149
        tok = int(prompt[-1])
        for step in range(4):
            blk = np.array([tok] + rng.integers(0, V, rows - 1).tolist(), np.int32)     # random drafts: rows run whatever is accepted
            print(f"xcd ffn {name} rows={rows} step={step} pos={pos}", flush=True)
            adv, out = gpu.forward_spec(blk, pos)
            hid = gpu.last_hidden(spec["n_embd"])
            logits = np.stack([gpu.logits_row(j, V) for j in range(rows)])
            oadv, oout, ohid = o.forward_spec_all(okv, blk, pos, ob.I8, want_hidden=True)
            assert adv == oadv and out[:adv].tolist() == oout[:adv].tolist()
            assert np.array_equal(hid.view(np.uint32), ohid.view(np.uint32))
            if step == 0:       # the same block with the separate kernels: every row's logits and successor agree bit for bit
                lg.hiplib.hip_check(gpu.H.lg_hip_kv_restore_prefix(gpu.dkv, 149), "restore")
                gpu.set_option("xcd_ffn", 0)
                adv0, out0 = gpu.forward_spec(blk, pos)
                logits0 = np.stack([gpu.logits_row(j, V) for j in range(rows)])
                assert adv0 == adv and np.array_equal(out0, out)
                assert np.array_equal(logits0.view(np.uint32), logits.view(np.uint32))
                gpu.set_option("xcd_ffn", 1)
            pos += adv; tok = int(out[adv - 1])
    finally:
        gpu.close(); o.close()


@pytest.mark.parametrize("name", ["tiny_full"])
@pytest.mark.parametrize("rows,spread", [(1, 1), (2, 1), (3, 1), (4, 1), (5, 1), (6, 1), (7, 1), (8, 1), (5, 0), (6, 0), (8, 0), (3, 2), (4, 2)])
def test_verify_steps_with_the_one_xcd_tail_match_the_oracle(lg, ob, gpu_required, model_path, name, rows, spread):
    """Whole verify steps with the per-layer-input block and the following row work as one launch on one XCD
    (lg_k_ple_tail, option xcd_tail = 2: for every block width, also the ones that otherwise fold the row work into
    the q/k/v matmul; at 1, 2 and 5..8 rows lg_k_ple_tail_s, units of 8 wavefronts that fit one per CU, unless xcd_tail_spread = 0; at 3 and 4 rows too with xcd_tail_spread = 2): accept counts, successors, every row's logits and the kept hidden state are the oracle's, bit
    for bit, over several steps (each step is one launch per layer: the hand-over flags of a launch start from what the
    launch before left), and the same as with the separate kernels."""
    path, spec = model_path(name)
    V = spec["n_vocab"]
    rng = np.random.default_rng(rows + 80)
    prompt = rng.integers(0, V, 150).astype(np.int32)
    o = ob.Oracle(path)
    gpu = lg.hiplib.HipBackend(path, 400, max_rows=8)
    try:
        gpu.set_option("xcd_tail", 2)
        gpu.set_option("xcd_tail_spread", spread)
        gpu.prefill(prompt[:-1], 0)
        gpu.set_option("store_logits", 1)
        okv = o.kv_new(400, ob.I8)
        o.prefill(okv, prompt[:-1], 0, ob.I8)
        lg.hiplib.hip_check(gpu.H.lg_hip_kv_save_prefix(gpu.dkv, 149), "save")
        pos = 149
        tok = int(prompt[-1])
        for step in range(5):
            blk = np.array([tok] + rng.integers(0, V, rows - 1).tolist(), np.int32)
            print(f"xcd tail {name} rows={rows} step={step} pos={pos}", flush=True)
            adv, out = gpu.forward_spec(blk, pos)
            hid = gpu.last_hidden(spec["n_embd"])
            logits = np.stack([gpu.logits_row(j, V) for j in range(rows)])
            oadv, oout, ohid = o.forward_spec_all(okv, blk, pos, ob.I8, want_hidden=True)
            assert adv == oadv and out[:adv].tolist() == oout[:adv].tolist()
            assert np.array_equal(hid.view(np.uint32), ohid.view(np.uint32))
            if step == 0:
                lg.hiplib.hip_check(gpu.H.lg_hip_kv_restore_prefix(gpu.dkv, 149), "restore")
                gpu.set_option("xcd_tail", 0)
                adv0, out0 = gpu.forward_spec(blk, pos)
                logits0 = np.stack([gpu.logits_row(j, V) for j in range(rows)])
                assert adv0 == adv and np.array_equal(out0, out)
                assert np.array_equal(logits0.view(np.uint32), logits.view(np.uint32))
                gpu.set_option("xcd_tail", 2)
            pos += adv; tok = int(out[adv - 1])
    finally:
        gpu.close(); o.close()


@pytest.mark.parametrize("name", ["tiny", "tiny_full"])
@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 6, 7, 8])
def test_verify_steps_with_the_one_xcd_attention_tail_match_the_oracle(lg, ob, gpu_required, model_path, monkeypatch, name, rows):
    """Whole verify steps with attention merge, output projection (on the matrix cores) and the row work after it as
    one launch on one XCD (lg_k_attn_tail, option xcd_attn_tail = 2: every block width): accept counts, successors,
    every row's logits and the kept hidden state are the oracle's, bit for bit, over several steps, and the same as
    with the separate kernels.  tiny has 64-wide heads everywhere, tiny_full 128-wide ones in its global layers (two
    chain lengths), sliding windows that start inside the cache and per-layer inputs (so both one-XCD launches run)."""
    monkeypatch.setenv("LG_HIP_XCD_ATTN_TAIL", "2")     # (builds the copy of attn_output that the kernel reads)
    path, spec = model_path(name)
    V = spec["n_vocab"]
    rng = np.random.default_rng(rows + 160)
    prompt = rng.integers(0, V, 150).astype(np.int32)
    o = ob.Oracle(path)
    gpu = lg.hiplib.HipBackend(path, 400, max_rows=8)
    try:
        gpu.set_option("xcd_attn_tail", 2)
        gpu.prefill(prompt[:-1], 0)
        gpu.set_option("store_logits", 1)
        okv = o.kv_new(400, ob.I8)
        o.prefill(okv, prompt[:-1], 0, ob.I8)
        lg.hiplib.hip_check(gpu.H.lg_hip_kv_save_prefix(gpu.dkv, 149), "save")
        pos = 149
        tok = int(prompt[-1])
        for step in range(5):
            blk = np.array([tok] + rng.integers(0, V, rows - 1).tolist(), np.int32)
            print(f"xcd attention tail {name} rows={rows} step={step} pos={pos}", flush=True)
            adv, out = gpu.forward_spec(blk, pos)
            hid = gpu.last_hidden(spec["n_embd"])
            logits = np.stack([gpu.logits_row(j, V) for j in range(rows)])
            oadv, oout, ohid = o.forward_spec_all(okv, blk, pos, ob.I8, want_hidden=True)
            assert adv == oadv and out[:adv].tolist() == oout[:adv].tolist()
            assert np.array_equal(hid.view(np.uint32), ohid.view(np.uint32))
            if step == 0:
                lg.hiplib.hip_check(gpu.H.lg_hip_kv_restore_prefix(gpu.dkv, 149), "restore")
                gpu.set_option("xcd_attn_tail", 0)
                adv0, out0 = gpu.forward_spec(blk, pos)
                logits0 = np.stack([gpu.logits_row(j, V) for j in range(rows)])
                assert adv0 == adv and np.array_equal(out0, out)
                assert np.array_equal(logits0.view(np.uint32), logits.view(np.uint32))
                gpu.set_option("xcd_attn_tail", 2)
            pos += adv; tok = int(out[adv - 1])
    finally:
        gpu.close(); o.close()


@pytest.mark.parametrize("rows,E,FF", [(4, 512, 5120), (6, 512, 5120), (5, 2560, 10240), (8, 2560, 10240), (4, 2560, 10240), (5, 3840, 15360), (7, 3840, 15360)])
def test_down_m_matches_oracle(lg, ob, gpu_required, rows, E, FF):
    """ffn_down of a verify block on the matrix cores (lg_k_down_m: 64 row groups x 4 K quarters, one K segment per
    wavefront, four slabs) against the oracle's q4_0 x q8 matmul of the same rows: 8, 40 and 60 output rows per
    workgroup (one operand, 32 + 8, 32 + 28), segments of 5, 10 and 15 blocks (odd counts are padded)."""
    rng = np.random.default_rng(rows * 17 + E + FF)
    act = (rng.normal(0, 1, (rows, FF)) * rng.uniform(0.2, 3.0, (rows, 1))).astype(np.float32)
    act[0, :96] = 0.0
    w = random_q4_0(rng, E, FF)
    print(f"down_m rows={rows} E={E} FF={FF}", flush=True)
    _, _, _, want, _ = oracle_matmul(ob, w, FF, E, act)
    for join in (1, 0):       # the row group's workgroups add their slabs themselves (several launches in a row: the flags go on from launch to launch) / the caller does
        got, ms = lg.hiplib.down_m(act, w, E, repeats=3, join=join)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), join
        print(f"  join={join}: kernel {1e3 * ms:.2f} us", flush=True)
