#!/usr/bin/env python3
"""Benchmark of the MTP speculative-verify step on one MI355X.

A "step" is one verify step: a block of M = K+1 rows (the chosen token and K drafts) through the
whole E4B-shaped q4_0 decoder, lm_head, argmax and the accept rule, all on the device, with the
position and the token schedule device-resident (no host round trip between steps).  Weights and
the 2048-position KV cache are in HBM before the timed region.  The drafts are the model's own
greedy continuation with the first mismatch drawn from a seeded Geometric(0.6), so the number of
accepted tokens per step is known in advance and is checked.

Prints one JSON line: verified tokens/s, the roofline figure of the dominant kernel (measured with
device events on the library's stream), the whole-step HBM figure, and the CPU baseline (the
reference's own CPU backend when its build is present, else this repository's restatement).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
lg = importlib.import_module("little-gemma_amd")

HBM_PEAK_GBS = 8000.0
FLOOR_LAUNCH_US = 1.55          # a dependent kernel boundary inside a captured graph on this part (bench.py --launch-floor)
FLOOR_STREAM_GBS = 6000.0       # what a plain streaming kernel sustains from HBM here
i32a = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
# HBM bytes per launch of the dominant kernel (gate/up + GeGLU at the E4B shape), from the FETCH_SIZE and
# WRITE_SIZE counter runs summarised in the file named below (scaled by the copy-kernel calibration given
# there): reads 29.40 MB for M = 5 (29.27 MB for M = 1), writes 0.15 MB (0.03 MB).  Counters cannot be read
# from inside this process, so the figure is quoted with its source; shapes without a counter run report null.
MEASURED_TRAFFIC = {("e4b", "gate_up_geglu", 5): 29.41e6 + 0.07e6, ("e4b", "gate_up_geglu", 1): 29.27e6 + 0.03e6}
TRAFFIC_SOURCE = "profiles/verify_step_e4b_rows5_hbm_counters.md"
CTX = 2048
WORKLOADS = {
    "e4b": ("E4B-shape q4_0 verify step (42 layers, d 2560, 8/2 heads x 256, FFN 10240, PLE 256, vocab 262144, "
            "5 sliding-512 : 1 global), ctx 2048", lg.synth.E4B),
    "g12b": ("12B-shape q4_0 verify step (48 layers, d 3840, 16/8 heads x 256, FFN 15360, no PLE, vocab 262144, "
             "5 sliding-1024 : 1 global), ctx 8192", lg.synth.G12B),
    "tiny": ("tiny 4-layer shape (plumbing check only: fits in cache, no bandwidth claim)", lg.synth.TINY),
}
WORKLOAD_CTX = {"e4b": CTX, "g12b": 8192, "tiny": 256}


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


def seed_cache(gpu, info, layers, ctx, seed):
    """Fill every owning layer with f16 values shaped like real rows: K ~ N(0, q/k-norm weight),
    V ~ unit RMS.  Returns {layer: (K, V)} as uint16 arrays indexed by ring row."""
    rng = np.random.default_rng(seed)
    filled = {}
    for L in range(info["n_layer"]):
        rows, width = gpu.kv_layout(L)
        if rows == 0:
            continue
        hd = layers[L]["head_dim"]
        kstd = np.sqrt(1.28 / np.sqrt(hd))
        n = min(rows, ctx)
        K = np.zeros((rows, width), np.float16)
        V = np.zeros((rows, width), np.float16)
        K[:n] = (rng.standard_normal((n, width), np.float32) * kstd).astype(np.float16)
        V[:n] = rng.standard_normal((n, width), np.float32).astype(np.float16)
        # (a ring of fewer rows than ctx: row r stands for the latest position p < ctx with p % rows == r; any filled row will do)
        gpu.kv_write(L, 0, K.view(np.uint16))
        gpu.kv_write(L, 1, V.view(np.uint16))
        filled[L] = (K, V)
    return filled


def build_schedule(greedy, first_tok, rows, n_steps, n_vocab, seed, p=0.6):
    """Blocks [chosen, d1..dK] along the greedy sequence; first mismatch ~ Geometric(p)."""
    rng = np.random.default_rng(seed)
    seq = [first_tok] + list(greedy)          # seq[i] = token at position pos0 + i
    blocks, advs, at = [], [], 0
    for _ in range(n_steps):
        first_bad = int(rng.geometric(p))     # 1-based index of the first wrong draft
        blk = [seq[at]]
        for j in range(1, rows):
            good = seq[at + j]
            blk.append(good if j < first_bad else (good + 1 + int(rng.integers(0, n_vocab - 1))) % n_vocab)
        adv = min(first_bad, rows)
        blocks.append(blk)
        advs.append(adv)
        at += adv
    return np.array(blocks, np.int32), np.array(advs, np.int32)


def cpu_baseline(path, filled, info, layers, blocks, pos0, rows, budget_s):
    from oracle import binding as ob
    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    kind = "reference" if ob.ref_available(rows) else "port"
    if kind == "reference":
        m = ob.Reference(path, rows)
        kv = m.kv_new(pos0 + len(blocks) * rows + 8)
        views = m.kv_views(kv)
    else:
        m = ob.Oracle(path)
        ob.lib().lgo_set_threads(threads)
        kv = m.kv_new(pos0 + len(blocks) * rows + 8, ob.REF)
        views = m.kv_views(kv)
    # same cache contents as the GPU (f16-representable values, so f32 sliding rings hold the same numbers)
    for L, (K, V) in views.items():
        gk, gv = filled[L]
        n_cpu = K.shape[0]
        for p_ in range(max(0, pos0 - n_cpu), pos0):
            src = p_ % gk.shape[0]
            dst = p_ % n_cpu
            if K.dtype == np.uint16:
                K[dst] = gk[src].view(np.uint16); V[dst] = gv[src].view(np.uint16)
            else:
                K[dst] = gk[src].astype(np.float32); V[dst] = gv[src].astype(np.float32)
    t0 = time.time()
    toks_done = steps = 0
    pos = pos0
    for blk in blocks:
        if kind == "reference":
            adv, _ = m.forward_spec(kv, blk, pos)
        else:
            adv, _, _ = m.forward_spec(kv, blk, pos, ob.REF)
        pos += adv
        toks_done += adv
        steps += 1
        if time.time() - t0 > budget_s:
            break
    dt = time.time() - t0
    m.kv_free(kv)
    m.close()
    return {"value": toks_done / dt, "unit": "verified tok/s", "cores": threads, "kind": kind,
            "sample": f"{steps} verify steps of the same schedule ({toks_done} tokens) on the same GGUF and cache contents, {dt:.1f} s",
            "ms_per_step": 1e3 * dt / steps}


def ref_f32_gap(model_dir):
    """The device against the committed reference fixtures (tests/golden/ref_tiny*.npz: 64 greedy tokens and four
    logit rows recorded from the reference's CPU `run` path, f32 activations): teacher-forced on those tokens,
    relative L2 of the device logits to the recorded rows and the number of steps whose argmax is the reference's
    token.  The gap is the q8 activation noise of the int8 class, not an error of the device."""
    out = {}
    for name in ("tiny", "tiny_full"):
        fx = os.path.join(ROOT, "tests", "golden", f"ref_{name}.npz")
        if not os.path.exists(fx):
            continue
        g = np.load(fx)
        path = os.path.join(model_dir, f"lg_bench_{name}.gguf")
        spec = lg.synth.write_model(path, **getattr(lg.synth, name.upper()))
        prompt, toks = g["prompt"], g["tokens"]
        steps = {int(s): i for i, s in enumerate(g["logit_steps"])}
        gpu = lg.hiplib.HipBackend(path, len(prompt) + len(toks) + 16, max_rows=1)
        try:
            gpu.prefill(prompt[:-1], 0)
            tok, pos, gaps, agree = int(prompt[-1]), len(prompt) - 1, [], 0
            for step in range(len(toks)):
                row = gpu.forward(tok, pos, spec["n_vocab"])
                if step in steps:
                    want = g["logits"][steps[step]]
                    gaps.append(float(np.linalg.norm(row - want) / np.linalg.norm(want)))
                agree += int(np.argmax(row)) == int(toks[step])
                tok, pos = int(toks[step]), pos + 1
        finally:
            gpu.close()
        out[name] = {"logits_rel_l2_max": max(gaps), "logits_rel_l2_median": float(np.median(gaps)),
                     "argmax_equal_steps": agree, "steps": int(len(toks))}
    return out


def xcd_handover():
    """Placement of workgroups over the XCDs and the cost of a flag hand-over inside one XCD / across XCDs."""
    import ctypes as C
    H = lg.hiplib.load_hip()
    H.lg_hip_xcd_map.argtypes = [C.c_int] * 4 + [i32a, i32a]
    H.lg_hip_xcd_handover.argtypes = [C.c_int] * 7 + [i32a, C.POINTER(C.c_float)]
    placement = []
    for grid, block, lds in ((256, 256, 0), (256, 512, 96 * 1024), (320, 512, 0), (512, 256, 0), (2048, 64, 0)):
        xcc = np.zeros((4, grid), np.int32); hw = np.zeros((4, grid), np.int32)
        lg.hiplib.hip_check(H.lg_hip_xcd_map(grid, block, lds, 4, xcc, hw), "xcd_map")
        turn = bool(np.all((xcc - xcc[:, :1]) % 8 == (np.arange(grid) % 8)[None, :]))   # (the first XCD of a launch depends on what ran before)
        cu = ((hw >> 8) & 15) | (((hw >> 12) & 1) << 4) | (((hw >> 13) & 7) << 5)          # cu, sh, se fields of HW_ID
        per_cu = [int(np.unique(np.stack([xcc[l], cu[l]]), axis=1, return_counts=True)[1].max()) for l in range(4)]
        placement.append({"grid": grid, "block": block, "lds": lds, "consecutive_workgroups_on_consecutive_xcds": turn, "first_xcd_per_launch": xcc[:, 0].tolist(),
                          "xcd_of_first_16": xcc[0, :16].tolist(), "same_in_4_launches": bool(np.all(xcc == xcc[0])),
                          "per_xcd": np.bincount(xcc[0], minlength=8).tolist(), "max_workgroups_on_one_cu": per_cu})
    names = {0: "plain", 1: "sc0", 2: "sc1", 3: "sc0 sc1"}
    rows = []
    rounds = 200
    for what, set_mode, sel, n in (("one XCD (workgroups 0,8,..,248)", 0, 0, 32), ("one XCD (workgroups 3,11,..)", 0, 3, 32),
                                   ("spread (workgroups 0..31)", 1, 0, 32), ("spread (workgroups 0..7)", 1, 0, 8),
                                   ("one XCD, 8 members", 0, 0, 8)):
        for st, ld in ((0, 2), (0, 1), (2, 2), (3, 3), (0, 3), (0, 0)):
            for nbytes in (0, 1024, 16384):
                res = np.zeros((n, 4), np.int32); tick = C.c_float(0)
                lg.hiplib.hip_check(H.lg_hip_xcd_handover(set_mode, sel, n, st, ld, nbytes, rounds, res, C.byref(tick)), "xcd_handover")
                rows.append({"group": what, "members": n, "store": names[st], "load": names[ld], "bytes_per_member": nbytes,
                             "us_per_round_max": round(float(res[:, 0].max()) * tick.value / rounds / 1e3, 4),
                             "us_per_round_min": round(float(res[:, 0].min()) * tick.value / rounds / 1e3, 4),
                             "stale_words": int(res[:, 1].sum()), "polls_given_up": int(res[:, 2].sum()),
                             "xcds_seen": sorted(set(res[:, 3].tolist()))})
    print(json.dumps({"metric": "workgroup placement over XCDs and flag hand-over cost", "rounds": rounds,
                      "placement": placement, "handover": rows}), flush=True)


def tail_stamps(rows, model_dir):
    """Phase boundaries of the one-XCD layer tail (lg_k_ple_tail; lg_k_ple_tail_s from 5 rows on, where every stamp is its
    workgroup's first wavefront's) at the E4B shape: device wall-clock stamps of every
    unit of the last layer's launch, over four verify steps from a 600-position cache."""
    path = os.path.join(model_dir, f"lg_bench_e4b_seed{lg.synth.E4B['seed']}.gguf")
    if not os.path.exists(path):
        lg.synth.write_model(path + ".tmp", **lg.synth.E4B)
        os.replace(path + ".tmp", path)
    gpu = lg.hiplib.HipBackend(path, 2400, max_rows=8)
    gpu.set_option("xcd_tail_stamps", 1)
    rng = np.random.default_rng(1)
    gpu.prefill(rng.integers(1, 262144, 600).astype(np.int32), 0)
    pos, steps = 600, []
    names = ["start", "rows + per-layer gate done", "hand-over 1 done", "gated rows copied", "projection done", "hand-over 2 done",
             "projected row loaded", "row work done"]
    for _ in range(4):
        adv, _ = gpu.forward_spec(rng.integers(1, 262144, rows).astype(np.int32), pos)
        pos += adv
        st = gpu.tail_stamps().astype(np.int64)
        s = st[st[:, 0] >= st[:, 0].max() - 1000]          # the units of the latest launch (older launches of other widths left theirs: > 10 us back)
        rel = (s - s[:, 0].min()) * 10                     # ns (100 MHz clock)
        seen = s >= s[:, :1]                               # (a unit that leaves after the projection keeps older stamps in its last slots)
        steps.append({n: {"first_unit_ns": int(rel[:, i][seen[:, i]].min()), "last_unit_ns": int(rel[:, i][seen[:, i]].max())}
                      for i, n in enumerate(names)})
        units = int(s.shape[0])
    gpu.close()
    print(json.dumps({"metric": "phase boundaries of lg_k_ple_tail, ns since the first unit's start", "rows": rows, "units": units,
                      "steps": steps}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rows", type=int, default=5, help="verify rows M = K drafts + 1")
    ap.add_argument("--workload", default="e4b", choices=sorted(WORKLOADS))
    ap.add_argument("--ctx", type=int, default=0, help="positions already in the cache (0: the workload's own: 2048 for e4b, 8192 for g12b)")
    ap.add_argument("--model-dir", default=os.environ.get("LG_BENCH_DIR", "/tmp"))
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--seed", type=int, default=7)
    ap.add_argument("--prefill", type=int, default=1024, help="positions of the prompt-processing measurement; 0 skips it")
    ap.add_argument("--mtp-steps", type=int, default=24, help="steps of the draft-head loop measurement (4 chained device drafts + verify); 0 skips it")
    ap.add_argument("--launch-floor", action="store_true",
                    help="measure only what a captured chain of dependent kernels costs (empty, and with a 64-byte hand-over) and exit")
    ap.add_argument("--xcd-handover", action="store_true",
                    help="measure only where workgroups run (XCD of every workgroup) and what a flag hand-over among the "
                         "workgroups of one XCD costs next to one spread over all XCDs, and exit")
    ap.add_argument("--tail-stamps", action="store_true",
                    help="print the phase boundaries of the one-XCD layer tail at --rows rows instead of the benchmark line")
    a = ap.parse_args()
    if a.tail_stamps:
        tail_stamps(a.rows, a.model_dir)
        return
    if a.xcd_handover:
        xcd_handover()
        return
    if a.launch_floor:
        import ctypes as C
        H = lg.hiplib.load_hip()
        H.lg_hip_launch_floor.argtypes = [C.c_int] * 5 + [C.POINTER(C.c_float)]
        rows = []
        for n in (426, 300):
            for mode, what in ((0, "empty"), (1, "64-byte load+store hand-over")):
                for grid, block in ((1, 64), (256, 256)):
                    us = C.c_float(0)
                    lg.hiplib.hip_check(H.lg_hip_launch_floor(n, mode, grid, block, 30, C.byref(us)), "launch_floor")
                    rows.append({"kernels_per_graph": n, "kernel": what, "grid": grid, "block": block,
                                 "us_per_kernel": round(us.value, 4), "ms_per_graph": round(us.value * n / 1e3, 4)})
        print(json.dumps({"metric": "launch floor of a captured chain of dependent kernels", "unit": "us per kernel", "rows": rows}), flush=True)
        return
    if a.gpus != 1:
        print("bench.py: this build measures one GPU; the verify step is not sharded (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    rank = int(os.environ.get("RANK", "0"))
    if rank != 0:
        return
    desc, spec = WORKLOADS[a.workload]
    ctx = a.ctx if a.ctx > 0 else WORKLOAD_CTX[a.workload]
    if ctx != WORKLOAD_CTX[a.workload]:
        desc = desc.rsplit(", ctx ", 1)[0] + f", ctx {ctx}"
    path = os.path.join(a.model_dir, f"lg_bench_{a.workload}_seed{spec['seed']}.gguf")
    if not os.path.exists(path):
        t0 = time.time()
        lg.synth.write_model(path + ".tmp", **spec)
        os.replace(path + ".tmp", path)
        log(f"wrote {path} in {time.time() - t0:.1f}s")
    total = a.steps + a.warmup
    max_seq = max(ctx + (total + 2) * a.rows + 64, a.prefill + 64, ctx + (a.mtp_steps + 4) * a.rows + 64)
    t0 = time.time()
    gpu = lg.hiplib.HipBackend(path, max_seq, max_rows=max(a.rows, 1))
    log(f"weights on the device in {time.time() - t0:.1f}s")

    info, layers = gpu.info, gpu.layers
    filled = seed_cache(gpu, info, layers, ctx, a.seed)
    H = gpu.H
    lg.hiplib.hip_check(H.lg_hip_kv_save_prefix(gpu.dkv, ctx), "kv_save_prefix")

    # the model's own greedy continuation from the seeded cache (plain one-row decode)
    first_tok = 1 + a.seed % (info["n_vocab"] - 1)
    need = total * a.rows + a.rows + 1
    t0 = time.time()
    greedy, tok, pos = [], first_tok, ctx
    for _ in range(need):
        tok = gpu.forward_next(tok, pos)
        greedy.append(tok)
        pos += 1
    decode_ms = 1e3 * (time.time() - t0) / need
    log(f"plain decode: {need} tokens, {decode_ms:.3f} ms/token (host-synchronised)")
    blocks, expect_adv = build_schedule(greedy, first_tok, a.rows, total, info["n_vocab"], a.seed)

    # timed region: warm-up steps, then exactly --steps steps, device events on the library's stream
    lg.hiplib.hip_check(H.lg_hip_kv_restore_prefix(gpu.dkv, ctx), "kv_restore_prefix")
    gpu.schedule(blocks, ctx)
    if a.warmup:
        gpu.schedule_time(a.warmup)
    wall0 = time.time()
    ms = gpu.schedule_time(a.steps)
    wall = time.time() - wall0
    out, adv, final_pos = gpu.schedule_wait()
    ok_adv = bool(np.array_equal(adv, expect_adv))
    # greedy successors must reproduce the plain-decode sequence wherever they are valid
    seq = [first_tok] + greedy

    def successors_follow_plain_decode(out, adv):
        at, ok = 0, True
        for s in range(len(adv)):
            for j in range(int(adv[s])):
                ok &= int(out[s, j]) == seq[at + j + 1]
            at += int(adv[s])
        return bool(ok)
    ok_tok = successors_follow_plain_decode(out, adv)
    timed_tokens = int(adv[a.warmup:].sum())
    value = timed_tokens / (ms * 1e-3)

    # per-kernel-class device time of one step (un-captured, start/stop events filled in by each launch)
    prof = gpu.profile_step(blocks[0], ctx, repeats=10)
    step_bytes = sum(c["bytes"] for c in prof)
    # the roofline kernel: the class that moves the most bytes per step (gate/up + GeGLU: 47% of them at the E4B
    # shape).  By device time several classes of a layer are within 10% of it (kernel_classes lists them all).
    dom = max((c for c in prof if c["bytes"] > 0 and c["launches"] > 1), key=lambda c: c["bytes"])
    dom_gbs = dom["bytes"] / (dom["ms"] * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": dom["name"], "achieved": dom_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": dom_gbs / HBM_PEAK_GBS,
                "traffic": MEASURED_TRAFFIC.get((a.workload, dom["name"], a.rows)),
                "traffic_source": TRAFFIC_SOURCE if (a.workload, dom["name"], a.rows) in MEASURED_TRAFFIC else None,
                "timing": "HIP start/stop events filled in by each launch itself (hipExtLaunchKernelGGL on the library's "
                          "stream, un-captured): the kernel's own begin-to-end time, what the rocprofv3 kernel trace under "
                          "profiles/ reports for the same kernel",
                "bytes_per_launch": dom["bytes"] / max(dom["launches"], 1), "ms_per_launch": dom["ms"] / max(dom["launches"], 1),
                "launches_per_step": dom["launches"]}
    step_gbs = step_bytes / (ms / a.steps * 1e-3) / 1e9
    # what a class cannot go below as long as it keeps its launches: a kernel boundary per launch plus its bytes at the
    # rate a streaming kernel reaches on this part; the ratio says how much of a class's time is neither of the two
    for c in prof:
        c["floor_us"] = c["launches"] * FLOOR_LAUNCH_US + c["bytes"] / (FLOOR_STREAM_GBS * 1e9) * 1e6
        c["over_floor"] = (c["ms"] * 1e3 / c["floor_us"]) if c["floor_us"] > 0 else None
    floor_ms = sum(c["floor_us"] for c in prof) * 1e-3
    uncaptured_ms = sum(c["ms"] for c in prof)
    # matrix-core utilisation of the verify step's one MFMA GEMM (gate/up for blocks of 4..8 rows): the weights of a
    # launch (bytes / 0.5625 elements) times the block's rows are the useful MACs, the 8 row slots of the tiles the
    # issued ones.  It is a bandwidth-bound kernel: the figure says how far the matrix cores are from mattering.
    mfma = None
    gu = next((c for c in prof if c["name"] == "gate_up_geglu" and c["launches"] > 0), None)
    if gu and 4 <= a.rows <= 8:
        w_elems = gu["bytes"] / gu["launches"] / (18.0 / 32.0)
        sec = gu["ms"] / gu["launches"] * 1e-3
        mfma = {"kernel": "gate_up_geglu (v_mfma_i32_32x32x32_i8, activations as the 8-row operand)",
                "useful_int8_TOPs": 2.0 * w_elems * a.rows / sec / 1e12, "issued_int8_TOPs": 2.0 * w_elems * 8 / sec / 1e12,
                "mfma_peak_TOPs": 5000.0, "mfma_utilisation": 2.0 * w_elems * a.rows / sec / 5.0e15}
    line = {
        "metric": ("verified tok/s (E4B-shape q4_0, block-4, ctx 2048) + achieved HBM GB/s vs peak" if a.workload == "e4b" and ctx == CTX else
                   f"verified tok/s ({a.workload} shape q4_0, {a.rows} rows, ctx {ctx}) + achieved HBM GB/s vs peak"),
        "value": value, "unit": "verified tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms / a.steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 x int4 -> int32 block dots, f32 accumulate", "data": "synthetic",
        "config": {"workload": desc, "verify_rows": a.rows, "drafts": a.rows - 1, "ctx": ctx,
                   "mean_accepted_per_step": float(adv[a.warmup:].mean()), "first_mismatch": "Geometric(0.6), seeded"},
        "roofline": roofline,
        "step_hbm": {"bytes_per_step": step_bytes, "achieved": step_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": step_gbs / HBM_PEAK_GBS},
        "floor": {"launch_us": FLOOR_LAUNCH_US, "stream_GBs": FLOOR_STREAM_GBS, "step_floor_ms": floor_ms,
                  "ms_per_step_over_floor": (ms / a.steps) / floor_ms,
                  "launches_per_step": int(sum(c["launches"] for c in prof)),
                  "uncaptured_class_sum_ms": uncaptured_ms, "uncaptured_over_graph_step": uncaptured_ms / (ms / a.steps),
                  "note": "kernel_classes are timed un-captured, kernel begin to end; in the captured step the launch gaps "
                          "overlap the tails of the kernels before them, so the class durations (each also carrying its event pair) add up to more than "
                          "ms_per_step"},
        "verify_mfma": mfma,
        "kernel_classes": [{k: (round(v, 5) if isinstance(v, float) else v) for k, v in c.items()} for c in prof],
        "checks": {"accept_counts_as_scheduled": ok_adv, "tokens_equal_plain_decode": ok_tok, "final_pos": final_pos,
                   "wall_ms_per_step": 1e3 * wall / a.steps, "plain_decode_ms_per_token_host_sync": decode_ms},
    }
    # the same model and cache at the reference's "block-4" width (LG_MTP_N = 4: the chosen token + 3 drafts,
    # include/model.h:179-183) when the headline ran at another width: same greedy chain, same draft model
    if a.rows > 4 and a.workload == "e4b":             # (narrower runs hold neither the greedy chain nor the rows for it)
        blocks4, expect4 = build_schedule(greedy, first_tok, 4, total, info["n_vocab"], a.seed)
        lg.hiplib.hip_check(H.lg_hip_kv_restore_prefix(gpu.dkv, ctx), "kv_restore_prefix")
        gpu.schedule(blocks4, ctx)
        if a.warmup:
            gpu.schedule_time(a.warmup)
        ms4 = gpu.schedule_time(a.steps)
        out4, adv4, _ = gpu.schedule_wait()
        ok4 = bool(np.array_equal(adv4, expect4)) and successors_follow_plain_decode(out4, adv4)
        line["block4"] = {"verify_rows": 4, "drafts": 3, "ms_per_step": ms4 / a.steps,
                          "value": int(adv4[a.warmup:].sum()) / (ms4 * 1e-3), "unit": "verified tok/s",
                          "mean_accepted_per_step": float(adv4[a.warmup:].mean()),
                          "accept_counts_as_scheduled": bool(np.array_equal(adv4, expect4)),
                          "tokens_equal_plain_decode": successors_follow_plain_decode(out4, adv4)}
        ok_tok = ok_tok and ok4
    # the loop a draft head drives (the reference's run.c with -mtp): per step K = rows-1 chained drafts on the
    # device head (synthetic gemma4-assistant weights: its drafts are rarely accepted, the step cost does not
    # depend on that), then the verify step; host clock around synchronous calls, from the seeded cache
    if a.mtp_steps > 0 and a.rows >= 2:
        apath = os.path.join(a.model_dir, f"lg_bench_{a.workload}_assistant.gguf")
        if not os.path.exists(apath):
            lg.synth.write_assistant(apath + ".tmp", **lg.synth.assistant_for(spec))
            os.replace(apath + ".tmp", apath)
        lg.hiplib.hip_check(H.lg_hip_kv_restore_prefix(gpu.dkv, ctx), "kv_restore_prefix")
        head = gpu.mtp_open(apath)
        tok, pos, t_draft, t_verify, emitted = first_tok, ctx, 0.0, 0.0, 0
        tok = gpu.forward_next(tok, pos); pos += 1               # the head reads the target's hidden state of this token
        for step in range(a.mtp_steps + 2):
            t0 = time.time()
            toks = [tok]
            for j in range(1, a.rows):
                d = gpu.mtp_draft(head, toks[-1], pos + j - 1, chain=j > 1)
                toks.append(d if d >= 0 else toks[-1])
            t1 = time.time()
            adv, out = gpu.forward_spec(np.array(toks, np.int32), pos)
            t2 = time.time()
            if step >= 2:                                        # two untimed steps: graph captures of the head and its chain
                t_draft += t1 - t0; t_verify += t2 - t1; emitted += adv
            pos += adv; tok = int(out[adv - 1])
        # the same rounds kept on the device (lg_hip_mtp_rounds: one graph per round, the host waits once at the end)
        lg.hiplib.hip_check(H.lg_hip_kv_restore_prefix(gpu.dkv, ctx), "kv_restore_prefix")
        tok = gpu.forward_next(first_tok, ctx)
        gpu.mtp_rounds(head, tok, ctx + 1, a.rows, 2)             # captures the round
        lg.hiplib.hip_check(H.lg_hip_kv_restore_prefix(gpu.dkv, ctx), "kv_restore_prefix")
        tok = gpu.forward_next(first_tok, ctx)
        t0 = time.time()
        _, _, radv, _ = gpu.mtp_rounds(head, tok, ctx + 1, a.rows, a.mtp_steps)
        t_rounds = time.time() - t0
        gpu.mtp_close(head)
        line["mtp_loop"] = {"device_rounds_ms_per_step": 1e3 * t_rounds / a.mtp_steps,
                            "device_rounds_tokens_per_step": float(radv.mean()),"steps": a.mtp_steps, "drafts_per_step": a.rows - 1,
                            "draft_ms_per_step": 1e3 * t_draft / a.mtp_steps, "verify_ms_per_step": 1e3 * t_verify / a.mtp_steps,
                            "ms_per_step": 1e3 * (t_draft + t_verify) / a.mtp_steps, "tokens_per_step": emitted / a.mtp_steps,
                            "head": "synthetic gemma4-assistant (4 blocks, 256 wide), host round trip per draft"}
    # prompt processing on the matrix cores: 32-row blocks through the int8 MFMA kernels (a fresh cache, host clock
    # around a synchronised call; the first call captures the graph and is not timed)
    if a.prefill > 0:
        prng = np.random.default_rng(a.seed + 1)
        ptoks = prng.integers(1, info["n_vocab"], a.prefill).astype(np.int32)
        gpu.new_cache(max_seq)
        gpu.prefill(ptoks[:64], 0)
        gpu.new_cache(max_seq)
        t0 = time.time()
        gpu.prefill(ptoks, 0)
        dt = time.time() - t0
        macs = sum(c["bytes"] for c in prof if c["name"] != "lm_head" and c["name"] != "attn_tiles") / (18.0 / 32.0)   # weights touched per position
        line["prefill"] = {"positions": int(a.prefill), "ms": 1e3 * dt, "tok_per_s": a.prefill / dt,
                           "kernel": "v_mfma_i32_32x32x32_i8, 512-row blocks", "int8_TOPs": 2.0 * macs * a.prefill / dt / 1e12,
                           "mfma_peak_TOPs": 5000.0, "mfma_utilisation": 2.0 * macs * a.prefill / dt / 5.0e15}
    gpu.close()
    try:
        line["checks"]["ref_f32_gap"] = ref_f32_gap(a.model_dir)
    except Exception as e:                  # reported, never allowed to break the line
        line["checks"]["ref_f32_gap"] = {"error": repr(e)}
    if a.cpu_seconds > 0:
        try:
            line["cpu_baseline"] = cpu_baseline(path, filled, info, layers, blocks, ctx, a.rows, a.cpu_seconds)
        except Exception as e:              # the baseline is reported, never allowed to break the GPU line
            line["cpu_baseline"] = {"value": None, "error": repr(e)}
    print(json.dumps(line), flush=True)
    if not (ok_adv and ok_tok):
        log("CHECK FAILED: verify output differs from plain decode / schedule")
        sys.exit(1)


if __name__ == "__main__":
    main()
