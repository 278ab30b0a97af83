"""GPU parity at the benchmark shapes (the E4B and 12B configurations of the benchmark list): a seeded 2048 / 8192-position cache,
K=4 draft blocks, the GPU against the int8-class oracle on the same GGUF and cache contents, plus the
size-independent properties (verify == decode, accept counts as planted, fully accepting run)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def seed_both(gpu, o, ob, okv, ctx, seed):
    rng = np.random.default_rng(seed)
    views = o.kv_views(okv)
    for L, (K, V) in views.items():
        rows, width = gpu.kv_layout(L)
        assert (rows, width) == K.shape
        hd = o.layers[L]["head_dim"]
        n = min(rows, ctx)
        k = np.zeros((rows, width), np.float16); v = np.zeros((rows, width), np.float16)
        k[:n] = (rng.standard_normal((n, width), np.float32) * np.sqrt(1.28 / np.sqrt(hd))).astype(np.float16)
        v[:n] = rng.standard_normal((n, width), np.float32).astype(np.float16)
        K[:] = k.view(np.uint16); V[:] = v.view(np.uint16)
        gpu.kv_write(L, 0, k.view(np.uint16)); gpu.kv_write(L, 1, v.view(np.uint16))


@pytest.mark.parametrize("name,ctx,steps,rows,opts", [("e4b", 2048, 3, 5, {}), ("g12b", 8192, 2, 5, {}),
                                                      ("e4b", 2048, 2, 4, {}), ("g12b", 8192, 2, 4, {}),    # 4 rows: the reference's "block-4" (include/model.h:179-186)
                                                      ("e4b", 2048, 2, 5, {"rows_geglu": 1}), ("g12b", 8192, 2, 5, {"rows_geglu": 1})])   # (the row work inside the gate/up launch: an option, off by default)
def test_verify_steps_at_full_shape(lg, ob, gpu_required, model_path, name, ctx, steps, rows, opts):
    path, spec = model_path(name)
    V = spec["n_vocab"]
    print(f"{name}: model written, loading", flush=True)
    o = ob.Oracle(path)
    gpu = lg.hiplib.HipBackend(path, ctx + 64, max_rows=rows)
    try:
        for k, v in opts.items():
            gpu.set_option(k, v)
        okv = o.kv_new(ctx + 64, ob.I8)
        seed_both(gpu, o, ob, okv, ctx, 11)
        lg.hiplib.hip_check(gpu.H.lg_hip_kv_save_prefix(gpu.dkv, ctx), "save")
        # plain decode on the GPU gives the greedy chain; the oracle confirms its first tokens
        tok, pos, chain = 17, ctx, [17]
        for _ in range(rows * steps + rows):
            tok = gpu.forward_next(tok, pos); chain.append(tok); pos += 1
        lg.hiplib.hip_check(gpu.H.lg_hip_kv_restore_prefix(gpu.dkv, ctx), "restore")
        gpu.set_option("store_logits", 1)
        at, pos = 0, ctx
        plan = [2, rows + 1, 1][:steps] if name == "e4b" else [rows + 1, 3][:steps]   # 12B: fully accepting, then a miss
        for step, first_bad in enumerate(plan):
            blk = np.array([chain[at + j] if j < first_bad else (chain[at + j] + 12345) % V for j in range(rows)], np.int32)
            print(f"{name} step={step} pos={pos} first_bad={first_bad}", flush=True)
            adv, out = gpu.forward_spec(blk, pos)
            assert adv == min(first_bad, rows) and out[:adv].tolist() == chain[at + 1:at + 1 + adv]
            oadv, oout, ohid = o.forward_spec(okv, blk, pos, ob.I8, want_hidden=True)     # sequential CPU forwards
            assert oadv == adv and oout[:adv].tolist() == out[:adv].tolist()
            assert np.array_equal(gpu.last_hidden(spec["n_embd"]).view(np.uint32), ohid.view(np.uint32))
            # logits of the last valid row: bit-identical, hence within the 1e-3 relative-L2 bar
            probe = o.kv_new(ctx + 64, ob.I8)
            for L, (K, Vv) in o.kv_views(okv).items():
                pk, pv = o.kv_views(probe)[L]
                pk[:] = K; pv[:] = Vv
            _, row, _ = o.forward(probe, int(blk[adv - 1]), pos + adv - 1, ob.I8)
            o.kv_free(probe)
            got = gpu.logits_row(adv - 1, V)
            assert np.linalg.norm(got - row) <= 1e-3 * np.linalg.norm(row)
            assert np.array_equal(got.view(np.uint32), row.view(np.uint32))
            at += adv; pos += adv
    finally:
        gpu.close(); o.close()
