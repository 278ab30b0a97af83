"""GPU parity of the wide (32-row) blocks that prefill runs on the matrix cores
(v_mfma_i32_32x32x32_i8): the isolated matmul with 32 activation rows against the oracle
(int32 block dots bit-exact, f32 bit-identical in this build's order), and whole prompts whose
cache rows and next-token logits must equal the position-by-position oracle."""
import numpy as np
import pytest

from conftest import q4_0_codes, random_q4_0
from test_gpu_kernels import oracle_matmul

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,k", [(10240, 2560), (2560, 10240), (256, 2560), (2560, 256), (512, 5120), (3072, 512)])
def test_wide_matmul_matches_oracle(lg, ob, gpu_required, m, k):
    """32 rows at once: both K segmentations (8 and 32), one-step rows (k = 256) and the FFN shapes."""
    rng = np.random.default_rng(m * 7 + k)
    w = random_q4_0(rng, m, k)
    x = rng.normal(0, 1, (32, k)).astype(np.float32)
    x[3, :96] = 0.0
    print(f"wide matmul m={m} k={k}", flush=True)
    r = lg.hiplib.matmul_q4q8(w, k, m, x, want_dots=True)
    xq, xd, xs, out, dots = oracle_matmul(ob, w, k, m, x)
    assert np.array_equal(r["xq"], xq) and np.array_equal(r["xsum"], xs)
    dw, codes = q4_0_codes(w, m, k)
    want_dots = np.einsum("ibe,jbe->jib", codes - 8, xq.reshape(32, k // 32, 32).astype(np.int32))
    assert np.array_equal(r["dots"], want_dots) and np.array_equal(r["dots"], dots)
    assert np.array_equal(r["out"].view(np.uint32), out.view(np.uint32))


@pytest.mark.parametrize("name,n_prompt", [("tiny", 97), ("tiny_full", 200), ("tiny", 32), ("tiny_full", 427), ("tiny", 128), ("tiny_full_f32", 200), ("tiny_full_f16", 171),
                                           ("tiny", 1100), ("tiny_full", 1061)])
def test_wide_prefill_leaves_the_same_cache_and_logits(lg, ob, gpu_required, model_path, name, n_prompt):
    """A prompt through 512-row blocks (caches of 1024 positions and more; the two long prompts also wrap the
    640-row sliding rings), 128-row blocks, 32-row blocks and a verify-width tail against one oracle forward per position:
    every cache row identical, the logits of the next position identical; and identical to the same
    prompt pushed through 8-row blocks only."""
    path, spec = model_path(name)
    check_wide_prefill(lg, ob, path, spec, name, n_prompt)


def test_wide_prefill_with_an_attention_output_of_32_segments(lg, ob, gpu_required, model_path):
    """n_head * head_dim = 5120 > 4096: the attention output projection of a wide block is cut into four K quarters
    whose slabs the next row kernel adds (as ffn_down's are at the larger shapes)."""
    path, spec = model_path("tiny", n_head=80, n_head_kv=10)
    check_wide_prefill(lg, ob, path, spec, "tiny with 80 heads", 200)


def check_wide_prefill(lg, ob, path, spec, name, n_prompt):
    rng = np.random.default_rng(n_prompt)
    prompt = rng.integers(1, spec["n_vocab"], n_prompt).astype(np.int32)
    o = ob.Oracle(path)
    gpu = lg.hiplib.HipBackend(path, n_prompt + 40, max_rows=8)
    try:
        kv = o.kv_new(n_prompt + 40, ob.I8)
        o.prefill(kv, prompt, 0, ob.I8)
        print(f"{name}: prefill of {n_prompt} positions in wide blocks", flush=True)
        gpu.prefill(prompt, 0)
        views = o.kv_views(kv)
        for L, (K, V) in views.items():
            assert np.array_equal(gpu.kv_read(L, 0), K) and np.array_equal(gpu.kv_read(L, 1), V), f"cache of layer {L}"
        want = o.forward(kv, 5, n_prompt, ob.I8)[1]
        got = gpu.forward(5, n_prompt, spec["n_vocab"])
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        wide = {L: (gpu.kv_read(L, 0).copy(), gpu.kv_read(L, 1).copy()) for L in views}
        gpu.new_cache()
        gpu.set_option("wide_prefill", 0)
        gpu.prefill(prompt, 0)
        gpu.forward(5, n_prompt, spec["n_vocab"])
        for L, (K, V) in wide.items():
            assert np.array_equal(gpu.kv_read(L, 0), K) and np.array_equal(gpu.kv_read(L, 1), V)
    finally:
        gpu.close(); o.close()
