"""The C ABI without a GPU: the library loads, exports every symbol include/lg_hip.h declares,
its host-side pieces work, and compute entry points refuse loudly when no device exists."""
import ctypes as C
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from conftest import ROOT, has_gpu, random_q4_0


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "lg_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lg_hip_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lg):
    H = lg.hiplib.load_hip()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(H, n), f"{n} is declared in include/lg_hip.h but not exported"


def test_backend_library_defines_the_model_h_symbols(lg):
    B = lg.hiplib.load_backend()
    for n in ("kvcache_init", "kvcache_free", "kvcache_save_prefix", "kvcache_restore_prefix", "model_forward",
              "model_forward_next", "model_prefill", "model_prefill_embd", "model_prefill_mixed", "model_prefill_reserve",
              "model_forward_spec", "mtp_draft_device", "mtp_draft_chain_device", "mtp_free_device", "model_kv_host",
              "model_init", "model_free", "config_load", "load_gguf"):
        assert hasattr(B, n), n
    assert C.c_int.in_dll(B, "model_kv_host").value == 0


def test_repack_layout_against_numpy(lg):
    """Tile (group g, it): lane r*S+c holds block c*nit+it of row g*(64/S)+r — 16 nibble bytes, then scales."""
    H = lg.hiplib.load_hip()
    rng = np.random.default_rng(8)
    for m, k in ((16, 256), (24, 2560), (8, 512), (8, 10240), (16, 15360)):
        w = random_q4_0(rng, m, k)
        nb = k // 32
        S = H.lg_hip_segments(k)
        assert S == (32 if nb > 128 else 8)
        rw, nit = 64 // S, nb // S
        n = H.lg_hip_repacked_bytes(k, m)
        assert n == (m // rw) * nit * 1152 == w.size                 # same bytes, reordered
        out = np.zeros(n, np.uint8)
        assert H.lg_hip_repack_q4_0(w, k, m, out) == 0
        blocks = w.reshape(m, nb, 18)
        tiles = out.reshape(m // rw, nit, 1152)
        for g in range(m // rw):
            for it in range(nit):
                for r in range(rw):
                    for c in range(S):
                        blk = blocks[g * rw + r, c * nit + it]
                        lane = r * S + c
                        assert np.array_equal(tiles[g, it, lane * 16:lane * 16 + 16], blk[2:])
                        assert np.array_equal(tiles[g, it, 1024 + lane * 2:1024 + lane * 2 + 2], blk[:2])
    assert H.lg_hip_repacked_bytes(100, 8) == 0 and H.lg_hip_repacked_bytes(256, 12) == 0
    assert H.lg_hip_repack_q4_0(np.zeros(18, np.uint8), 32, 8, np.zeros(18, np.uint8)) < 0
    assert b"multiple of 256" in H.lg_hip_last_error()


def test_ring_rows_agree_with_the_oracle(lg, ob):
    H, L = lg.hiplib.load_hip(), ob.lib()
    for k in (256, 2560, 4096, 4352, 10240):
        assert H.lg_hip_segments(k) == L.lgo_segments(k)
    for window, max_seq in ((128, 4096), (512, 2300), (1024, 8300), (512, 400), (7, 64)):
        assert H.lg_hip_ring_rows(window, max_seq) == L.lgo_ring_rows(window, max_seq)


def test_attention_partials_of_a_cache_stay_within_their_budget(lg):
    """The byte count lg_hip_kv_create asks for beside the rings, at the E4B and 12B shapes (8 verify rows): the
    widest prompt block steps down with the cache length so that rows x heads x key tiles x (head_dim + 2) floats
    never pass 2 GiB; the closed form is recomputed here from the returned block width."""
    import ctypes as C
    H = lg.hiplib.load_hip()
    H.lg_hip_kv_partials.restype = C.c_size_t
    H.lg_hip_kv_partials.argtypes = [C.c_int] * 6 + [C.POINTER(C.c_int)] * 2
    cases = {  # (heads, window) -> max_seq -> widest prompt block
        (8, 512): {600: 128, 4136: 512, 8192: 512, 32768: 128, 131072: 32},
        (16, 1024): {4136: 512, 32768: 32, 131072: 0},
    }
    for (heads, window), by_seq in cases.items():
        for max_seq, want_wide in by_seq.items():
            wide, tiles = C.c_int(-1), C.c_int(-1)
            got = H.lg_hip_kv_partials(max_seq, window, 1, 8, heads, 256, C.byref(wide), C.byref(tiles))
            assert wide.value == want_wide, (heads, max_seq, wide.value)
            assert tiles.value == max_seq // 32 + 2
            assert got == max(wide.value, 8) * heads * tiles.value * (256 * 4 + 8)
            assert got <= 2 << 30
    # sliding layers only: the tiles a block can touch are bounded by window + block
    wide, tiles = C.c_int(), C.c_int()
    H.lg_hip_kv_partials(131072, 512, 0, 8, 8, 256, C.byref(wide), C.byref(tiles))
    assert wide.value == 512 and tiles.value == (512 + 512) // 32 + 2


@pytest.mark.skipif(has_gpu(), reason="checks the behaviour of a machine without a GPU")
def test_compute_calls_fail_loudly_without_a_device(lg, model_path):
    H = lg.hiplib.load_hip()
    assert H.lg_hip_device_count() == 0
    rng = np.random.default_rng(1)
    with pytest.raises(lg.hiplib.HipError, match="no HIP device"):
        lg.hiplib.matmul_q4q8(random_q4_0(rng, 8, 256), 256, 8, np.zeros((1, 256), np.float32))
    path, _ = model_path("tiny")
    with pytest.raises(lg.hiplib.HipError, match="no HIP device"):
        lg.hiplib.HipBackend(path, 64)


def test_model_hip_compiles_against_the_reference_headers():
    """Drop-in check: the backend translation unit builds against the reference's own model.h/gguf.h."""
    ref = "/root/reference"
    if not os.path.isdir(os.path.join(ref, "include")) or not shutil.which("gcc"):
        pytest.skip("reference headers absent")
    src = os.path.join(ROOT, "little-gemma_amd", "host", "model-hip.c")
    for n in ("2", "4"):
        subprocess.run(["gcc", "-fsyntax-only", "-std=gnu11", "-Wall", "-Wextra", "-Werror", f"-DLG_MTP_N={n}",
                        f"-I{ref}/include", f"-I{ref}/src", f"-I{ROOT}/include", src], check=True)


def test_reference_core_links_against_the_hip_backend(lg, tmp_path):
    """The drop-in claim as a link: the reference's unmodified CLI core (the CORE list of its CMakeLists.txt:42-45:
    run.c gguf.c quant.c model.c tokenizer.c media.c mtp.c + the no-op media GPU seam) compiled from where it
    lies, with this repository's model-hip.c as the backend translation unit and liblg_hip.so behind it, must
    link with no undefined symbol (what `-fsyntax-only` cannot show) and start (it prints its usage)."""
    ref = "/root/reference"
    if not os.path.isdir(os.path.join(ref, "src")) or not shutil.which("gcc"):
        pytest.skip("reference sources absent")
    lg.hiplib.load_hip()                                   # the library must be built
    csrc = os.path.join(ROOT, "little-gemma_amd", "csrc")
    exe = str(tmp_path / "run-hip-from-reference-core")
    core = [os.path.join(ref, "src", f) for f in ("run.c", "gguf.c", "quant.c", "model.c", "tokenizer.c", "media.c", "mtp.c")]
    core.append(os.path.join(ref, "src", "cpu", "media-gpu-stub.c"))
    cmd = ["gcc", "-std=gnu11", "-O1", "-DLG_MTP_N=4", f"-I{ref}/include", f"-I{ref}/src", f"-I{ROOT}/include", *core,
           os.path.join(ROOT, "little-gemma_amd", "host", "model-hip.c"), f"-L{csrc}", "-llg_hip", f"-Wl,-rpath,{csrc}",
           "-Wl,--no-undefined", "-lm", "-fopenmp", "-o", exe]
    subprocess.run(cmd, check=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert "Usage" in (r.stdout + r.stderr) and "-mtp" in (r.stdout + r.stderr)


def test_product_sources_do_not_touch_the_oracle():
    """Nothing that ships may include, link or import anything under oracle/."""
    pkg = os.path.join(ROOT, "little-gemma_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".c", ".h", ".hip", ".py", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                for pat in (r'#\s*include\s*[<"][^>"]*oracle', r"\bfrom\s+oracle\b", r"\bimport\s+oracle\b",
                            r"lg_oracle", r"\blgo_[a-z]", r"oracle/"):
                    assert not re.search(pat, text), (os.path.join(dirpath, f), pat)
