"""Host C layer: GGUF writer/reader, refusals the reference makes (src/gguf.c:263-279,131,183,369-375),
model geometry (src/model.c:67-196), generator determinism."""
import ctypes as C
import os
import struct
import subprocess

import numpy as np
import pytest

from conftest import ROOT, file_sha256


def open_gguf(lg, path):
    return lg.hostlib.lib().load_gguf(os.fsencode(path))


def test_generated_file_loads_and_geometry(lg, ob, model_path):
    path, spec = model_path("tiny_full")
    o = ob.Oracle(path)                      # goes through this repo's load_gguf + model_init
    try:
        assert o.info["n_layer"] == 6 and o.info["n_embd"] == 512 and o.info["n_vocab"] == 8192
        assert o.info["ple"] == 256 and o.info["n_kv_start"] == 4 and o.info["window"] == 128
        assert [l["is_local"] for l in o.layers] == [1, 0, 1, 0, 1, 0]
        assert [l["head_dim"] for l in o.layers] == [64, 128, 64, 128, 64, 128]      # from attn_q shapes
        assert all(l["n_head_kv"] == 2 for l in o.layers)                             # shared layers inherit it
        assert all(l["ffn_len"] == 2048 for l in o.layers)
    finally:
        o.close()


def test_geometry_matches_reference_loader(ob, model_path):
    """The reference's own config_load/model_init read the same numbers out of the same file."""
    if not ob.ref_available(4):
        pytest.skip("reference build absent (needs /root/reference; run make -C oracle ref)")
    for name in ("tiny", "tiny_full"):
        path, _ = model_path(name)
        o, r = ob.Oracle(path), ob.Reference(path, 4)
        try:
            c = r.config()
            assert (c["n_layer"], c["n_embd"], c["n_head"], c["n_vocab"], c["n_embd_per_layer"], c["n_kv_start"],
                    c["sliding_window"], c["n_ff"]) == tuple(o.info[k] for k in
                    ("n_layer", "n_embd", "n_head", "n_vocab", "ple", "n_kv_start", "window", "n_ff"))
            for L in range(o.info["n_layer"]):
                v = np.zeros(4, np.int32)
                r.R.ref_layer_info(r.h, L, v)
                assert v.tolist() == [o.layers[L][k] for k in ("is_local", "head_dim", "n_head_kv", "ffn_len")]
        finally:
            o.close(); r.close()


def test_generator_is_deterministic_across_thread_counts(lg, tmp_path):
    spec = dict(lg.synth.TINY, n_vocab=1024)
    code = ("import importlib,sys; sys.path.insert(0, %r); lg = importlib.import_module('little-gemma_amd'); "
            "lg.synth.write_model(sys.argv[1], **%r)" % (ROOT, spec))
    hashes = []
    for threads in ("1", "5"):
        p = str(tmp_path / f"t{threads}.gguf")
        subprocess.run(["python", "-c", code, p], check=True, env=dict(os.environ, OMP_NUM_THREADS=threads))
        hashes.append(file_sha256(p))
    assert hashes[0] == hashes[1]
    other = str(tmp_path / "seed.gguf")
    lg.synth.write_model(other, **dict(spec, seed=99))
    assert file_sha256(other) != hashes[0]


def test_golden_models_still_generate_bit_identically(model_path, golden):
    """The committed fixtures describe exactly the files this generator writes."""
    for name in ("tiny", "tiny_full"):
        path, _ = model_path(name)
        want = bytes(golden(f"ref_{name}.npz")["gguf_sha256"]).decode()
        assert file_sha256(path) == want


def _minimal_gguf(version=3, magic=0x46554747, n_meta=1, nested=False, str_len=None):
    key = b"general.architecture"
    out = struct.pack("<IIQQ", magic, version, 0, n_meta)
    out += struct.pack("<Q", len(key)) + key
    if nested:
        out += struct.pack("<I", 9) + struct.pack("<IQ", 9, 0)
    else:
        val = b"gemma4"
        out += struct.pack("<I", 8) + struct.pack("<Q", len(val) if str_len is None else str_len) + val
    return out


@pytest.mark.parametrize("what,blob", [
    ("bad magic", _minimal_gguf(magic=0x12345678)),
    ("big endian", _minimal_gguf(magic=0x47475546)),
    ("version 1", _minimal_gguf(version=1)),
    ("version 4", _minimal_gguf(version=4)),
    ("nested array", _minimal_gguf(nested=True)),
    ("string longer than the file", _minimal_gguf(str_len=1 << 20)),
    ("string over 1 GiB", _minimal_gguf(str_len=(1 << 30) + 1)),
    ("truncated header", _minimal_gguf()[:20]),
    ("truncated metadata", _minimal_gguf()[:40]),
    ("absurd counts", struct.pack("<IIQQ", 0x46554747, 3, 1 << 60, 1 << 60)),
])
def test_reader_refuses_bad_files(lg, tmp_path, what, blob):
    p = tmp_path / "bad.gguf"
    p.write_bytes(blob)
    assert open_gguf(lg, str(p)) is None, what


def test_reader_accepts_v2_and_v3_and_refuses_offsets_past_the_data(lg, tmp_path):
    H = lg.hostlib.lib()
    for version in (2, 3):
        p = tmp_path / f"v{version}.gguf"
        p.write_bytes(_minimal_gguf(version=version))
        ctx = open_gguf(lg, str(p))
        assert ctx is not None
        H.free_gguf(ctx)
    # one tensor whose offset lies beyond the data section
    name = b"t"
    blob = struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + struct.pack("<Q", 1) + name + struct.pack("<IQIQ", 1, 32, 0, 4096)
    blob += b"\0" * (-len(blob) % 32) + b"\0" * 128
    p = tmp_path / "off.gguf"
    p.write_bytes(blob)
    assert open_gguf(lg, str(p)) is None


def test_data_cap_is_enforced(lg, model_path):
    H = lg.hostlib.lib()
    path, _ = model_path("tiny")
    H.gguf_set_max_data_bytes.argtypes = [C.c_size_t]
    H.gguf_set_max_data_bytes(1024)
    try:
        assert open_gguf(lg, path) is None
    finally:
        H.gguf_set_max_data_bytes(0)
    ctx = open_gguf(lg, path)
    assert ctx is not None
    H.free_gguf(ctx)


def test_model_init_reports_missing_tensors(lg, ob, tmp_path):
    """A file without attn_q for a layer is refused by model_init (src/model.c:175-178)."""
    H = lg.hostlib.lib()
    H.lg_gw_open.restype = C.c_void_p
    H.lg_gw_open.argtypes = [C.c_char_p, C.c_uint32, C.c_uint32]
    for f in ("lg_gw_meta_str", "lg_gw_meta_u32"):
        getattr(H, f).argtypes = [C.c_void_p, C.c_char_p, C.c_char_p if f.endswith("str") else C.c_uint32]
    H.lg_gw_commit.argtypes = [C.c_void_p]
    H.lg_gw_close.argtypes = [C.c_void_p]
    p = str(tmp_path / "empty.gguf")
    w = H.lg_gw_open(p.encode(), 3, 32)
    H.lg_gw_meta_str(w, b"general.architecture", b"gemma4")
    H.lg_gw_meta_u32(w, b"gemma4.block_count", 2)
    H.lg_gw_meta_u32(w, b"gemma4.attention.head_count", 8)
    assert H.lg_gw_commit(w) == 0 and H.lg_gw_close(w) == 0
    with pytest.raises(RuntimeError):
        ob.Oracle(p)
    # no architecture at all / zero layers: config_load refuses (src/model.c:70-75,104-113)
    w = H.lg_gw_open(p.encode(), 3, 32)
    H.lg_gw_meta_u32(w, b"gemma4.block_count", 2)
    assert H.lg_gw_commit(w) == 0 and H.lg_gw_close(w) == 0
    with pytest.raises(RuntimeError):
        ob.Oracle(p)


def test_bench_refuses_more_than_one_gpu():
    """The verify step is not sharded: bench.py --gpus N with N > 1 exits with a message that says so
    (before anything touches a device)."""
    import subprocess, sys, os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""
