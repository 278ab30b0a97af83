"""Shared fixtures.  CPU tests (`-m "not gpu"`) cover the oracle, the host layer and the C ABI's
surface; GPU tests (`-m gpu`) are the parity tests proper and call the HIP path through the C ABI
and the model.h backend."""
import hashlib
import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lg():
    return importlib.import_module("little-gemma_amd")


@pytest.fixture(scope="session")
def ob():
    from oracle import binding
    binding.lib()
    return binding


@pytest.fixture(scope="session")
def model_dir(tmp_path_factory):
    return tmp_path_factory.mktemp("models")


@pytest.fixture(scope="session")
def model_path(lg, model_dir):
    """model_path(name, **overrides) -> path of a generated GGUF (cached per session)."""
    made = {}

    def make(name, **over):
        spec = dict(getattr(lg.synth, name.upper()))
        spec.update(over)
        key = name + "".join(f"_{k}{v}" for k, v in sorted(over.items()))
        if key not in made:
            path = os.path.join(str(model_dir), key + ".gguf")
            lg.synth.write_model(path, **spec)
            made[key] = (path, spec)
        return made[key]
    return make


@pytest.fixture(scope="session")
def golden():
    def load(name):
        return np.load(os.path.join(GOLDEN, name))
    return load


def file_sha256(path):
    h = hashlib.sha256()
    with open(path, "rb") as f:
        for chunk in iter(lambda: f.read(1 << 20), b""):
            h.update(chunk)
    return h.hexdigest()


def random_q4_0(rng, m, k, scale_std=0.01):
    """m rows of k/32 q4_0 blocks: f16 scale ~ N(0, scale_std), codes uniform 0..15."""
    nb = k // 32
    w = np.zeros((m, nb, 18), np.uint8)
    d = rng.normal(0, scale_std, (m, nb)).astype(np.float16)
    w[:, :, 0:2] = d.view(np.uint8).reshape(m, nb, 2)
    w[:, :, 2:] = rng.integers(0, 256, (m, nb, 16), dtype=np.uint8)
    return w.reshape(-1)


def q4_0_codes(w, m, k):
    """(scales f32 [m, nb], codes int [m, nb, 32]) of a q4_0 byte array."""
    nb = k // 32
    b = np.asarray(w, np.uint8).reshape(m, nb, 18)
    d = b[:, :, 0:2].copy().view(np.float16).reshape(m, nb).astype(np.float32)
    qs = b[:, :, 2:]
    codes = np.concatenate([qs & 15, qs >> 4], axis=2).astype(np.int32)
    return d, codes


def quant_q8_numpy(x):
    """numpy restatement of the activation quantization: per 32, f32 arithmetic, ties to even."""
    x = np.asarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(d > 0, np.float32(1.0) / np.where(d > 0, d, np.float32(1)), np.float32(0)).astype(np.float32)
    q = np.rint((x * inv[:, None]).astype(np.float32)).astype(np.int32)
    return q.astype(np.int8), d, q.sum(axis=1).astype(np.int32)


def has_gpu():
    lg_ = importlib.import_module("little-gemma_amd")
    try:
        return lg_.hiplib.device_count() > 0
    except Exception:
        return False


@pytest.fixture(scope="session")
def gpu_required(lg):
    if lg.hiplib.device_count() < 1:
        pytest.fail("a test marked gpu ran without a GPU: the HIP path has no CPU fallback")
    return True


def gguf_tensor_span(path, name):
    """(file offset, byte length, dims) of one tensor's data in a GGUF file: a minimal reader of the container
    (header, metadata, tensor infos, alignment) for tests that edit a generated model in place."""
    import struct
    sizes = {0: 1, 1: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 7: 1, 10: 8, 11: 8, 12: 8}
    type_bytes = {0: (1, 4), 1: (1, 2), 2: (32, 18), 8: (32, 34), 30: (1, 2)}       # ggml type -> (block elems, block bytes)
    with open(path, "rb") as f:
        data = f.read()
    at = 0

    def take(fmt):
        nonlocal at
        v = struct.unpack_from("<" + fmt, data, at)
        at += struct.calcsize("<" + fmt)
        return v[0] if len(v) == 1 else v

    def string():
        nonlocal at
        n = take("Q")
        s = data[at:at + n].decode()
        at += n
        return s

    def skip_value(t):
        nonlocal at
        if t == 8:
            string()
        elif t == 9:
            et, n = take("I"), take("Q")
            for _ in range(n):
                skip_value(et)
        else:
            at += sizes[t]

    magic, version, n_tensors, n_meta = take("I"), take("I"), take("Q"), take("Q")
    assert magic == 0x46554747 and version in (2, 3)
    align = 32
    for _ in range(n_meta):
        key, t = string(), take("I")
        if key == "general.alignment" and t == 4:
            align = take("I")
        else:
            skip_value(t)
    found = None
    for _ in range(n_tensors):
        tname, nd = string(), take("I")
        dims = [take("Q") for _ in range(nd)]
        ttype, off = take("I"), take("Q")
        if tname == name:
            found = (ttype, dims, off)
    assert found, f"{name} not in {path}"
    base = (at + align - 1) // align * align
    ttype, dims, off = found
    be, bb = type_bytes[ttype]
    n = 1
    for d in dims:
        n *= d
    return base + off, n // be * bb, dims
