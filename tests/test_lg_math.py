"""The elementary functions of include/lg_math.h against double-precision libm: they replace the
libm calls of the reference (src/cpu/model-cpu.c:87-119) and must stay within a few ulp of them."""
import ctypes as C

import numpy as np


def ulp_err(got, want64):
    want32 = want64.astype(np.float32)
    spacing = np.spacing(np.abs(want32)).astype(np.float64)
    spacing = np.maximum(spacing, np.float64(np.finfo(np.float32).tiny))
    return np.abs(got.astype(np.float64) - want64) / spacing


def test_expf(ob):
    L = ob.lib()
    xs = np.concatenate([np.linspace(-87, 20, 20001), -np.logspace(-8, 1.9, 2000), [0.0, -0.0, -87.0, -88.0, -200.0]]).astype(np.float32)
    got = np.array([L.lgo_expf(float(x)) for x in xs], np.float32)
    want = np.exp(xs.astype(np.float64))
    live = xs >= -87.0
    assert ulp_err(got[live], want[live]).max() <= 2.0
    assert np.all(got[~live] == 0.0)                     # softmax tail flushes to zero below -87
    assert L.lgo_expf(0.0) == 1.0


def test_tanhf_and_gelu(ob):
    L = ob.lib()
    xs = np.concatenate([np.linspace(-12, 12, 24001), np.logspace(-10, 0, 500), [0.0, 0.625, -0.625, 9.0, 30.0]]).astype(np.float32)
    got = np.array([L.lgo_tanhf(float(x)) for x in xs], np.float32)
    want = np.tanh(xs.astype(np.float64))
    assert ulp_err(got, want).max() <= 4.0
    assert np.all(np.abs(got) <= 1.0)
    # gelu: both variants against the closed form in float64; absolute error (1+tanh cancels for x << 0)
    g_exact = np.array([L.lgo_gelu(float(x), 1) for x in xs], np.float32)
    g_libm = np.array([L.lgo_gelu(float(x), 0) for x in xs], np.float32)
    x64 = xs.astype(np.float64)
    want_g = 0.5 * x64 * (1.0 + np.tanh(0.7978845608028654 * (x64 + 0.044715 * x64 ** 3)))
    tol = 4e-7 * np.maximum(1.0, np.abs(x64))
    assert np.all(np.abs(g_exact - want_g) <= tol)
    assert np.all(np.abs(g_libm - want_g) <= tol)


def test_sincosf(ob):
    L = ob.lib()
    rng = np.random.default_rng(5)
    xs = np.concatenate([np.linspace(-10, 10, 4001), rng.uniform(0, 140000, 20000), np.arange(0, 9000, 1.0),
                         [0.0, 1e-8, 131071.0]]).astype(np.float32)
    s, c = C.c_float(), C.c_float()
    got_s, got_c = np.zeros(len(xs), np.float32), np.zeros(len(xs), np.float32)
    for i, x in enumerate(xs):
        L.lgo_sincosf(float(x), C.byref(s), C.byref(c))
        got_s[i], got_c[i] = s.value, c.value
    x64 = xs.astype(np.float64)
    assert np.abs(got_s - np.sin(x64)).max() <= 2.5e-7       # rotary angles: absolute accuracy is what matters
    assert np.abs(got_c - np.cos(x64)).max() <= 2.5e-7
    assert np.abs(got_s ** 2 + got_c ** 2 - 1).max() <= 5e-7


def test_f16_conversions(ob):
    L = ob.lib()
    # every binary16 value round-trips, and f16->f32 matches numpy exactly
    allh = np.arange(65536, dtype=np.uint16)
    f = np.array([L.lgo_f16_to_f32(int(h)) for h in allh], np.float32)
    want = allh.view(np.float16).astype(np.float32)
    same = (f.view(np.uint32) == want.view(np.uint32)) | (np.isnan(f) & np.isnan(want))
    assert same.all()
    back = np.array([L.lgo_f32_to_f16(float(v)) for v in want[~np.isnan(want)]], np.uint16)
    assert np.array_equal(back, allh[~np.isnan(want)])
    # f32 -> f16: dense random bit patterns plus ties, subnormals, overflow (the reference's f16_of,
    # src/cpu/model-cpu.c:185-200, is IEEE round-to-nearest-even == numpy astype)
    rng = np.random.default_rng(11)
    bits = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)
    special = np.array([0x33000000, 0x33000001, 0x32FFFFFF, 0x477FE000, 0x477FEFFF, 0x477FF000, 0x38800000, 0x387FFFFF,
                        0x3F801000, 0x3F803000, 0x3F802FFF, 0x3F801001, 0x7F800000, 0xFF800000, 0x00000001, 0x80000000], np.uint32)
    vals = np.concatenate([bits, special]).view(np.float32)
    vals = vals[~np.isnan(vals)]
    with np.errstate(over="ignore"):
        want_h = vals.astype(np.float16).view(np.uint16)
    got_h = np.array([L.lgo_f32_to_f16(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got_h, want_h)
