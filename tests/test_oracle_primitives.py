"""Pins the oracle's primitives: against the reference-produced q4_0 fixture, against closed forms by
brute force, and against float64 restatements chosen so that a dropped term, a wrong index or a
transposed operand fails."""
import itertools

import numpy as np
import pytest

from conftest import q4_0_codes, quant_q8_numpy, random_q4_0


def test_q4_0_dequant_matches_reference_fixture(lg, golden):
    """bytes -> floats exactly as the reference's dequantize_into produced them (src/quant.c:276-285)."""
    g = golden("q4_0_dequant.npz")
    blocks, want = g["blocks"], g["values"]
    out = np.zeros(want.size, np.float32)
    assert lg.hostlib.lib().dequantize_into(2, blocks.ctypes.data, out.ctypes.data, out.size)
    assert np.array_equal(out.view(np.uint32), want.reshape(-1).view(np.uint32))
    # and the closed form: d * (nibble - 8), low nibbles first
    d, codes = q4_0_codes(blocks.reshape(-1), 64, 32)
    closed = (d[:, :, None] * (codes - 8).astype(np.float32)).reshape(64, 32).astype(np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(closed[finite], want[finite])


def test_q4_0_quantize_roundtrip(lg):
    rng = np.random.default_rng(2)
    x = rng.normal(0, 0.02, 64 * 32).astype(np.float32)
    x[:32] = 0.0
    packed = np.zeros(64 * 18, np.uint8)
    H = lg.hostlib.lib()
    H.lg_quantize_q4_0(x.ctypes.data, packed.ctypes.data, x.size)
    back = np.zeros_like(x)
    assert H.dequantize_into(2, packed.ctypes.data, back.ctypes.data, x.size)
    amax = np.abs(x.reshape(64, 32)).max(axis=1)
    err = np.abs(back - x).reshape(64, 32).max(axis=1)
    assert np.all(err <= amax / 8 * 1.001 + 1e-9)      # one code step (the +8 end clips at 15)
    assert np.all(back[:32] == 0.0)


def test_block_dot_closed_form(ob):
    rng = np.random.default_rng(3)
    L = ob.lib()
    for _ in range(200):
        blk = rng.integers(0, 256, 18, dtype=np.uint8)
        q = rng.integers(-127, 128, 32).astype(np.int8)
        _, codes = q4_0_codes(blk, 1, 32)
        assert L.lgo_block_dot(blk, q) == int(((codes.reshape(32) - 8) * q.astype(np.int32)).sum())
    # extremes: |dot| <= 32 * 8 * 127
    blk = np.zeros(18, np.uint8)
    assert L.lgo_block_dot(blk, np.full(32, 127, np.int8)) == -8 * 127 * 32
    blk[2:] = 0xFF
    assert L.lgo_block_dot(blk, np.full(32, 127, np.int8)) == 7 * 127 * 32


def test_quant_q8_against_numpy(ob):
    rng = np.random.default_rng(4)
    L = ob.lib()
    x = rng.normal(0, 1, 64 * 32).astype(np.float32)
    x[0:32] = 0.0                                         # all-zero group: d = 0, id = 0, q = 0
    x[32:64] = np.float32(2.5)                            # every value at amax -> +127
    x[64:96] = np.linspace(-1, 1, 32, dtype=np.float32) * np.float32(127.0 * 0.5)   # .5 ties round to even
    x[96:128] = rng.normal(0, 1e-30, 32).astype(np.float32)
    q = np.zeros(x.size, np.int8); d = np.zeros(x.size // 32, np.float32); s = np.zeros(x.size // 32, np.int32)
    L.lgo_quant_q8(x, x.size, q, d, s)
    wq, wd, ws = quant_q8_numpy(x)
    assert np.array_equal(q, wq.reshape(-1)) and np.array_equal(d.view(np.uint32), wd.view(np.uint32)) and np.array_equal(s, ws)
    assert np.all(q[:32] == 0) and d[0] == 0 and np.all(q[32:64] == 127)
    assert np.abs(q.astype(np.int32)).max() <= 127


@pytest.mark.parametrize("m,k,rows", [(64, 256, 1), (96, 2560, 5), (32, 10240, 4), (40, 512, 2)])
def test_matmul_q4q8_against_float64(ob, m, k, rows):
    rng = np.random.default_rng(m + k + rows)
    L = ob.lib()
    nb = k // 32
    w = random_q4_0(rng, m, k)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    xq, xd, _ = quant_q8_numpy(x)
    xq = np.ascontiguousarray(xq.reshape(rows, k)); xd = np.ascontiguousarray(xd.reshape(rows, nb))
    dw, codes = q4_0_codes(w, m, k)
    dots_want = np.einsum("ibe,jbe->jib", codes - 8, xq.reshape(rows, nb, 32).astype(np.int32))
    want = np.einsum("jib,ib,jb->ji", dots_want.astype(np.float64), dw.astype(np.float64), xd.astype(np.float64))
    outs = {}
    for order in (ob.ORDER_SEG, ob.ORDER_CUDA32):
        out = np.zeros((rows, m), np.float32); dots = np.zeros((rows, m, nb), np.int32)
        L.lgo_matmul_q4q8(w, k, m, xq, xd, rows, out, dots.ctypes.data, order)
        assert np.array_equal(dots, dots_want)                         # int32 block dots: exact
        scale = np.abs(want).max()
        assert np.abs(out - want).max() <= 1e-5 * scale
        outs[order] = out
    # the two summation orders are the same mathematics: they differ by rounding only
    assert np.abs(outs[ob.ORDER_SEG] - outs[ob.ORDER_CUDA32]).max() <= 2e-6 * np.abs(want).max()
    # transposition / indexing check: the f32-activation matmul on the dequantized operands agrees to q8 noise
    xdeq = (xq.reshape(rows, nb, 32).astype(np.float32) * xd[:, :, None]).reshape(rows, k)
    ref = np.zeros(m, np.float32)
    L.lgo_matmul_f32(w, 2, k, m, np.ascontiguousarray(xdeq[0]), ref)
    assert np.abs(ref - outs[ob.ORDER_SEG][0]).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("gtype,k,m", [(0, 2560, 48), (1, 256, 40), (30, 512, 33), (0, 256, 8)])
def test_matmul_float_weights_against_float64(ob, gtype, k, m):
    """f32 / f16 / bf16 weight rows x one f32 vector: within reorder noise of float64, exact where the arithmetic
    is exact (unit rows pick an element, small integers sum exactly in any order), and the same value as the
    serial-order matmul up to rounding (a transposed or mis-strided operand fails all three)."""
    rng = np.random.default_rng(gtype + k + m)
    L = ob.lib()
    wf = rng.normal(0, 0.02, (m, k)).astype(np.float32)
    wf[0] = 0.0; wf[0, k - 3] = 1.0                                   # unit row: out = x[k-3] exactly
    wf[1] = rng.integers(-4, 5, k).astype(np.float32)                 # small integers x small integers: exact
    if gtype == 1:
        raw = wf.astype(np.float16); wf = raw.astype(np.float32); raw = raw.view(np.uint16)
    elif gtype == 30:
        raw = (wf.view(np.uint32) >> 16).astype(np.uint16); wf = (raw.astype(np.uint32) << 16).view(np.float32)
    else:
        raw = wf
    x = rng.normal(0, 1, k).astype(np.float32)
    xi = rng.integers(-8, 9, k).astype(np.float32)
    out = np.zeros(m, np.float32); outi = np.zeros(m, np.float32); ser = np.zeros(m, np.float32)
    wb = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    L.lgo_matmul_fw(wb, gtype, k, m, x, out)
    L.lgo_matmul_fw(wb, gtype, k, m, xi, outi)
    L.lgo_matmul_f32(wb, gtype, k, m, x, ser)
    want = wf.astype(np.float64) @ x.astype(np.float64)
    mag = np.abs(wf).astype(np.float64) @ np.abs(x).astype(np.float64)   # rounding scales with the sum of magnitudes
    assert np.all(np.abs(out - want) <= 1e-6 * mag + 1e-12)
    assert np.all(np.abs(out - ser) <= 2e-6 * mag + 1e-12)
    assert out[0] == x[k - 3]
    assert outi[1] == np.float32(wf[1].astype(np.float64) @ xi.astype(np.float64))


def test_rmsnorm_both_orders(ob):
    rng = np.random.default_rng(6)
    L = ob.lib()
    for n in (64, 256, 512, 2560, 3840):
        x = rng.normal(0, 3, n).astype(np.float32); w = rng.normal(1, 0.1, n).astype(np.float32)
        want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-6) * w
        for tree in (0, 1):
            out = np.zeros(n, np.float32)
            L.lgo_rmsnorm(out, x, w.ctypes.data, n, 1e-6, tree)
            assert np.abs(out - want).max() <= 3e-6 * np.abs(want).max()
        out = np.zeros(n, np.float32)
        L.lgo_rmsnorm(out, x, None, n, 1e-6, 1)                 # weightless form (V rows)
        assert np.abs(out - want / w).max() <= 3e-6 * np.abs(want / w).max()


def test_rope_neox_pairs(ob):
    rng = np.random.default_rng(7)
    L = ob.lib()
    for d, pos, base in ((64, 0, 1e4), (256, 2051, 1e6), (128, 8191, 1e4)):
        v = rng.normal(0, 1, d).astype(np.float32)
        tab = np.array([np.float32(base) ** np.float32(-2.0 * i / d) for i in range(d // 2)], np.float32)
        ff = rng.uniform(1, 4, d // 2).astype(np.float32)
        for ffp in (None, ff):
            ang = pos * tab.astype(np.float64) / (ff if ffp is not None else 1.0)
            a, b = v[: d // 2].astype(np.float64), v[d // 2:].astype(np.float64)
            want = np.concatenate([a * np.cos(ang) - b * np.sin(ang), a * np.sin(ang) + b * np.cos(ang)])
            for exact in (0, 1):
                got = v.copy()
                L.lgo_rope(got, d, pos, tab, ffp.ctypes.data if ffp is not None else None, exact)
                assert np.abs(got - want).max() <= 2e-3 if pos > 1000 else np.abs(got - want).max() <= 1e-5
        # position 0 is the identity
        got = v.copy()
        L.lgo_rope(got, d, 0, tab, None, 1)
        assert np.array_equal(got, v)


def attention_f64(q, kc, vc, hd, kd, kvh, seq, start, pos):
    K = kc.view(np.float16).astype(np.float64).reshape(seq, kd)[:, kvh * hd:(kvh + 1) * hd]
    V = vc.view(np.float16).astype(np.float64).reshape(seq, kd)[:, kvh * hd:(kvh + 1) * hd]
    rows = [t % seq for t in range(start, pos + 1)]
    s = K[rows] @ q.astype(np.float64)
    p = np.exp(s - s.max()); p /= p.sum()
    return p @ V[rows]


@pytest.mark.parametrize("hd,seq,window,pos", [(64, 160, 128, 5), (64, 160, 128, 127), (64, 160, 128, 401),
                                                (256, 300, 0, 299), (128, 96, 0, 0), (256, 544, 512, 2050)])
def test_attention_tiled_and_two_pass(ob, hd, seq, window, pos):
    rng = np.random.default_rng(hd + pos)
    L = ob.lib()
    nkv, kvh = 2, 1
    kd = nkv * hd
    kc = rng.normal(0, 1, seq * kd).astype(np.float16).view(np.uint16)
    vc = rng.normal(0, 1, seq * kd).astype(np.float16).view(np.uint16)
    q = (rng.normal(0, 1, hd) * 0.3).astype(np.float32)
    start = max(0, pos - window + 1) if window else 0
    want = attention_f64(q, kc, vc, hd, kd, kvh, seq, start, pos)
    outs = []
    for tiled, exact in ((0, 0), (1, 0), (1, 1)):
        out = np.zeros(hd, np.float32)
        L.lgo_attention_f16(out, q, kc, vc, hd, kd, kvh, seq, start, pos, tiled, exact)
        assert np.abs(out - want).max() <= 1e-5 * max(1.0, np.abs(want).max())   # f32 sums over up to 512 keys
        outs.append(out)
    # keys outside [start, pos] must not matter: scramble them and the result is bit-identical
    k2, v2 = kc.copy().reshape(seq, kd), vc.copy().reshape(seq, kd)
    live = {t % seq for t in range(start, pos + 1)}
    for r in range(seq):
        if r not in live:
            k2[r] = rng.integers(0, 0x7BFF, kd); v2[r] = rng.integers(0, 0x7BFF, kd)
    out2 = np.zeros(hd, np.float32)
    L.lgo_attention_f16(out2, q, k2.reshape(-1), v2.reshape(-1), hd, kd, kvh, seq, start, pos, 1, 1)
    assert np.array_equal(out2.view(np.uint32), outs[2].view(np.uint32))


def test_accept_rule_exhaustive(ob):
    """adv = 1 + length of the leading run of held drafts (src/cuda/mtp-kernel.cuh:114-116), every pattern."""
    L = ob.lib()
    for rows in range(1, 6):
        for pattern in itertools.product((0, 1), repeat=rows - 1):
            toks = np.arange(10, 10 + rows, dtype=np.int32)
            out = np.array([toks[j + 1] if j + 1 < rows and pattern[j] else 999 for j in range(rows)], np.int32)
            want = 1
            for held in pattern:
                if not held:
                    break
                want += 1
            assert L.lgo_accept(toks, out, rows) == want


def test_ring_rows(ob):
    L = ob.lib()
    assert L.lgo_ring_rows(128, 4096) == 640 and L.lgo_ring_rows(512, 4096) == 1024 and L.lgo_ring_rows(1024, 9000) == 1536
    assert L.lgo_ring_rows(128, 400) == 256 and L.lgo_ring_rows(512, 1000) == 640     # short caches: 128 spare rows
    assert L.lgo_ring_rows(512, 300) == 300                     # never more rows than positions
    for w in (100, 128, 511, 512, 1000):
        assert L.lgo_ring_rows(w, 1 << 20) % 32 == 0 and L.lgo_ring_rows(w, 1 << 20) >= w + 128 - 1


def test_division_by_127_in_three_instructions_is_the_ieee_quotient():
    """The device quantizer forms amax/127 as fma(fma(-127, q0, amax), r, q0) with q0 = amax*r, r = fl(1/127).
    Exact rational arithmetic with one rounding per operation (what mul and fma do) must land on the
    correctly rounded quotient: edge values and a seeded sample here; the full sweep over every non-negative
    finite float was run once offline (0 mismatches)."""
    from fractions import Fraction

    def fl(x):                       # nearest float32 to a rational, ties to even, subnormals included
        if x == 0:
            return Fraction(0)
        if x < 0:
            return -fl(-x)
        e = x.numerator.bit_length() - x.denominator.bit_length()
        if Fraction(2) ** e > x:
            e -= 1                   # 2^e <= x < 2^(e+1)
        e = max(e, -126)             # below the normal range the spacing stays 2^-149
        q = Fraction(2) ** (e - 23)
        n = x / q
        lo = n.numerator // n.denominator
        rem = n - lo
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
            lo += 1
        return lo * q

    r = fl(Fraction(1, 127))
    assert float(r) == float(np.float32(1.0) / np.float32(127.0))
    rng = np.random.default_rng(127)
    bits = np.concatenate([
        np.array([0, 1, 2, 126, 127, 128, 0x007FFFFF, 0x00800000, 0x00800001, 0x3F800000, 0x42FE0000, 0x7F7FFFFF], np.uint32),
        rng.integers(0, 0x7F800000, 3000, dtype=np.uint32),
        rng.integers(0, 0x01000000, 500, dtype=np.uint32)])           # dense around the subnormal boundary
    for b in bits:
        a = Fraction(float(np.array([b], np.uint32).view(np.float32)[0]))
        q0 = fl(a * r)
        e = fl(a - 127 * q0)
        q = fl(e * r + q0)
        assert q == fl(a / 127), hex(int(b))
