"""GPU parity of the parts, through the C ABI: the isolated q4_0 x q8 matmul (the benchmark list's isolated-matmul configuration),
the decode attention over an f16 ring (config 3), the row kernel (add-norm, norm, q8), the fused
rows + per-layer gate kernel and the per-layer inputs.  Bar: int32 block dots and every integer
bit-exact; f32 outputs bit-identical to the oracle in this build's summation order and within
1e-5 relative of float64."""
import numpy as np
import pytest

from conftest import q4_0_codes, quant_q8_numpy, random_q4_0

pytestmark = pytest.mark.gpu


def oracle_matmul(ob, w, k, m, x):
    L = ob.lib()
    rows, nb = x.shape[0], k // 32
    xq = np.zeros((rows, k), np.int8); xd = np.zeros((rows, nb), np.float32); xs = np.zeros((rows, nb), np.int32)
    for j in range(rows):
        L.lgo_quant_q8(x[j], k, xq[j], xd[j], xs[j])
    out = np.zeros((rows, m), np.float32); dots = np.zeros((rows, m, nb), np.int32)
    L.lgo_matmul_q4q8(w, k, m, xq, xd, rows, out, dots.ctypes.data, ob.ORDER_SEG)
    return xq, xd, xs, out, dots


@pytest.mark.parametrize("rows", [1, 2, 4, 5])
def test_matmul_config2_full_size(lg, ob, gpu_required, rows):
    """W 10240 x 2560 q4_0 (f16 scales ~N(0,0.01), codes uniform), X ~ N(0,1), M in {1,2,4,5}."""
    m, k = 10240, 2560
    rng = np.random.default_rng(100 + rows)
    w = random_q4_0(rng, m, k)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    print(f"matmul m={m} k={k} rows={rows}", flush=True)
    r = lg.hiplib.matmul_q4q8(w, k, m, x, want_dots=True)
    xq, xd, xs, out, dots = oracle_matmul(ob, w, k, m, x)
    nq, nd, ns = quant_q8_numpy(x)
    assert np.array_equal(r["xq"], nq.reshape(rows, k)) and np.array_equal(r["xq"], xq)
    assert np.array_equal(r["xd"].view(np.uint32), nd.reshape(rows, -1).view(np.uint32))
    assert np.array_equal(r["xsum"], ns.reshape(rows, -1)) and np.array_equal(r["xsum"], xs)
    # int32 block dots: bit-exact against the closed form sum((nibble-8)*q), all 10240*80*rows of them
    dw, codes = q4_0_codes(w, m, k)
    want_dots = np.einsum("ibe,jbe->jib", codes - 8, xq.reshape(rows, k // 32, 32).astype(np.int32))
    assert np.array_equal(r["dots"], want_dots) and np.array_equal(r["dots"], dots)
    # f32: bit-identical to the oracle's order, 1e-5 relative against float64
    assert np.array_equal(r["out"].view(np.uint32), out.view(np.uint32))
    want = np.einsum("jib,ib,jb->ji", want_dots.astype(np.float64), dw.astype(np.float64), xd.astype(np.float64))
    assert np.abs(r["out"] - want).max() <= 1e-5 * np.abs(want).max()


@pytest.mark.parametrize("m,k,rows", [(8, 256, 1), (2560, 10240, 5), (2048, 256, 8), (512, 3840, 3), (264, 15360, 8),
                                      (512, 3840, 5), (264, 4096, 8), (72, 3072, 4)])   # (the last three: a row group's tiles cut over four wavefronts)
def test_matmul_edge_shapes(lg, ob, gpu_required, m, k, rows):
    rng = np.random.default_rng(m + k)
    w = random_q4_0(rng, m, k)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[0, :64] = 0.0                                      # zero groups: scale 0, no NaN
    x[rows - 1, 32:64] = 1e-30
    print(f"matmul m={m} k={k} rows={rows}", flush=True)
    r = lg.hiplib.matmul_q4q8(w, k, m, x, want_dots=True)
    xq, xd, xs, out, dots = oracle_matmul(ob, w, k, m, x)
    assert np.array_equal(r["xq"], xq) and np.array_equal(r["xsum"], xs) and np.array_equal(r["dots"], dots)
    assert np.array_equal(r["out"].view(np.uint32), out.view(np.uint32))
    # without the dump of the block dots the launcher may pick another kernel for the same shape (K cut over
    # several wavefronts): the same bits
    r2 = lg.hiplib.matmul_q4q8(w, k, m, x)
    assert np.array_equal(r2["out"].view(np.uint32), out.view(np.uint32))
    assert np.all(np.isfinite(r["out"]))


@pytest.mark.parametrize("m,k,rows", [(256, 2560, 5), (2560, 256, 8), (10, 512, 1), (77, 1024, 21)])
def test_matmul_float_weights_matches_oracle(lg, ob, gpu_required, m, k, rows):
    """f32 weight matrix x f32 rows (what a float-typed per-layer-embedding matrix goes through): bit-identical to
    the oracle's order for every row of the block, ragged row counts and row groups included."""
    rng = np.random.default_rng(m * 7 + k + rows)
    w = rng.normal(0, 0.02, (m, k)).astype(np.float32)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[0, :64] = 0.0
    print(f"matmul_f32w m={m} k={k} rows={rows}", flush=True)
    got = lg.hiplib.matmul_f32w(w, x)
    L = ob.lib()
    for j in range(rows):
        want = np.zeros(m, np.float32)
        L.lgo_matmul_fw(w.view(np.uint8).reshape(-1), 0, k, m, np.ascontiguousarray(x[j]), want)
        assert np.array_equal(got[j].view(np.uint32), want.view(np.uint32)), f"row {j}"


@pytest.mark.parametrize("rows,E,with_dout,with_os,with_pre", [(5, 2560, True, True, True), (1, 512, True, False, True),
                                                            (8, 3840, True, True, False), (3, 256, False, False, True),
                                                            (4, 4096, False, False, False)])
def test_rows_kernel_matches_oracle(lg, ob, gpu_required, rows, E, with_dout, with_os, with_pre):
    """The row work between two matmuls in isolation (add-norm, output scale, norm, q8): the updated residual, the
    normed row and its q8 are the oracle's, bit for bit, with and without each optional part."""
    rng = np.random.default_rng(rows * 1000 + E)
    L = ob.lib()
    x = rng.normal(0, 1, (rows, E)).astype(np.float32)
    dout = rng.normal(0, 3, (rows, E)).astype(np.float32) if with_dout else None
    w_post = (1 + 0.1 * rng.normal(0, 1, E)).astype(np.float32) if with_dout else None
    w_pre = (1 + 0.1 * rng.normal(0, 1, E)).astype(np.float32) if with_pre else None
    os_ = 0.9 if with_os else None
    x[0, :64] = 0.0
    print(f"rows kernel rows={rows} E={E} dout={with_dout} os={with_os} pre={with_pre}", flush=True)
    r = lg.hiplib.rows_norm_q8(x, dout, w_post, os_, w_pre, eps=1e-6)
    for j in range(rows):
        xn = x[j].copy()
        if with_dout:
            ob_ = np.zeros(E, np.float32)
            L.lgo_rmsnorm(ob_, np.ascontiguousarray(dout[j]), w_post.ctypes.data, E, 1e-6, 1)
            xn = xn + ob_
            if with_os:
                xn = xn * np.float32(os_)
        h = np.zeros(E, np.float32)
        if with_pre:
            L.lgo_rmsnorm(h, np.ascontiguousarray(xn), w_pre.ctypes.data, E, 1e-6, 1)
        else:
            h = xn
        q = np.zeros(E, np.int8); d = np.zeros(E // 32, np.float32); sm = np.zeros(E // 32, np.int32)
        L.lgo_quant_q8(np.ascontiguousarray(h), E, q, d, sm)
        assert np.array_equal(r["x_out"][j].view(np.uint32), xn.view(np.uint32)), f"row {j}: residual"
        assert np.array_equal(r["h"][j].view(np.uint32), h.view(np.uint32)), f"row {j}: normed row"
        assert np.array_equal(r["xq"][j], q) and np.array_equal(r["xsum"][j], sm), f"row {j}: q8"
        assert np.array_equal(r["xd"][j].view(np.uint32), d.view(np.uint32)), f"row {j}: scales"


@pytest.mark.parametrize("rows,E,ple", [(1, 2560, 256), (5, 2560, 256), (8, 1536, 256), (4, 256, 256), (3, 3840, 256)])
def test_rows_ple_gate_kernel_matches_oracle(lg, ob, gpu_required, rows, E, ple):
    """The kernel between ffn_down and the per-layer projection in isolation: FFN residual update, inp_gate matmul on
    the q8 of the new row, gelu(.) * per-layer input, q8 -- every output the oracle's, bit for bit."""
    rng = np.random.default_rng(rows * 7 + E + ple)
    L = ob.lib()
    x = rng.normal(0, 1, (rows, E)).astype(np.float32)
    dout = rng.normal(0, 3, (rows, E)).astype(np.float32)
    w_post = (1 + 0.1 * rng.normal(0, 1, E)).astype(np.float32)
    wg = random_q4_0(rng, ple, E)
    ipl = rng.normal(0, 1, (rows, ple)).astype(np.float32)
    ipl[0, :32] = 0.0                                    # a zero group in the result: scale 0, no NaN
    print(f"rows + ple gate rows={rows} E={E} ple={ple}", flush=True)
    r = lg.hiplib.rows_ple_gate(x, dout, w_post, wg, ipl, eps=1e-6)
    xn = np.zeros_like(x)
    for j in range(rows):
        o = np.zeros(E, np.float32)
        L.lgo_rmsnorm(o, np.ascontiguousarray(dout[j]), w_post.ctypes.data, E, 1e-6, 1)
        xn[j] = x[j] + o
    assert np.array_equal(r["x_out"].view(np.uint32), xn.view(np.uint32)), "residual"
    _, _, _, gate, _ = oracle_matmul(ob, wg, E, ple, xn)
    for j in range(rows):
        g = np.array([L.lgo_gelu(float(v), 1) for v in gate[j]], np.float32) * ipl[j]
        q = np.zeros(ple, np.int8); d = np.zeros(ple // 32, np.float32); sm = np.zeros(ple // 32, np.int32)
        L.lgo_quant_q8(np.ascontiguousarray(g), ple, q, d, sm)
        assert np.array_equal(r["pq"][j], q) and np.array_equal(r["psum"][j], sm), f"row {j}: q8 of the gated row"
        assert np.array_equal(r["pd"][j].view(np.uint32), d.view(np.uint32)), f"row {j}: scales"


@pytest.mark.parametrize("rows,n_layer,ple,E", [(1, 42, 256, 2560), (5, 42, 256, 2560), (8, 3, 32, 256), (4, 5, 128, 1536)])
def test_ple_inputs_kernel_matches_oracle(lg, ob, gpu_required, rows, n_layer, ple, E):
    """The per-layer inputs of a block in isolation: (rmsnorm(proj / sqrt(E)) * w + token row * sqrt(ple)) / sqrt(2),
    the token rows read from plain q4_0 -- the oracle's values, bit for bit (the oracle's order of operations:
    oracle/lg_oracle.c, the per-layer-input part of forward_i8)."""
    rng = np.random.default_rng(rows + n_layer + ple)
    L = ob.lib()
    n_tok, w = 37, n_layer * ple
    pmp = rng.normal(0, 20, (rows, w)).astype(np.float32)
    pmp[0, :ple] = 0.0                                   # a zero row under the norm: eps only
    norm = (1 + 0.1 * rng.normal(0, 1, ple)).astype(np.float32)
    pte = random_q4_0(rng, n_tok, w)
    toks = rng.integers(0, n_tok, rows).astype(np.int32)
    toks[0] = n_tok - 1
    print(f"ple inputs rows={rows} layers={n_layer} ple={ple}", flush=True)
    got = lg.hiplib.ple_inputs(pmp, norm, pte, n_tok, toks, n_layer, ple, E, eps=1e-6)
    dw, codes = q4_0_codes(pte, n_tok, w)                # scales [n_tok, w/32], codes [n_tok, w/32, 32]
    table = ((codes.astype(np.int32) - 8).astype(np.float32) * dw.astype(np.float32)[:, :, None]).reshape(n_tok, w)
    ts, ps, r2 = np.float32(np.sqrt(np.float32(ple))), np.float32(1) / np.float32(np.sqrt(np.float32(E))), np.float32(1) / np.float32(np.sqrt(np.float32(2)))
    for j in range(rows):
        tok = table[toks[j]] * ts
        p = pmp[j] * ps
        for Lr in range(n_layer):
            seg = np.ascontiguousarray(p[Lr * ple:(Lr + 1) * ple])
            o = np.zeros(ple, np.float32)
            L.lgo_rmsnorm(o, seg, norm.ctypes.data, ple, 1e-6, 1)
            want = (o + tok[Lr * ple:(Lr + 1) * ple]) * r2
            assert np.array_equal(got[j, Lr * ple:(Lr + 1) * ple].view(np.uint32), want.view(np.uint32)), f"row {j} layer {Lr}"


def test_matmul_is_linear_in_the_scales(lg, gpu_required):
    """Size-independent property: doubling every weight scale doubles every output exactly
    (powers of two commute with rounding), negating codes around 8 negates it."""
    m, k, rows = 512, 2560, 5
    rng = np.random.default_rng(9)
    w = random_q4_0(rng, m, k).reshape(m, k // 32, 18)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    base = lg.hiplib.matmul_q4q8(w.reshape(-1), k, m, x)["out"]
    w2 = w.copy()
    d = w2[:, :, :2].copy().view(np.float16)
    w2[:, :, :2] = (d * np.float16(2)).view(np.uint8)
    assert np.array_equal(lg.hiplib.matmul_q4q8(w2.reshape(-1), k, m, x)["out"], base * 2)
    x2 = lg.hiplib.matmul_q4q8(w.reshape(-1), k, m, -x)["out"]
    assert np.array_equal(x2, -base)


def attention_f64(q, kc, vc, H, KV, hd, window, pos):
    rows, seq = q.shape[0], kc.shape[0]
    K = kc.view(np.float16).astype(np.float64).reshape(seq, KV, hd)
    V = vc.view(np.float16).astype(np.float64).reshape(seq, KV, hd)
    out = np.zeros((rows, H, hd))
    for j in range(rows):
        pj = pos + j
        start = max(0, pj - window + 1) if window else 0
        idx = [t % seq for t in range(start, pj + 1)]
        for h in range(H):
            kvh = h // (H // KV)
            s = K[idx, kvh] @ q[j, h * hd:(h + 1) * hd].astype(np.float64)
            p = np.exp(s - s.max()); p /= p.sum()
            out[j, h] = p @ V[idx, kvh]
    return out.reshape(rows, H * hd)


def oracle_attention(ob, q, kc, vc, H, KV, hd, window, pos):
    L = ob.lib()
    rows, seq, kd = q.shape[0], kc.shape[0], KV * hd
    out = np.zeros_like(q)
    for j in range(rows):
        pj = pos + j
        start = max(0, pj - window + 1) if window else 0
        for h in range(H):
            o = np.zeros(hd, np.float32)
            L.lgo_attention_f16(o, np.ascontiguousarray(q[j, h * hd:(h + 1) * hd]), kc.reshape(-1), vc.reshape(-1),
                                hd, kd, h // (H // KV), seq, start, pj, 1, 1)
            out[j, h * hd:(h + 1) * hd] = o
    return out


@pytest.mark.parametrize("seq,window,pos", [(4096 + 8, 0, 4091), (544, 512, 4091), (544, 512, 300), (4104, 0, 0), (160, 128, 31)])
def test_attention_config3(lg, ob, gpu_required, seq, window, pos):
    """8 query heads, 2 KV heads, head_dim 256, N(0,1) f16 K/V, 5 draft rows, causal among themselves:
    context 4096 global, and the 512-window ring variant (plus a short context and position 0)."""
    H, KV, hd, rows = 8, 2, 256, 5
    rng = np.random.default_rng(seq + pos)
    kc = rng.normal(0, 1, (seq, KV * hd)).astype(np.float16).view(np.uint16)
    vc = rng.normal(0, 1, (seq, KV * hd)).astype(np.float16).view(np.uint16)
    q = (rng.normal(0, 1, (rows, H * hd)) * 0.08).astype(np.float32)       # score std ~1.3, like a normed q.k
    print(f"attention seq={seq} window={window} pos={pos}", flush=True)
    out, _ = lg.hiplib.attention(q, kc, vc, H, KV, hd, window, pos)
    want = oracle_attention(ob, q, kc, vc, H, KV, hd, window, pos)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    f64 = attention_f64(q, kc, vc, H, KV, hd, window, pos)
    assert np.abs(out - f64).max() <= 1e-5 * max(1.0, np.abs(f64).max())
    # causal mask among the draft rows: row j must not see rows > j.  Change the K/V of the last
    # row's position and every earlier row's output stays bit-identical.
    k2, v2 = kc.copy(), vc.copy()
    last = (pos + rows - 1) % seq
    k2[last] = rng.normal(0, 1, KV * hd).astype(np.float16).view(np.uint16)
    v2[last] = rng.normal(0, 1, KV * hd).astype(np.float16).view(np.uint16)
    out2, _ = lg.hiplib.attention(q, k2, v2, H, KV, hd, window, pos)
    assert np.array_equal(out2[: rows - 1].view(np.uint32), out[: rows - 1].view(np.uint32))
    assert not np.array_equal(out2[rows - 1], out[rows - 1])


@pytest.mark.parametrize("H,KV,hd,rows", [(8, 2, 64, 8), (16, 8, 256, 4), (4, 4, 128, 1), (8, 2, 512, 2), (8, 8, 256, 5)])
def test_attention_other_geometries(lg, ob, gpu_required, H, KV, hd, rows):
    rng = np.random.default_rng(H * hd + rows)
    seq, window, pos = 288, 256, 700
    kc = rng.normal(0, 1, (seq, KV * hd)).astype(np.float16).view(np.uint16)
    vc = rng.normal(0, 1, (seq, KV * hd)).astype(np.float16).view(np.uint16)
    q = (rng.normal(0, 1, (rows, H * hd)) * 0.1).astype(np.float32)
    print(f"attention H={H} KV={KV} hd={hd} rows={rows}", flush=True)
    out, _ = lg.hiplib.attention(q, kc, vc, H, KV, hd, window, pos)
    want = oracle_attention(ob, q, kc, vc, H, KV, hd, window, pos)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_bad_arguments_are_refused(lg, gpu_required):
    rng = np.random.default_rng(1)
    with pytest.raises(lg.hiplib.HipError):
        lg.hiplib.matmul_q4q8(random_q4_0(rng, 8, 256), 256, 8, np.zeros((9, 256), np.float32))      # 9 rows
    with pytest.raises(lg.hiplib.HipError):
        lg.hiplib.matmul_q4q8(np.zeros(12 * 18 * 8, np.uint8), 256, 12, np.zeros((1, 256), np.float32))   # rows % 8
    with pytest.raises(lg.hiplib.HipError):
        lg.hiplib.attention(np.zeros((2, 8 * 256), np.float32), np.zeros((64, 512), np.uint16), np.zeros((64, 512), np.uint16),
                            8, 2, 256, 0, 100)                                                        # cache too short


@pytest.mark.parametrize("rows,E,FF", [(1, 2560, 10240), (3, 2560, 10240), (4, 2560, 10240), (5, 2560, 10240), (8, 2560, 10240),
                                       (2, 512, 2048), (6, 512, 2048), (5, 3840, 15360), (1, 3840, 15360)])
def test_gate_up_geglu_matches_oracle(lg, ob, gpu_required, rows, E, FF):
    """The gate/up kernels in isolation (lg_k_geglu_t for 1..3 rows, lg_k_geglu_m on the matrix cores for 4..8): the
    q8 of gelu(gate . x) * (up . x) against the oracle's matmuls, GELU and quantization, at the E4B and 12B widths
    and a small one; a row that starts with zeros and rows of different scale."""
    rng = np.random.default_rng(rows * 13 + E + FF)
    x = (rng.normal(0, 1, (rows, E)) * rng.uniform(0.3, 2.0, (rows, 1))).astype(np.float32)
    x[0, :64] = 0.0
    wg, wu = random_q4_0(rng, FF, E), random_q4_0(rng, FF, E)
    print(f"gate/up rows={rows} E={E} FF={FF}", flush=True)
    r = lg.hiplib.gate_up_geglu(x, wg, wu, FF, repeats=3)
    L = ob.lib()
    _, _, _, gate, _ = oracle_matmul(ob, wg, E, FF, x)
    _, _, _, up, _ = oracle_matmul(ob, wu, E, FF, x)
    act = np.zeros((rows, FF), np.float32)
    for j in range(rows):
        act[j] = np.array([L.lgo_gelu(float(v), 1) for v in gate[j]], np.float32) * up[j]
    aq = np.zeros((rows, FF), np.int8); ad = np.zeros((rows, FF // 32), np.float32); asum = np.zeros((rows, FF // 32), np.int32)
    for j in range(rows):
        L.lgo_quant_q8(act[j], FF, aq[j], ad[j], asum[j])
    assert np.array_equal(r["ad"].view(np.uint32), ad.view(np.uint32)), "scales"
    assert np.array_equal(r["aq"], aq), "values"
    assert np.array_equal(r["asum"], asum), "sums"
    print(f"  kernel {1e3 * r['ms']:.2f} us", flush=True)

