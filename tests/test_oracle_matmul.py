"""Pins of the oracle's matmul-level functions (CPU only): every check is against something the oracle's own
formula does not supply: integer brute force in numpy, f64 definitions built from already-pinned pieces
(quantize_act, decode_i8, dequantize), cases where f32 arithmetic is exact, and the invariants the reference's own
tests state (src/kernels.rs:2484-2488, src/ggml.rs:1712-1747, :1904, src/cuda.rs:1684-1685, :2145-2179)."""
import numpy as np
import pytest

Q8_0, Q4_K, Q5_K, Q6_K, MXFP4 = 8, 12, 13, 14, 39


def row_err(y, ref):
    m = np.maximum(np.abs(ref).max(axis=-1, keepdims=True), 1e-30)
    return float((np.abs(y - ref) / m).max())


def bf16_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def q4_codes(q, n_out, n_in):
    """Planar Q4 bytes -> centered codes [n_out, n_in] (byte j of a block: element j low, j + 16 high)."""
    b = q.reshape(n_out, n_in // 32, 16).astype(np.int32)
    return np.concatenate([(b & 15) - 8, (b >> 4) - 8], axis=2).reshape(n_out, n_in)


def mlx_case(oxref, n_out, n_in, seed, reference_like=True):
    from oxinfer_amd import synth
    wq, sc, bi = synth.mlx_q4(n_out, n_in, seed)
    if reference_like:  # the reference's test distribution: biases -8 s + 0.01 u (src/kernels.rs:2470-2480)
        rng = np.random.default_rng(seed + 1)
        bi = synth.bf16_bits((np.float32(-8.0) * bf16_f32(sc) + 0.01 * rng.uniform(-1, 1, sc.shape)).astype(np.float32))
    return (wq, sc, bi), oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, 64)


def test_from_mlx_q4_regroups_nibbles_and_keeps_the_values(oxref):
    n_out, n_in = 9, 256
    (wq, sc, bi), (q, s16, off) = mlx_case(oxref, n_out, n_in, 3)
    # nibble e of a row is (word[e / 8] >> 4 (e % 8)) & 15, independent of the oracle
    nib = ((wq.reshape(n_out, n_in // 8, 1) >> (4 * np.arange(8, dtype=np.uint32))) & 15).reshape(n_out, n_in).astype(np.int32)
    assert np.array_equal(q4_codes(q, n_out, n_in), nib - 8)
    # scale: f16 of the bf16 scale; offset: bf16 of b + 8 s
    assert np.array_equal(s16.reshape(n_out, -1)[:, ::2], bf16_f32(sc).astype(np.float16).view(np.uint16).reshape(n_out, -1))
    mlx = oxref.mlx_dequant_rows(wq, sc, bi, n_out, n_in)
    direct = (bf16_f32(sc).astype(np.float64).repeat(64, axis=-1).reshape(n_out, n_in) * nib
              + bf16_f32(bi).astype(np.float64).repeat(64, axis=-1).reshape(n_out, n_in))
    assert np.abs(mlx - direct).max() < 1e-6
    deq = oxref.dequant_rows_q4(q, s16, off, 64, n_out, n_in)
    assert np.abs(deq - mlx).max() < 2e-4          # the reference's bound (src/kernels.rs:2484-2488)
    # exact when the scale is f16-representable and b + 8 s is bf16-representable: b = -8 s, power-of-two s
    sc2 = np.full_like(sc, 0x3C00 >> 0)           # bf16 bits 0x3C00 = 2^-7
    from oxinfer_amd import synth
    bi2 = synth.bf16_bits((np.float32(-8.0) * bf16_f32(sc2)).astype(np.float32))
    q2, s2, o2 = oxref.from_mlx_q4(wq, sc2, bi2, n_out, n_in, 64)
    assert np.array_equal(oxref.dequant_rows_q4(q2, s2, o2, 64, n_out, n_in), oxref.mlx_dequant_rows(wq, sc2, bi2, n_out, n_in))


def q4_f64(oxref, q, s16, off, n_out, n_in, x, t):
    """f64 definition of the Q4 decode product from pinned pieces: exact integer block sums times f16 scale times
    activation scale, plus offsets times the exact activation sums."""
    xq, xs, _, fs, _ = oxref.quantize_act(x, t, n_in)
    codes = q4_codes(q, n_out, n_in).reshape(n_out, n_in // 32, 32).astype(np.int64)
    isum = np.einsum("rbk,tbk->trb", codes, xq.reshape(t, n_in // 32, 32).astype(np.int64))
    d = s16.view(np.float16).astype(np.float64).reshape(n_out, n_in // 32)
    y = np.einsum("trb,rb,tb->tr", isum.astype(np.float64), d, xs.reshape(t, -1).astype(np.float64))
    if off is not None:
        gs = fs.reshape(t, n_in // 64, 2).astype(np.float64).sum(axis=2)
        y = y + np.einsum("rg,tg->tr", bf16_f32(off).astype(np.float64).reshape(n_out, n_in // 64), gs)
    return y, isum


@pytest.mark.parametrize("t", [1, 3, 8])
def test_q4_decode_against_integer_brute_force_and_f64(oxref, t):
    from oxinfer_amd import synth
    n_out, n_in = 48, 512
    _, (q, s16, off) = mlx_case(oxref, n_out, n_in, 5)
    x = synth.activations(t, n_in, 6)
    y, isums = oxref.q4_decode(q, s16, off, 64, n_out, n_in, x, t, want_isums=True)
    ref, isum = q4_f64(oxref, q, s16, off, n_out, n_in, x, t)
    assert np.array_equal(isums, isum)
    assert row_err(y, ref) < 1e-4
    ya = oxref.q4_decode(q, s16, off, 64, n_out, n_in, x, t, avx2=True, threads=2)
    assert row_err(ya, ref) < 1e-4
    # against the exact product of the dequantized weights: the int8 activations' bound (src/ggml.rs:1904)
    exact = x.astype(np.float64) @ oxref.dequant_rows_q4(q, s16, off, 64, n_out, n_in).astype(np.float64).T
    assert row_err(y, exact) < 3e-2
    # the int8 GEMM restatement shares the integer sums and the value
    yg, ig = oxref.i8gemm_q4(q, s16, off, 64, n_out, n_in, x, t, want_isums=True)
    assert np.array_equal(ig, isum)
    assert row_err(yg, ref) < 1e-4


@pytest.mark.parametrize("t", [1, 3])
def test_q8_matrix_against_integer_brute_force_and_f64(oxref, t):
    """QMatrix (src/quant.rs:128-133, src/kernels.rs:1156-1167): block sums against numpy integers, the product against
    the f64 definition from the pinned quantize_act, the dequantized rows exactly (an int8 times an f32 is one rounding)."""
    from oxinfer_amd import synth
    n_out, n_in = 40, 384
    q, sc = synth.q8_matrix(n_out, n_in, 9)
    x = synth.activations(t, n_in, 10)
    y, isums = oxref.q8_decode(q, sc, n_out, n_in, x, t, want_isums=True)
    xq, xs, _, _, _ = oxref.quantize_act(x, t, n_in)
    isum = (xq.reshape(t, 1, n_in // 32, 32).astype(np.int64) * q.reshape(1, n_out, n_in // 32, 32).astype(np.int64)).sum(axis=3)
    assert np.array_equal(isums, isum)
    ref = (isum * sc.astype(np.float64)[None] * xs.reshape(t, 1, -1).astype(np.float64)).sum(axis=2)
    assert row_err(y, ref) < 1e-4
    deq = oxref.q8_dequant_rows(q, sc, n_out, n_in)
    assert np.array_equal(deq, (q.astype(np.float32).reshape(n_out, -1, 32) * sc[:, :, None]).reshape(n_out, n_in))
    assert np.array_equal(oxref.q8_dequant_rows(q, sc, n_out, n_in, r0=3, r1=5), deq[3:5])
    assert row_err(y, x.astype(np.float64) @ deq.astype(np.float64).T) < 3e-2  # the int8 activations' bound (src/ggml.rs:1904)


def gguf_f64(oxref, kind, data, n_out, n_in, x, t):
    bs, ts = oxref.block_size(kind), oxref.type_size(kind)
    xq, xs, _, _, hs = oxref.quantize_act(x, t, n_in)
    nb = n_in // bs
    y = np.zeros((t, n_out))
    isums = np.zeros((t, n_out, n_in // 16), np.int64)
    raw = data.reshape(n_out, nb, ts)
    for r in range(n_out):
        for b in range(nb):
            q, s, m, has_min = oxref.decode_i8(kind, raw[r, b])
            e0 = b * bs
            xi = xq[:, e0:e0 + bs].reshape(t, bs // 16, 16).astype(np.int64)
            ig = (xi * q.reshape(1, bs // 16, 16).astype(np.int64)).sum(axis=2)          # [t, bs/16]
            isums[:, r, e0 // 16:e0 // 16 + bs // 16] = ig
            xsg = xs.reshape(t, -1)[:, (e0 // 32):(e0 // 32) + bs // 32].repeat(2, axis=1).astype(np.float64)
            y[:, r] += (ig * s.astype(np.float64)[None, :] * xsg).sum(axis=1)
            if has_min:
                y[:, r] += (m.astype(np.float64)[None, :] * hs.reshape(t, -1)[:, e0 // 16:e0 // 16 + bs // 16]).sum(axis=1)
    return y, isums


@pytest.mark.parametrize("kind", [Q8_0, Q4_K, Q5_K, Q6_K, MXFP4])
def test_gguf_decode_against_integer_brute_force_and_f64(oxref, kind):
    from oxinfer_amd import synth
    n_out, n_in, t = 12, 512, 3
    data, _ = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 77 + kind)
    x = synth.activations(t, n_in, 8)
    y, isums = oxref.gguf_decode(kind, data, n_out, n_in, x, t, want_isums=True)
    ref, ig = gguf_f64(oxref, kind, data, n_out, n_in, x, t)
    assert np.array_equal(isums, ig)
    assert row_err(y, ref) < 1e-4                                       # src/ggml.rs:1712-1747
    ya = oxref.gguf_decode(kind, data, n_out, n_in, x, t, avx2=True, threads=2)
    assert np.array_equal(ya.view(np.uint32), y.view(np.uint32))        # the AVX2 kernels give the portable bits
    exact = x.astype(np.float64) @ oxref.dequantize_rows(kind, data, n_out, n_in).astype(np.float64).T
    assert row_err(y, exact) < 3e-2                                      # src/ggml.rs:1904


def test_decode_is_exact_when_f32_arithmetic_is(oxref):
    """Power-of-two scales and integer activations whose block maximum is 127 * 2^k: every f32 product and sum is
    exact, so the result must equal the integer computation bit for bit (src/kernels_x86.rs:799-803)."""
    rng = np.random.default_rng(4)
    n_out, n_in, t = 16, 256, 2
    xi = rng.integers(-127, 128, (t, n_in))
    xi[:, ::32] = 127
    x = (xi * 2.0 ** -5).astype(np.float32)
    codes = rng.integers(-127, 128, (n_out, n_in // 32, 32)).astype(np.int8)
    blocks = np.zeros((n_out, n_in // 32, 34), np.uint8)
    blocks[:, :, :2] = np.array([2.0 ** -6], np.float16).view(np.uint8)
    blocks[:, :, 2:] = codes.view(np.uint8)
    y = oxref.gguf_decode(Q8_0, blocks.reshape(-1), n_out, n_in, x, t)
    exact = (xi.astype(np.int64) @ codes.reshape(n_out, n_in).astype(np.int64).T) * 2.0 ** -11
    assert np.array_equal(y, exact.astype(np.float32))
    # extremes: every weight and activation at +-127 (src/kernels_x86.rs:829, :893)
    blocks[:, :, 2:] = np.int8(-127).view(np.uint8)
    x = np.full((1, n_in), 127.0, np.float32)
    y = oxref.gguf_decode(Q8_0, blocks.reshape(-1), n_out, n_in, x, 1)
    assert np.array_equal(y, np.full((1, n_out), -127.0 * 127.0 * n_in * 2.0 ** -6, np.float32))


def test_prefill_gemm_is_the_f64_product_of_the_dequantized_rows(oxref):
    from oxinfer_amd import synth
    n_out, n_in, t = 40, 512, 19
    _, (q, s16, off) = mlx_case(oxref, n_out, n_in, 9)
    x = synth.activations(t, n_in, 10)
    wf = oxref.dequant_rows_q4(q, s16, off, 64, n_out, n_in)
    ref = x.astype(np.float64) @ wf.astype(np.float64).T
    assert row_err(oxref.gemm_quant(-1, q, s16, off, n_out, n_in, x, t), ref) < 1e-4      # src/cuda.rs:1684-1685
    assert row_err(oxref.gemm_f32(wf, n_out, n_in, x, t), ref) < 1e-4
    for kind in (Q8_0, Q4_K, Q5_K, Q6_K, MXFP4):
        data, _ = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 5)
        ref = x.astype(np.float64) @ oxref.dequantize_rows(kind, data, n_out, n_in).astype(np.float64).T
        assert row_err(oxref.gemm_quant(kind, data, None, None, n_out, n_in, x, t), ref) < 1e-4
    data, scales = synth.fp8_e4m3(n_out, n_in, 6)
    ref = x.astype(np.float64) @ oxref.fp8_dequant_rows(data, scales, n_out, n_in).astype(np.float64).T
    assert row_err(oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t), ref) < 1e-4
    # small integers: one fma chain per output is exact, whatever the order
    wi = np.random.default_rng(1).integers(-8, 9, (n_out, n_in)).astype(np.float32)
    xi = np.random.default_rng(2).integers(-8, 9, (t, n_in)).astype(np.float32)
    assert np.array_equal(oxref.gemm_f32(wi, n_out, n_in, xi, t), xi @ wi.T)


def test_fast_exp_and_silu(oxref):
    xs = np.concatenate([np.linspace(-87, 88, 3001), [0.0, -0.0, 1e-8, -100.0, 100.0]]).astype(np.float32)
    got = np.array([oxref.fast_exp(v) for v in xs], np.float64)
    ref = np.exp(np.clip(xs.astype(np.float64), -87, 88))
    assert np.abs(got / ref - 1).max() < 3e-7       # Cody-Waite + degree-6 polynomial (src/kernels.rs:2225-2231)
    assert oxref.fast_exp(0.0) == 1.0
    g = np.linspace(-20, 20, 801).astype(np.float32)
    u = np.linspace(-3, 3, 801).astype(np.float32)
    ref = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.abs(oxref.silu_mul(g, u) - ref).max() < 1e-5 * np.abs(ref).max()


def test_route_top_k_is_softmax_topk_renormalized(oxref):
    rng = np.random.default_rng(0)
    for trial in range(20):
        logits = rng.normal(0, 1, 128).astype(np.float32)
        if trial == 0:
            logits[5] = logits[60] = logits.max() + 1          # tie: lower index first
        idx, w = oxref.route_top_k(logits, 8)
        order = sorted(range(128), key=lambda i: (-float(logits[i]), i))[:8]
        assert list(idx) == order
        p = np.exp(logits.astype(np.float64) - logits.max())
        p /= p.sum()
        assert np.allclose(w, p[order] / p[order].sum(), rtol=1e-5)
        assert abs(float(w.sum()) - 1) < 1e-6
    idx, _ = oxref.route_top_k(np.full(16, 0.5, np.float32), 4)
    assert list(idx) == [0, 1, 2, 3]


def test_moe_against_the_f64_definition(oxref):
    """Tiny shapes, brute force (src/cuda.rs:2145-2179): y[t] += sum_j w_j * Down_e (silu(G_e x) * (U_e x))."""
    from oxinfer_amd import synth
    ne, h, inter, k, t = 6, 128, 64, 2, 9
    gu = [mlx_case(oxref, 2 * inter, h, 100 + e, False)[1] for e in range(ne)]
    dn = [mlx_case(oxref, h, inter, 200 + e, False)[1] for e in range(ne)]
    x = synth.activations(t, h, 1)
    logits = synth.router_logits(t, ne, 2)
    idx = np.zeros((t, k), np.uint32)
    w = np.zeros((t, k), np.float32)
    for i in range(t):
        idx[i], w[i] = oxref.route_top_k(logits[i], k)
    y0 = np.zeros((t, h), np.float32)   # (the call adds into y; a non-zero start is covered below)
    ref = y0.astype(np.float64).copy()
    for i in range(t):
        for j in range(k):
            e = int(idx[i, j])
            wg = oxref.dequant_rows_q4(*gu[e], 64, 2 * inter, h).astype(np.float64)
            wd = oxref.dequant_rows_q4(*dn[e], 64, h, inter).astype(np.float64)
            g = wg @ x[i].astype(np.float64)
            a = g[:inter] / (1 + np.exp(-g[:inter])) * g[inter:]
            ref[i] += float(w[i, j]) * (wd @ a)
    grouped = oxref.moe_q4(gu, dn, 64, h, inter, x, t, idx, w, y0, decode_path=False)
    assert row_err(grouped - y0, ref - y0) < 1e-4
    # the decode path (int8 activations at both matmuls): the composition of the pinned kernels, bit for bit,
    # and within the int8 bound of the definition
    dec = oxref.moe_q4(gu, dn, 64, h, inter, x, t, idx, w, y0, decode_path=True)
    comp = y0.copy()
    for i in range(t):
        for j in range(k):
            e = int(idx[i, j])
            g = oxref.q4_decode(*gu[e], 64, 2 * inter, h, x[i], 1)[0]
            o = oxref.q4_decode(*dn[e], 64, h, inter, oxref.silu_mul(g[:inter], g[inter:]), 1)[0]
            comp[i] = comp[i] + w[i, j] * o
    assert np.array_equal(dec.view(np.uint32), comp.view(np.uint32))
    assert row_err(dec - y0, ref - y0) < 3e-2
    y1 = synth.activations(t, h, 3)
    dec1 = oxref.moe_q4(gu, dn, 64, h, inter, x, t, idx, w, y1, decode_path=True)
    assert np.abs(dec1 - (y1 + dec)).max() < 1e-5
    # the baseline's AVX2-scheduled decode pass is the same computation up to the f32 order inside the kernels
    fast = oxref.moe_q4(gu, dn, 64, h, inter, x, t, idx, w, y0, decode_path=True, avx2=True, threads=4)
    assert row_err(fast - y0, dec - y0) < 1e-5
    one = oxref.moe_q4(gu, dn, 64, h, inter, x[:1], 1, idx[:1], w[:1], y0[:1], decode_path=True, avx2=True, threads=3)
    assert row_err(one, dec[:1] - y0[:1]) < 1e-5


def test_gated_activations_match_the_library_definitions(oxref):
    """Act::apply / Act::scalar (src/moe.rs:18-46): SiLU, GELU-tanh (gelu_pytorch_tanh, src/kernels.rs:2233-2239) and
    DeepSeek V4's clamped SiLU against torch's silu, gelu(approximate="tanh") and clamp evaluated in f64: a dropped clamp,
    a clamp on the wrong side, a wrong constant or gate and up swapped each fail one of these."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(3)
    g = np.concatenate([rng.normal(0, 3, 4000), np.linspace(-30, 30, 301), [0.0, -0.0, 7.0, -7.0, 6.999, 7.001]]).astype(np.float32)
    u = np.concatenate([rng.normal(0, 4, 4000), np.linspace(12, -12, 301), [1.0, -1.0, 9.0, -9.0, 7.0, -7.0]]).astype(np.float32)
    g64, u64 = torch.from_numpy(g).double(), torch.from_numpy(u).double()
    lim = 7.0
    refs = {0: F.silu(g64) * u64, 1: F.gelu(g64, approximate="tanh") * u64,
            2: F.silu(torch.clamp(g64, max=lim)) * torch.clamp(u64, -lim, lim)}
    for kind, ref in refs.items():
        ref = ref.numpy()
        tol = 2e-6 * np.maximum(np.abs(ref), 1e-3)
        got = oxref.act_apply(kind, lim, g, u)
        assert (np.abs(got - ref) <= tol).all(), kind
        sc = np.array([oxref.act_scalar(kind, lim, a, b) for a, b in zip(g[:500], u[:500])], np.float64)
        assert (np.abs(sc - ref[:500]) <= tol[:500]).all(), kind
    # kind 0 is silu_mul bit for bit (the MoE decode path's composition rests on it)
    assert np.array_equal(oxref.act_apply(0, 0.0, g, u).view(np.uint32), oxref.silu_mul(g, u).view(np.uint32))
    # the clamp really bites: an up value past the limit and a gate past it change the result
    assert oxref.act_scalar(2, 1.0, 0.5, 5.0) == oxref.act_scalar(0, 0.0, 0.5, 1.0)
    assert oxref.act_scalar(2, 1.0, 5.0, 0.5) == oxref.act_scalar(0, 0.0, 1.0, 0.5)
    assert oxref.act_scalar(2, 1.0, -5.0, 0.5) == oxref.act_scalar(0, 0.0, -5.0, 0.5)  # the gate is clamped from above only


@pytest.mark.parametrize("act,param", [(1, 0.0), (2, 0.1)])
@pytest.mark.parametrize("split", [False, True])
def test_moe_activation_kinds_and_split_experts_against_f64(oxref, act, param, split):
    """MoeAct::GeluTanh / SiluClamp(l) and split gate / up experts (src/gpu.rs:35-54, :206-216) against the f64 definition
    y[t] += sum_j w_j * Down_e(act(G_e x) * (U_e x)), brute force on tiny shapes; fused and split experts holding the
    same rows give the same bits."""
    import torch
    import torch.nn.functional as F
    from oxinfer_amd import synth
    ne, h, inter, k, t = 5, 128, 64, 2, 9
    g_ = [mlx_case(oxref, inter, h, 300 + e, False)[1] for e in range(ne)]
    u_ = [mlx_case(oxref, inter, h, 400 + e, False)[1] for e in range(ne)]
    dn = [mlx_case(oxref, h, inter, 500 + e, False)[1] for e in range(ne)]
    fused = [tuple(np.concatenate([a, b]) for a, b in zip(g_[e], u_[e])) for e in range(ne)]
    x = synth.activations(t, h, 11)
    logits = synth.router_logits(t, ne, 12)
    idx = np.zeros((t, k), np.uint32)
    w = np.zeros((t, k), np.float32)
    for i in range(t):
        idx[i], w[i] = oxref.route_top_k(logits[i], k)
    y0 = np.zeros((t, h), np.float32)

    def act64(g, u):
        g, u = torch.from_numpy(g), torch.from_numpy(u)
        if act == 1:
            return (F.gelu(g, approximate="tanh") * u).numpy()
        return (F.silu(torch.clamp(g, max=param)) * torch.clamp(u, -param, param)).numpy()
    ref = y0.astype(np.float64).copy()
    clamped = 0
    for i in range(t):
        for j in range(k):
            e = int(idx[i, j])
            wg = oxref.dequant_rows_q4(*g_[e], 64, inter, h).astype(np.float64)
            wu = oxref.dequant_rows_q4(*u_[e], 64, inter, h).astype(np.float64)
            wd = oxref.dequant_rows_q4(*dn[e], 64, h, inter).astype(np.float64)
            g, u = wg @ x[i].astype(np.float64), wu @ x[i].astype(np.float64)
            clamped += int((np.abs(u) > param).sum() + (g > param).sum())
            ref[i] += float(w[i, j]) * (wd @ act64(g, u))
    if act == 2:
        assert clamped > 50  # the limit is inside the data's range
    kw = dict(up=u_, act=act, act_param=param) if split else dict(act=act, act_param=param)
    first = g_ if split else fused
    grouped = oxref.moe_q4(first, dn, 64, h, inter, x, t, idx, w, y0, decode_path=False, **kw)
    assert row_err(grouped, ref) < 1e-4
    dec = oxref.moe_q4(first, dn, 64, h, inter, x, t, idx, w, y0, decode_path=True, **kw)
    assert row_err(dec, ref) < 3e-2
    if split:
        for path in (False, True):
            a = oxref.moe_q4(g_, dn, 64, h, inter, x, t, idx, w, y0, decode_path=path, up=u_, act=act, act_param=param)
            b = oxref.moe_q4(fused, dn, 64, h, inter, x, t, idx, w, y0, decode_path=path, act=act, act_param=param)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), path
