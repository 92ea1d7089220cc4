"""GPU parity of the prefill GEMMs against the CPU oracle, through the C ABI.

Variant (a), bf16 MFMA: against the x86 prefill definition (f32 dequantized rows, one fma chain per output,
src/kernels.rs:1998-2038) within 2e-2 (the bar for bf16 matrix-core products), and much tighter against the
same product with operands rounded to bf16 first, which is what the kernel computes."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from oxinfer_amd import HipBackend
    b = HipBackend(0)
    yield b
    b.close()


def row_err(y, ref):
    m = np.maximum(np.abs(ref).max(axis=1), 1e-30)
    return float((np.abs(y - ref).max(axis=1) / m).max())


def mlx_case(oxref, n_out, n_in, seed):
    from oxinfer_amd import synth
    wq, sc, bi = synth.mlx_q4(n_out, n_in, seed)
    rng = np.random.default_rng(seed + 1)
    sf = (sc.astype(np.uint32) << 16).view(np.float32)
    bi = synth.bf16_bits((np.float32(-8.0) * sf + 0.01 * rng.uniform(-1, 1, sc.shape)).astype(np.float32))
    q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, 64)
    return (wq, sc, bi), (q, s16, off)


@pytest.mark.parametrize("n_out,n_in", [(37, 4160), (256, 512), (200, 64), (900, 384)])  # (900 rows past 64 tokens: 112-row workgroups, a ragged last one)
def test_gemm_bf16_matches_oracle(be, oxref, n_out, n_in):
    import torch
    from oxinfer_amd import synth
    raw, (q, s16, off) = mlx_case(oxref, n_out, n_in, 7)
    w = be.upload_mlx_q4(*raw, 64, n_out, n_in)
    assert w is not None, be.last_error()
    wf = oxref.dequant_rows_q4(q, s16, off, 64, n_out, n_in)
    wb = synth.bf16_round(wf).astype(np.float64)
    for t in (1, 15, 16, 37, 64, 65, 100, 128, 150, 300, 513):  # (one token tile per wave up to 128 tokens, two past them)
        x = synth.activations(t, n_in, 100 + t, bf16=True)
        ref = oxref.gemm_quant(-1, q, s16, off, n_out, n_in, x, t)
        exact_bf16 = (x.astype(np.float64) @ wb.T).astype(np.float32)
        for xd in (torch.from_numpy(x).cuda(), torch.from_numpy(x).cuda().to(torch.bfloat16)):
            y = be.gemm(w, xd).cpu().numpy()
            assert row_err(y, ref) < 2e-2, (t, xd.dtype)
            assert row_err(y, exact_bf16) < 1e-3, (t, xd.dtype)
        yb = be.gemm(w, torch.from_numpy(x).cuda(), out_bf16=True).float().cpu().numpy()
        assert row_err(yb, ref) < 2e-2


def test_gemm_timed_records_the_kernel_and_changes_nothing(be, oxref):
    """oxhip_dev_gemm_timed: the same bytes as oxhip_dev_gemm for every variant, and the two events end up recorded in order
    (a span inside the whole call's)."""
    import torch
    from oxinfer_amd import synth
    raw, _ = mlx_case(oxref, 200, 1024, 11)
    w = be.upload_mlx_q4(*raw, 64, 200, 1024)
    data, scales = synth.fp8_e4m3(256, 512, 5)
    wf = be.upload_fp8(data, scales, 256, 512)
    for wt, variant, n_in in ((w, 0, 1024), (w, 1, 1024), (wf, 0, 512), (wf, 2, 512)):
        for t in (20, 300):  # 300 tokens of 1024 columns: K slices, so the span ends before the slice sum
            x = torch.from_numpy(synth.activations(t, n_in, 3 + t, bf16=True)).cuda().to(torch.bfloat16)
            e0, e1 = be.event(), be.event()
            o0, o1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            plain = be.gemm(wt, x, variant=variant)
            o0.record()
            timed = be.gemm(wt, x, variant=variant, events=(e0, e1))
            o1.record()
            torch.cuda.synchronize()
            assert torch.equal(plain, timed), (variant, t)
            span, whole = be.elapsed_ms(e0, e1), o0.elapsed_time(o1)
            assert 0.0 < span <= whole + 0.02, (variant, t, span, whole)  # (two clocks' readings: 20 us of slack)
            be.lib.oxhip_event_destroy(e0)
            be.lib.oxhip_event_destroy(e1)


def test_gemm_bf16_row_magnitudes_and_f32_inputs(be, oxref):
    """Token rows of magnitude 1e-3 / 1 / 300 / 2e5 (src/cuda.rs:1579-1581); f32 inputs are rounded to bf16."""
    import torch
    n_out, n_in, t = 128, 1024, 64
    raw, (q, s16, off) = mlx_case(oxref, n_out, n_in, 9)
    w = be.upload_mlx_q4(*raw, 64, n_out, n_in)
    rng = np.random.default_rng(3)
    x = (rng.normal(0, 1, (t, n_in)) * np.array([1e-3, 1.0, 300.0, 2e5])[np.arange(t) % 4][:, None]).astype(np.float32)
    ref = oxref.gemm_quant(-1, q, s16, off, n_out, n_in, x, t)
    y = be.gemm(w, torch.from_numpy(x).cuda()).cpu().numpy()
    assert row_err(y, ref) < 2e-2


GGUF_KINDS = {"Q4_0": 2, "Q8_0": 8, "Q4_K": 12, "Q5_K": 13, "Q6_K": 14, "MXFP4": 39}


def gguf_raw(name, n_out, n_in, seed):
    from oxinfer_amd import synth
    return {"Q4_0": synth.gguf_q4_0, "Q8_0": synth.gguf_q8_0, "Q4_K": synth.gguf_q4_k, "Q5_K": synth.gguf_q5_k, "Q6_K": synth.gguf_q6_k, "MXFP4": synth.gguf_mxfp4}[name](n_out, n_in, seed)


# 4352 columns = 34 steps of 128: K slices of 9 steps, so slices start inside a Q4_K super-block record; 1120 and 96
# columns (Q8_0 only): a last step of one record, and of one block
@pytest.mark.parametrize("name,n_out,n_in", [(k, n, c) for k in GGUF_KINDS for n, c in ((37, 1024), (256, 512), (200, 256), (130, 4352))]
                         + [("Q8_0", 100, 96), ("Q8_0", 64, 1120), ("Q4_0", 100, 96), ("Q4_0", 64, 1120), ("MXFP4", 64, 1120)])
def test_gemm_bf16_gguf_matches_oracle(be, oxref, name, n_out, n_in):
    """The GGUF formats on the bf16 matrix cores: within 2e-2 of the CPU's prefill product over the rows that
    dequantize_row yields (src/ggml.rs:630-793, src/kernels.rs:1998-2038), and 1e-3 of the same product with both
    operands rounded to bf16, which is what the kernel computes."""
    import torch
    from oxinfer_amd import synth
    kind = GGUF_KINDS[name]
    raw = gguf_raw(name, n_out, n_in, 17)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    assert w is not None, be.last_error()
    wb = synth.bf16_round(oxref.dequantize_rows(kind, raw, n_out, n_in)).astype(np.float64)
    for t in (1, 16, 37, 100, 150, 300, 513):
        x = synth.activations(t, n_in, 200 + t, bf16=True)
        ref = oxref.gemm_quant(kind, raw, None, None, n_out, n_in, x, t)
        exact_bf16 = (x.astype(np.float64) @ wb.T).astype(np.float32)
        for xd in (torch.from_numpy(x).cuda(), torch.from_numpy(x).cuda().to(torch.bfloat16)):
            y = be.gemm(w, xd).cpu().numpy()
            assert row_err(y, ref) < 2e-2, (t, xd.dtype)
            assert row_err(y, exact_bf16) < 1e-3, (t, xd.dtype)
    yb = be.gemm(w, torch.from_numpy(x).cuda(), out_bf16=True).float().cpu().numpy()
    assert row_err(yb, ref) < 2e-2


def test_gemm_bf16_gguf_reference_fixtures(be, oxref):
    """The reference's own block fixtures (random_blocks, src/ggml.rs:1446-1496: every bit pattern of codes and packed
    scales, signed Q6_K scales, d of either sign) through the GEMM."""
    import torch
    from oxinfer_amd import synth
    n_out, n_in, t = 48, 1024, 64
    for kind in GGUF_KINDS.values():
        raw = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 77 + kind)[0]
        w = be.upload_gguf(kind, raw, n_out, n_in)
        wb = synth.bf16_round(oxref.dequantize_rows(kind, raw, n_out, n_in)).astype(np.float64)
        x = synth.activations(t, n_in, 78, bf16=True)
        y = be.gemm(w, torch.from_numpy(x).cuda()).cpu().numpy()
        assert row_err(y, (x.astype(np.float64) @ wb.T).astype(np.float32)) < 1e-3, kind
        assert row_err(y, oxref.gemm_quant(kind, raw, None, None, n_out, n_in, x, t)) < 2e-2, kind


def test_gemm_bf16_random_shapes_match_oracle(be, oxref):
    """Seeded draws of (format, rows, columns, tokens) over the token counts where the launch changes shape (64 / 65, 128 /
    129, 256 / 257, 512 / 513: one or two token tiles per wave, one or more token blocks) and row counts around the 112-
    and 128-row workgroups, bf16 and f32 inputs, f32 and bf16 outputs: bf16 matrix-core bound (2e-2) against the oracle."""
    import torch
    from oxinfer_amd import synth
    rng = np.random.default_rng(20251)
    names = list(GGUF_KINDS) + ["MLX"]
    for it in range(21):
        name = names[it % len(names)]
        n_out = int(rng.choice([33, 112, 113, 128, 257, 600, 897]))
        t = int(rng.choice([17, 64, 65, 128, 129, 256, 257, 400, 512, 513]))
        if name == "MLX":
            n_in = int(rng.choice([64, 512, 1088, 4160]))
            wq, sc, bi = synth.mlx_q4(n_out, n_in, 100 + it)
            w = be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in)
            q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, 64)
            x = synth.activations(t, n_in, 200 + it, bf16=True)
            ref = oxref.gemm_quant(-1, q, s16, off, n_out, n_in, x, t)
        else:
            n_in = int(rng.choice([256, 768, 4352])) if name in ("Q4_K", "Q5_K", "Q6_K") else int(rng.choice([96, 544, 1120, 4096]))
            raw = gguf_raw(name, n_out, n_in, 100 + it)
            w = be.upload_gguf(GGUF_KINDS[name], raw, n_out, n_in)
            x = synth.activations(t, n_in, 200 + it, bf16=True)
            ref = oxref.gemm_quant(GGUF_KINDS[name], raw, None, None, n_out, n_in, x, t)
        assert w is not None, be.last_error()
        for xd, ob in ((torch.from_numpy(x).cuda().to(torch.bfloat16), False), (torch.from_numpy(x).cuda(), True)):
            y = be.gemm(w, xd, out_bf16=ob).float().cpu().numpy()
            assert np.isfinite(y).all() and row_err(y, ref) < 2e-2, (name, n_out, n_in, t, xd.dtype, ob)


@pytest.mark.parametrize("n_out,n_in", [(40, 640), (130, 96)])
def test_gemm_bf16_q8_matrix_matches_oracle(be, oxref, n_out, n_in):
    """QMatrix (int8 codes, f32 scale per 32; src/quant.rs:128-133) through the same kernel."""
    import torch
    from oxinfer_amd import synth
    q, sc = synth.q8_matrix(n_out, n_in, 23)
    w = be.upload_q8(q, sc, n_out, n_in)
    assert w is not None, be.last_error()
    wf = oxref.q8_dequant_rows(q, sc, n_out, n_in)
    for t in (17, 260):
        x = synth.activations(t, n_in, 300 + t, bf16=True)
        y = be.gemm(w, torch.from_numpy(x).cuda()).cpu().numpy()
        assert row_err(y, oxref.gemm_f32(wf, n_out, n_in, x, t)) < 2e-2
        assert row_err(y, (x.astype(np.float64) @ synth.bf16_round(wf).astype(np.float64).T).astype(np.float32)) < 1e-3


@pytest.mark.parametrize("n_out,n_in", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("name", list(GGUF_KINDS))
def test_gemm_gguf_full_size_sampled_rows(be, oxref, name, n_out, n_in):
    """The Llama-8B MLP shapes 512 x 4096 -> 14336 and 512 x 14336 -> 4096 (the K-sliced route) with GGUF weights: a
    sample of output rows against the oracle."""
    import torch
    from oxinfer_amd import synth
    t = 512
    kind = GGUF_KINDS[name]
    raw = gguf_raw(name, n_out, n_in, 13)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    assert w is not None, be.last_error()
    x = synth.activations(t, n_in, 14, bf16=True)
    y = be.gemm(w, torch.from_numpy(x).cuda().to(torch.bfloat16)).cpu().numpy()
    rows = np.r_[0:4, n_out // 2 - 3:n_out // 2 + 3, n_out - 4:n_out, np.random.default_rng(1).integers(0, n_out, 18)]
    rb = oxref.row_bytes(kind, n_in)
    sub = np.concatenate([raw[r * rb:(r + 1) * rb] for r in rows])
    ref = oxref.gemm_quant(kind, sub, None, None, len(rows), n_in, x, t)
    m = np.maximum(np.abs(y).max(axis=1), 1e-30)
    assert float((np.abs(y[:, rows] - ref).max(axis=1) / m).max()) < 2e-2


@pytest.mark.parametrize("n_out,n_in", [(14336, 4096), (4096, 14336)])
def test_gemm_full_size_sampled_rows(be, oxref, n_out, n_in):
    """BASELINE configs[2] variant (a) at both shapes, 512 x 4096 -> 14336 and 512 x 14336 -> 4096 (K sliced across
    workgroups, slices summed by a second kernel): a sample of output rows against the oracle."""
    import torch
    from oxinfer_amd import synth
    t = 512
    wq, sc, bi = synth.mlx_q4(n_out, n_in, 11)
    w = be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in)
    assert w is not None, be.last_error()
    x = synth.activations(t, n_in, 12, bf16=True)
    y = be.gemm(w, torch.from_numpy(x).cuda().to(torch.bfloat16)).cpu().numpy()
    rows = np.r_[0:4, n_out // 2 - 3:n_out // 2 + 3, n_out - 4:n_out, np.random.default_rng(1).integers(0, n_out, 18)]
    q, s16, off = oxref.from_mlx_q4(wq[rows], sc[rows], bi[rows], len(rows), n_in, 64)
    ref = oxref.gemm_quant(-1, q, s16, off, len(rows), n_in, x, t)
    m = np.maximum(np.abs(y).max(axis=1), 1e-30)
    assert float((np.abs(y[:, rows] - ref).max(axis=1) / m).max()) < 2e-2


def fp8_emulation(x, data, scales, oxref, rows=None):
    """What the fp8 kernel computes, in f64: activations quantized to e4m3 per token and 128 columns (scale =
    amax / 448, RNE), exact products, both scales applied per 128 x 128 block. `rows`: only these weight rows."""
    import torch
    t, n_in = x.shape
    rows = np.arange(data.shape[0]) if rows is None else np.asarray(rows)
    table = np.array([oxref.e4m3_to_f32(b) for b in range(256)], np.float64)
    wq = table[data[rows]]
    y = np.zeros((t, len(rows)))
    for kb in range(n_in // 128):
        xb = x[:, 128 * kb:128 * kb + 128]
        amax = np.abs(xb).max(axis=1, keepdims=True).astype(np.float32)
        inv = np.where(amax > 0, np.float32(448.0) / np.maximum(amax, np.float32(1e-38)), np.float32(0)).astype(np.float32)
        q = torch.from_numpy(np.clip(xb * inv, -448, 448).astype(np.float32)).to(torch.float8_e4m3fn).to(torch.float32).numpy().astype(np.float64)
        sxv = (amax / np.float32(448.0)).astype(np.float64)
        y += (q @ wq[:, 128 * kb:128 * kb + 128].T) * sxv * scales[rows // 128, kb].astype(np.float64)[None, :]
    return y.astype(np.float32)


# What e4m3 activations cost against the CPU's f32 product, from the format alone. An activation scaled into its
# tile's range moves by at most half an ulp of a 3-bit mantissa, 2^-4 of its value (2^-10 of the scaled unit in the
# subnormal range, i.e. amax * 2^-10 / 448), so every output obeys |y - ref| <= sum_k |w_k| max(2^-4 |x_k|, amax_k 2^-10 / 448).
# With roundings independent and uniform within half an ulp the error's rms is at most 2^-4 / sqrt(3) = 0.036 of the
# output's rms at any row length (signal and error both grow as sqrt(K)): the recipe's error does not average out, and
# measured it is 0.02-0.035 of a row's largest output, which is why this variant cannot meet the 2e-2 bar of the bf16
# matrix cores and is not the default.
E4M3_HALF_ULP = 2.0 ** -4
E4M3_RMS = E4M3_HALF_ULP / np.sqrt(3.0)


def fp8_activation_checks(y, ref, x, wf):
    """Asserts the two bounds above for outputs y [t, rows] against ref = x wf^T."""
    t, n_in = x.shape
    ax = np.abs(x).astype(np.float64)
    tile_amax = ax.reshape(t, n_in // 128, 128).max(axis=2, keepdims=True)
    dx = np.maximum(E4M3_HALF_ULP * ax.reshape(t, n_in // 128, 128), tile_amax * 2.0 ** -10 / 448.0).reshape(t, n_in)
    aw = np.abs(wf).astype(np.float64)
    bound = dx @ aw.T + 1e-3 * (ax @ aw.T)  # (f32 accumulation and the rounding of the scales)
    assert (np.abs(y.astype(np.float64) - ref) <= bound).all()
    rms = lambda a: float(np.sqrt(np.mean(np.square(a.astype(np.float64)))))
    assert rms(y - ref) <= E4M3_RMS * rms(ref), rms(y - ref) / rms(ref)


FP8_RECIPE_BOUND = 2e-2  # the bound BASELINE's north_star states for fp8 matrix-core outputs


def fp8_literal_recipe_status(y8, rows, ref, m):
    """The status of the literal configs[4] recipe (activations quantized to e4m3 per 1 x 128, fp8 matrix cores) at the
    config's own shape [7168, 18432] against the CPU's f32 product, by two measures, both printed:
      * the reference's own CPU-vs-accelerator report (src/bin/membench.rs:151-152): the largest absolute difference over
        the largest output magnitude of the whole product;
      * the stricter measure of this file's other tests: per token, the largest difference of its sampled outputs over
        that token's own largest output, the worst token of all.
    Rounding every activation to e4m3 leaves each with a relative error of up to 2^-4 (rms 2.6 to 2.9 %); the errors of a
    row's K products add up like the products themselves, so the error of an output stays near 2.6 % of the outputs' rms
    whatever K is, and the largest of M x N of them lands at 2 to 3 % of the largest output. Measured at M = 1024: 0.0205
    and 0.0269; at M = 32: below 0.02. The recipe therefore does NOT hold the stated 2e-2 at M = 1024 by either measure,
    which is why it is an explicit variant (OXHIP_GEMM_FP8) and the bf16 matrix cores, which do hold it, are the default
    for FP8 weights. What is asserted here is the bound it does keep (3e-2 / 4e-2); its arithmetic is pinned exactly
    (1e-3) against its own f64 definition by the callers."""
    mx = np.maximum(np.abs(y8).max(axis=1), 1e-30)
    diff = np.abs(y8[:, rows] - ref)
    per_token = float((diff.max(axis=1) / mx).max())
    whole = float(diff.max() / np.abs(y8).max())
    holds = "holds" if whole < FP8_RECIPE_BOUND else "does NOT hold"
    print(f"fp8-activation GEMM [7168, 18432] M = {m}: max abs diff / max output {whole:.4f} ({holds} the stated {FP8_RECIPE_BOUND}); "
          f"worst token by its own largest output {per_token:.4f}")
    assert whole < 3e-2, whole
    assert per_token < 4e-2, per_token


@pytest.mark.parametrize("n_out,n_in", [(200, 512), (384, 2304), (100, 128), (130, 256), (64, 640), (257, 896)])  # 1 to 18 K-blocks: every phase of the kernel's three-deep pipeline
def test_gemm_fp8_matches_oracle(be, oxref, n_out, n_in):
    import torch
    from oxinfer_amd import synth
    data, scales = synth.fp8_e4m3(n_out, n_in, 11)
    w = be.upload_fp8(data, scales, n_out, n_in)
    assert w is not None, be.last_error()
    wf = oxref.fp8_dequant_rows(data, scales, n_out, n_in)
    for t in (1, 17, 32, 100, 300):
        x = synth.activations(t, n_in, 60 + t, bf16=True)
        ref = oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t)
        emu = fp8_emulation(x, data, scales, oxref)
        for xd in (torch.from_numpy(x).cuda(), torch.from_numpy(x).cuda().to(torch.bfloat16)):
            # bf16 activations on the bf16 matrix cores (e4m3 x block scale rounded to bf16): the parity path
            y0 = be.gemm(w, xd, variant=0).cpu().numpy()
            assert row_err(y0, ref) < 2e-2, (t, xd.dtype)
            # e4m3 activations on the fp8 matrix cores: exact against its own definition (1e-3); against the CPU's
            # f32 product it is held to what the e4m3 rounding of the activations allows and no more
            y = be.gemm(w, xd, variant=2).cpu().numpy()
            assert row_err(y, emu) < 1e-3, (t, xd.dtype)
            fp8_activation_checks(y, ref, x, wf)
        yb = be.gemm(w, torch.from_numpy(x).cuda(), variant=2, out_bf16=True).float().cpu().numpy()
        assert row_err(yb, emu) < 1e-2
        yb0 = be.gemm(w, torch.from_numpy(x).cuda(), variant=0, out_bf16=True).float().cpu().numpy()
        assert row_err(yb0, ref) < 2e-2


def test_gemm_fp8_wide_scale_blocks_and_k_slices(be, oxref):
    """Scale blocks of 128 x 256: two K-steps share a scale, and with K sliced across workgroups a slice's first step
    may sit in the second half of a block. 64 x 4096 at 100 tokens runs sliced; 200 x 1024 does not."""
    import torch
    from oxinfer_amd import synth
    for n_out, n_in, t in ((64, 4096, 100), (200, 1024, 300), (64, 4096, 24)):  # 24 tokens: the skinny kernel
        data, _ = synth.fp8_e4m3(n_out, n_in, 71)
        scales = np.abs(np.random.default_rng(72).normal(0.0, 0.01, (-(-n_out // 128), n_in // 256))).astype(np.float32)
        w = be.upload_fp8(data, scales, n_out, n_in, block=(128, 256))
        assert w is not None, be.last_error()
        want = oxref.fp8_dequant_rows(data, scales, n_out, n_in, 128, 256)
        assert np.array_equal(be.dequantize(w).cpu().numpy().view(np.uint32), want.view(np.uint32))
        x = synth.activations(t, n_in, 73, bf16=True)
        ref = oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t, brows=128, bcols=256)
        y = be.gemm(w, torch.from_numpy(x).cuda().to(torch.bfloat16), variant=0).cpu().numpy()
        assert row_err(y, ref) < 2e-2, (n_out, n_in, t)
        xb, wb = x.astype(np.float64), synth.bf16_round(want).astype(np.float64)
        if t > 32:  # the GEMM rounds e4m3 x scale to bf16: tight against that product
            assert row_err(y, (xb @ wb.T).astype(np.float32)) < 1e-3, (n_out, n_in, t)
        y1 = be.decode(w, x=torch.from_numpy(x[:3]).cuda()).cpu().numpy()
        assert row_err(y1, ref[:3]) < 1e-3


def test_gemm_fp8_declines_other_shapes(be):
    import torch
    from oxinfer_amd import synth
    data, scales = synth.fp8_e4m3(64, 320, 1)
    w = be.upload_fp8(data, scales, 64, 320)
    for variant in (0, 2):
        with pytest.raises(RuntimeError):
            be.gemm(w, torch.zeros((4, 320), device="cuda"), variant=variant)


def test_gemm_fp8_config_m1024_sampled_rows(be, oxref):
    """BASELINE configs[4] at M = 1024, [7168, 18432]: sampled rows of both variants. bf16 activations on the bf16 matrix
    cores within 2e-2 of the CPU's f32 product (dequantize_rows then the f32 GEMM, src/ggml.rs:433-444); the literal
    recipe (activations to e4m3 per 1 x 128, fp8 matrix cores) within 1e-3 of its own f64 definition and within what
    the e4m3 rounding allows of the CPU product."""
    import torch
    from oxinfer_amd import synth
    n_out, n_in, m = 7168, 18432, 1024
    data, scales = synth.fp8_e4m3(n_out, n_in, 51)
    w = be.upload_fp8(data, scales, n_out, n_in)
    assert w is not None, be.last_error()
    rows = np.r_[0:3, 127:130, n_out - 3:n_out, np.random.default_rng(3).integers(0, n_out, 12)]
    x = synth.activations(m, n_in, 52, bf16=True)
    xd = torch.from_numpy(x).cuda().to(torch.bfloat16)
    wf = np.stack([oxref.fp8_dequant_rows(data, scales, n_out, n_in, r0=int(r), r1=int(r) + 1)[0] for r in rows])
    ref = oxref.gemm_f32(wf, len(rows), n_in, x, m)
    y = be.gemm(w, xd, variant=0).cpu().numpy()
    mx = np.maximum(np.abs(y).max(axis=1), 1e-30)
    assert float((np.abs(y[:, rows] - ref).max(axis=1) / mx).max()) < 2e-2
    yb = be.gemm(w, xd, variant=0, out_bf16=True).float().cpu().numpy()  # the config's output type
    assert float((np.abs(yb[:, rows] - ref).max(axis=1) / mx).max()) < 2e-2
    y8 = be.gemm(w, xd, variant=2).cpu().numpy()
    assert row_err(y8[:, rows], fp8_emulation(x, data, scales, oxref, rows)) < 1e-3
    fp8_activation_checks(y8[:, rows], ref, x, wf)
    fp8_literal_recipe_status(y8, rows, ref, m)


def test_gemm_fp8_full_size_sampled_rows(be, oxref):
    """The benchmark shape [7168, 18432] at M = 32: sampled rows against the CPU's f32 product within 2e-2 (bf16
    activations; the e4m3-activation variant within 1e-3 of its own definition and within what the e4m3 rounding of the
    activations allows of the CPU product), and the float-stored decode path (exact f32 activations) at M = 1 within 1e-3."""
    import torch
    from oxinfer_amd import synth
    n_out, n_in = 7168, 18432
    data, scales = synth.fp8_e4m3(n_out, n_in, 41)
    w = be.upload_fp8(data, scales, n_out, n_in)
    assert w is not None, be.last_error()
    rows = np.r_[0:3, 127:130, n_out - 3:n_out, np.random.default_rng(2).integers(0, n_out, 12)]
    x = synth.activations(32, n_in, 42, bf16=True)
    xd = torch.from_numpy(x).cuda().to(torch.bfloat16)
    y = be.gemm(w, xd, variant=0).cpu().numpy()
    y8 = be.gemm(w, xd, variant=2).cpu().numpy()
    # the sampled rows keep their block-scale row: dequantize them one by one
    wf = np.stack([oxref.fp8_dequant_rows(data, scales, n_out, n_in, r0=int(r), r1=int(r) + 1)[0] for r in rows])
    ref = oxref.gemm_f32(wf, len(rows), n_in, x, 32)
    m = np.maximum(np.abs(y).max(axis=1), 1e-30)
    assert float((np.abs(y[:, rows] - ref).max(axis=1) / m).max()) < 2e-2
    assert row_err(y8[:, rows], fp8_emulation(x, data, scales, oxref, rows)) < 1e-3
    fp8_activation_checks(y8[:, rows], ref, x, wf)
    fp8_literal_recipe_status(y8, rows, ref, 32)
    y1 = be.decode(w, x=torch.from_numpy(x[:1]).cuda()).cpu().numpy()
    assert float(np.abs(y1[0, rows] - ref[0]).max() / np.abs(y1).max()) < 1e-3


@pytest.mark.parametrize("n_out,n_in", [(37, 4160), (256, 512), (200, 64)])
def test_gemm_i8_block_sums_bit_exact_and_outputs(be, oxref, n_out, n_in):
    """Variant (b): the int32 block sums equal the CPU's bit for bit (src/kernels_i8gemm.rs:249-334); outputs within
    1e-3 of the oracle's restatement (same integer sums, f32 rescale in another order) and within the int8 bound
    of the exact product."""
    import torch
    from oxinfer_amd import synth
    raw, (q, s16, off) = mlx_case(oxref, n_out, n_in, 17)
    w = be.upload_mlx_q4(*raw, 64, n_out, n_in)
    assert w is not None, be.last_error()
    for t in (1, 16, 37, 64, 65, 150, 300):
        x = synth.activations(t, n_in, 200 + t, bf16=True)
        ref, isums = oxref.i8gemm_q4(q, s16, off, 64, n_out, n_in, x, t, want_isums=True)
        for xd in (torch.from_numpy(x).cuda(), torch.from_numpy(x).cuda().to(torch.bfloat16)):
            got = be.gemm_isums(w, xd).cpu().numpy()
            assert np.array_equal(got, isums), (t, xd.dtype)
            y = be.gemm(w, xd, variant=1).cpu().numpy()
            assert row_err(y, ref) < 1e-3, (t, xd.dtype)
        yb = be.gemm(w, torch.from_numpy(x).cuda(), variant=1, out_bf16=True).float().cpu().numpy()
        assert row_err(yb, ref) < 1e-2
        exact = oxref.gemm_quant(-1, q, s16, off, n_out, n_in, x, t)
        if n_in >= 512:
            assert row_err(y, exact) < 3e-2


def test_gemm_i8_extremes_bit_exact(be, oxref):
    """Nibbles 0, 8 and 15 against activations at the block maximum (src/kernels_x86.rs:829, :893)."""
    import torch
    from oxinfer_amd import synth
    n_out, n_in, t = 32, 256, 20
    rng = np.random.default_rng(5)
    wq = rng.choice(np.array([0x00000000, 0x88888888, 0xFFFFFFFF, 0xF0F0F0F0, 0x0F8F0F8F], np.uint32), (n_out, n_in // 8))
    sc = synth.bf16_bits(np.full((n_out, n_in // 64), 2.0 ** -6, np.float32))
    bi = synth.bf16_bits(np.full((n_out, n_in // 64), -8 * 2.0 ** -6, np.float32))
    q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, 64)
    w = be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in)
    x = rng.choice(np.array([-4.0, 4.0], np.float32), (t, n_in))
    ref, isums = oxref.i8gemm_q4(q, s16, off, 64, n_out, n_in, x, t, want_isums=True)
    assert np.array_equal(be.gemm_isums(w, torch.from_numpy(x).cuda()).cpu().numpy(), isums)
    assert row_err(be.gemm(w, torch.from_numpy(x).cuda(), variant=1).cpu().numpy(), ref) < 1e-5


@pytest.mark.parametrize("n_out,n_in", [(4096, 14336), (14336, 4096)])
def test_gemm_i8_full_size_sampled_rows(be, oxref, n_out, n_in):
    """BASELINE configs[2] variant (b) at both of its shapes, M = 512: the int32 block sums of sampled rows equal the
    CPU's bit for bit (all 512 tokens, every block of the row), outputs within 1e-3 of the oracle's restatement of
    kernels_i8gemm and within the int8 bound of the exact product."""
    import torch
    from oxinfer_amd import synth
    t = 512
    wq, sc, bi = synth.mlx_q4(n_out, n_in, 21)
    w = be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in)
    assert w is not None, be.last_error()
    x = synth.activations(t, n_in, 22, bf16=True)
    xd = torch.from_numpy(x).cuda().to(torch.bfloat16)
    y = be.gemm(w, xd, variant=1).cpu().numpy()
    rows = np.r_[0:4, n_out // 2 - 2:n_out // 2 + 2, n_out - 4:n_out, np.random.default_rng(1).integers(0, n_out, 12)]
    q, s16, off = oxref.from_mlx_q4(wq[rows], sc[rows], bi[rows], len(rows), n_in, 64)
    ref, isums = oxref.i8gemm_q4(q, s16, off, 64, len(rows), n_in, x, t, want_isums=True)
    m = np.maximum(np.abs(y).max(axis=1), 1e-30)
    assert float((np.abs(y[:, rows] - ref).max(axis=1) / m).max()) < 1e-3
    exact = oxref.gemm_quant(-1, q, s16, off, len(rows), n_in, x, t)
    assert float((np.abs(y[:, rows] - exact).max(axis=1) / m).max()) < 2e-2
    got = be.gemm_isums(w, xd)  # [t, n_out, n_in / 32] on the device; only the sampled rows come back
    got = got[:, torch.from_numpy(rows).cuda(), :].cpu().numpy()
    assert np.array_equal(got, isums)
