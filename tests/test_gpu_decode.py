"""GPU parity of the decode path against the CPU oracle, through the C ABI.

Bars: activation quantization, dequantized weights and the int32 accumulators bit-exact; matmul
outputs within 1e-3 of the oracle's (f32 accumulation), measured like the reference's `row_err`
(src/cuda.rs:1583-1592): worst error of a token row over that row's largest reference value.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4 = 2, 8, 12, 13, 14, 39
TOL = 1e-3


@pytest.fixture(scope="module")
def be():
    import torch
    assert torch.cuda.is_available(), "the gpu tests need a device"
    from oxinfer_amd import HipBackend
    b = HipBackend(0)
    yield b
    b.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def row_err(y, ref):
    m = np.maximum(np.abs(ref).max(axis=1), 1e-30)
    return float((np.abs(y - ref).max(axis=1) / m).max())


def lcg_input(t, n, seed, oxref):
    """Token rows of very different magnitudes (src/cuda.rs:1579-1581), values from the reference's LCG."""
    v, _ = oxref.lcg_stream(seed, t * n)
    x = ((v >> 7).astype(np.float64) / float(1 << 24) - 0.5).astype(np.float32).reshape(t, n)
    mags = np.array([1e-3, 1.0, 300.0, 2e5], np.float32)
    return x * mags[np.arange(t) % 4][:, None]


def test_probe_lists_the_device(be):
    """The GpuKind::Hip probe (beside platform::gpu::cuda::probe, src/platform.rs:446-482)."""
    from oxinfer_amd import hip
    gpus = hip.probe()
    assert len(gpus) >= 1 and gpus[0]["index"] == 0 and gpus[0]["arch"] == "gfx950" and gpus[0]["usable"]
    assert gpus[0]["memory_bytes"] > 200 * 2 ** 30 and gpus[0]["name"] and "gfx950" in gpus[0]["driver"]


def test_name_and_wants(be):
    assert be.name() == "hip (gfx950)"
    assert be.wants(4096, 4096, 1) and not be.wants(64, 40, 1) and not be.wants(64, 64, 0)


def test_quantize_act_bit_exact(be, oxref):
    t, n = 7, 4 * 256 + 96
    x = lcg_input(t, n, 7, oxref)
    x[0, 32:64] = 0.0          # an all-zero block
    x[0, 64 + 3] = 1e-30
    x[1, :32] = -0.0           # an all -0.0 block: the sums stay -0.0
    x[2, 5] = 3.0e38
    x[3, 96:128] = np.float32(0.5)  # ties: every product is 127.0 or rounds half away
    x[3, 97] = np.float32(0.5 * 64.5 / 127.0)
    xa = be.quantize_act(dev(x))
    q, scales, sums, fsums, hsums = oxref.quantize_act(x, t, n)
    assert np.array_equal(xa.q.cpu().numpy(), q)
    assert np.array_equal(xa.scales.cpu().numpy().view(np.uint32), scales.view(np.uint32))
    assert np.array_equal(xa.sums.cpu().numpy(), sums)
    assert np.array_equal(xa.fsums.cpu().numpy().view(np.uint32), fsums.view(np.uint32))
    assert np.array_equal(xa.hsums.cpu().numpy().view(np.uint32), hsums.view(np.uint32))
    s16 = q.astype(np.int32).reshape(t, n // 16, 16).sum(axis=2)
    assert np.array_equal(xa.sums16.cpu().numpy(), s16)


def test_quantize_act_batch_bit_exact(be, oxref):
    """Several matrices in one launch: every output equal to the reference's, as for one at a time."""
    from oxinfer_amd.hip import QAct
    shapes = [(1, 4096), (8, 4096), (3, 96), (1, 14336), (5, 32)] * 4  # 20 jobs: two launches
    xs = [lcg_input(t, n, 200 + i, oxref) for i, (t, n) in enumerate(shapes)]
    xd = [dev(x) for x in xs]
    outs = [QAct(t, n, "cuda") for t, n in shapes]
    be.quantize_act_batch(be.quantize_jobs(list(zip(xd, outs))))
    for x, (t, n), xa in zip(xs, shapes, outs):
        q, scales, sums, fsums, hsums = oxref.quantize_act(x, t, n)
        assert np.array_equal(xa.q.cpu().numpy(), q)
        assert np.array_equal(xa.scales.cpu().numpy().view(np.uint32), scales.view(np.uint32))
        assert np.array_equal(xa.sums.cpu().numpy(), sums)
        assert np.array_equal(xa.fsums.cpu().numpy().view(np.uint32), fsums.view(np.uint32))
        assert np.array_equal(xa.hsums.cpu().numpy().view(np.uint32), hsums.view(np.uint32))
        assert np.array_equal(xa.sums16.cpu().numpy(), q.astype(np.int32).reshape(t, n // 16, 16).sum(axis=2))


with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_hashes.json")) as _f:  # src/ggml.rs:1547-1577
    REF_HASHES = {e["ggml_type"]: int(e["fnv1a64"], 16) for e in json.load(_f)["hashes"].values()}


@pytest.mark.parametrize("kind", [Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4])
def test_gguf_dequant_matches_ggml_hash_on_device(be, oxref, kind):
    """The device dequantizer reproduces the reference's golden hashes (src/ggml.rs:1547-1577)."""
    raw, _ = oxref.random_blocks(kind, 1024 // oxref.block_size(kind), 1000 + kind)
    w = be.upload_gguf(kind, raw, 1, 1024)
    assert w is not None, be.last_error()
    y = be.dequantize(w).cpu().numpy()
    assert oxref.fnv1a_f32(y) == REF_HASHES[kind]


@pytest.mark.parametrize("kind", [Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4])
def test_gguf_dequant_and_isums_bit_exact(be, oxref, kind):
    n_out, n_in, t = 37, 3 * 256, 5
    raw, seed = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 13 + kind)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    assert w is not None, be.last_error()
    want = oxref.dequantize_rows(kind, raw, n_out, n_in)
    got = be.dequantize(w).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    part = be.dequantize(w, 5, 9).cpu().numpy()
    assert np.array_equal(part.view(np.uint32), want[5:9].view(np.uint32))
    x = lcg_input(t, n_in, seed, oxref)
    xa = be.quantize_act(dev(x))
    _, isums = oxref.gguf_decode(kind, raw, n_out, n_in, x, t, want_isums=True)
    if kind == Q6_K:  # per 16, as the CPU forms them
        assert np.array_equal(be.isums(w, xa, 16).cpu().numpy(), isums)
    else:  # the matrix-core kernel forms whole blocks of 32: the two halves' sums added, exactly
        assert np.array_equal(be.isums(w, xa, 32).cpu().numpy(), isums.reshape(t, n_out, -1, 2).sum(axis=3))


@pytest.mark.parametrize("kind", [Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4])
@pytest.mark.parametrize("t", [1, 2, 3, 5, 8, 11, 16])
def test_gguf_decode_matches_oracle(be, oxref, kind, t):
    # rows not a multiple of the wave's row group; Q8_0 with a block count that is not a multiple of 4
    n_out = 21
    n_in = 3 * 256 + 96 if kind == Q8_0 else 3 * 256
    raw, seed = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 77 + kind)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    v, _ = oxref.lcg_stream(seed, t * n_in)
    x = ((v % 2001).astype(np.float32) / np.float32(1000.0) - np.float32(1.0)).reshape(t, n_in)  # src/ggml.rs:1887
    ref = oxref.gguf_decode(kind, raw, n_out, n_in, x, t)
    y = be.decode(w, xa=be.quantize_act(dev(x))).cpu().numpy()
    assert row_err(y, ref) < TOL
    # batch invariance (src/ggml.rs:1829-1848): every token's row equals a one-token pass, bit for bit
    for c in range(t):
        y1 = be.decode(w, xa=be.quantize_act(dev(x[c:c + 1]))).cpu().numpy()
        assert np.array_equal(y1[0].view(np.uint32), y[c].view(np.uint32)), c


@pytest.mark.parametrize("kind", [Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4])
def test_gguf_decode_row_magnitudes(be, oxref, kind):
    n_out, n_in, t = 64, 4096, 4
    raw, seed = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 5 + kind)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    x = lcg_input(t, n_in, seed, oxref)
    ref = oxref.gguf_decode(kind, raw, n_out, n_in, x, t)
    y = be.decode(w, xa=be.quantize_act(dev(x))).cpu().numpy()
    assert row_err(y, ref) < TOL


def test_mlx_q4_repack_dequant_isums_decode(be, oxref):
    from oxinfer_amd import synth
    n_out, n_in, group = 37, 4160, 64  # src/kernels.rs:2458-2502 uses n_in = 4160
    wq, sc, bi = synth.mlx_q4(n_out, n_in, 3, group)
    # scales 0.002..0.012 and biases -8 s + 0.01 u as the reference's test draws them, plus scales in the
    # f16 subnormal range and ones f16 cannot hold exactly
    rng = np.random.default_rng(4)
    sc = synth.bf16_bits((0.002 + 0.01 * np.abs(rng.uniform(-1, 1, sc.shape))).astype(np.float32))
    sc[0, :4] = synth.bf16_bits(np.array([3e-6, 6.1e-5, 1e-7, 2.0 ** -17], np.float32))
    sf = (sc.astype(np.uint32) << 16).view(np.float32)
    bi = synth.bf16_bits((np.float32(-8.0) * sf + 0.01 * rng.uniform(-1, 1, sc.shape)).astype(np.float32))
    q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, group)
    want = oxref.dequant_rows_q4(q, s16, off, group, n_out, n_in)
    for w in (be.upload_mlx_q4(wq, sc, bi, group, n_out, n_in), be.upload_q4(q, s16, off, group, n_out, n_in)):
        assert w is not None, be.last_error()
        got = be.dequantize(w).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # invariant of the repack (src/kernels.rs:2484-2488)
        assert np.abs(got - oxref.mlx_dequant_rows(wq, sc, bi, n_out, n_in)).max() < 2e-4
        for t in (1, 2, 3, 5, 9):
            x = lcg_input(t, n_in, 100 + t, oxref)
            ref, isums = oxref.q4_decode(q, s16, off, group, n_out, n_in, x, t, want_isums=True)
            xa = be.quantize_act(dev(x))
            assert np.array_equal(be.isums(w, xa, 32).cpu().numpy(), isums)
            y = be.decode(w, xa=xa).cpu().numpy()
            assert row_err(y, ref) < TOL


@pytest.mark.parametrize("t", [1, 3, 8, 13])
def test_q8_matrix_dequant_isums_decode(be, oxref, t):
    """QMatrix (WeightRef::Q8, src/quant.rs:128-133): dequantized rows and int32 block sums bit for bit, the product
    within 1e-3 of the CPU's (src/kernels.rs:1156-1167); a block count that is not a multiple of the step, ragged rows,
    extreme codes in one row, and one job of a shared launch next to a GGUF one."""
    from oxinfer_amd import synth
    n_out, n_in = 45, 1024 + 96
    q, sc = synth.q8_matrix(n_out, n_in, 31)
    q[0, :] = 127
    q[1, :] = -128
    w = be.upload_q8(q, sc, n_out, n_in)
    assert w is not None, be.last_error()
    got = be.dequantize(w).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oxref.q8_dequant_rows(q, sc, n_out, n_in).view(np.uint32))
    x = synth.activations(t, n_in, 32 + t)
    x[0, :] = 3.0  # all activation codes 127 in token 0: the largest sums of a block
    ref, isum = oxref.q8_decode(q, sc, n_out, n_in, x, t, want_isums=True)
    xa = be.quantize_act(dev(x))
    assert np.array_equal(be.isums(w, xa, 32).cpu().numpy(), isum)
    y = be.decode(w, xa=xa).cpu().numpy()
    assert row_err(y, ref) < TOL
    for c in range(min(t, 3)):  # batch invariance
        y1 = be.decode(w, xa=be.quantize_act(dev(x[c:c + 1]))).cpu().numpy()
        assert np.array_equal(y1[0].view(np.uint32), y[c].view(np.uint32)), c
    if t <= 8:  # the host entry point: Q8 and Q8_0 jobs of one call share a launch
        raw = synth.gguf_q8_0(24, n_in, 33)
        w2 = be.upload_gguf(Q8_0, raw, 24, n_in)
        ya, yb = np.full((t, n_out), np.nan, np.float32), np.full((t, 24), np.nan, np.float32)
        assert be.matmul(x, t, n_in, [(w, ya), (w2, yb)]), be.last_error()
        assert np.array_equal(ya.view(np.uint32), y.view(np.uint32))
        assert row_err(yb, oxref.gguf_decode(Q8_0, raw, 24, n_in, x, t)) < TOL


def test_q4_without_offsets_and_mixed_scales(be, oxref):
    """A plain Q4_0-layout matrix (no offsets; src/quant.rs:457-513) keeps one scale per block of 32."""
    n_out, n_in = 10, 512
    rng = np.random.default_rng(9)
    q = rng.integers(0, 256, (n_out, n_in // 2), dtype=np.uint8)
    sc = np.abs(rng.normal(0, 0.01, (n_out, n_in // 32))).astype(np.float16).view(np.uint16)
    x = lcg_input(3, n_in, 1, oxref)
    for off, group in ((None, 0), (synth_offsets(n_out, n_in, 64), 64)):
        w = be.upload_q4(q, sc, off, group, n_out, n_in)
        assert w is not None, be.last_error()
        want = oxref.dequant_rows_q4(q, sc, off, group or 32, n_out, n_in)
        assert np.array_equal(be.dequantize(w).cpu().numpy().view(np.uint32), want.view(np.uint32))
        ref = oxref.q4_decode(q, sc, off, group or 32, n_out, n_in, x, 3)
        y = be.decode(w, xa=be.quantize_act(dev(x))).cpu().numpy()
        assert row_err(y, ref) < TOL


def synth_offsets(n_out, n_in, group):
    from oxinfer_amd import synth
    rng = np.random.default_rng(10)
    return synth.bf16_bits(rng.normal(0, 0.05, (n_out, n_in // group)).astype(np.float32))


def test_q4_integer_extremes(be, oxref):
    """Nibbles 0 / 8 / 15 against +-127 activations with power-of-two scales: every f32 operation is exact,
    so the outputs compare bit for bit (src/kernels_x86.rs:880-906)."""
    n_out, n_in = 4, 96
    for nib, xv in ((15, 127), (15, -127), (0, 127), (0, -127), (8, 127)):
        q = np.full((n_out, n_in // 2), nib | (nib << 4), np.uint8)
        sc = np.array([[0.5, 1.0, 2.0]] * n_out, np.float16).view(np.uint16)
        x = np.full((1, n_in), np.float32(xv))
        ref, isums = oxref.q4_decode(q, sc, None, 32, n_out, n_in, x, 1, want_isums=True)
        w = be.upload_q4(q, sc, None, 0, n_out, n_in)
        xa = be.quantize_act(dev(x))
        assert np.array_equal(be.isums(w, xa, 32).cpu().numpy(), isums)
        assert isums[0, 0, 0] == (nib - 8) * 127 * 32 * (1 if xv > 0 else -1)
        y = be.decode(w, xa=xa).cpu().numpy()
        assert np.array_equal(y.view(np.uint32), ref.view(np.uint32))


def test_fp8_dequant_and_decode(be, oxref):
    from oxinfer_amd import synth
    n_out, n_in = 200, 512
    data, scales = synth.fp8_e4m3(n_out, n_in, 11)
    data[0, :256] = np.arange(256, dtype=np.uint8)  # every byte value, NaNs included
    w = be.upload_fp8(data, scales, n_out, n_in)
    assert w is not None, be.last_error()
    want = oxref.fp8_dequant_rows(data, scales, n_out, n_in)
    got = be.dequantize(w).cpu().numpy()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan) and nan.sum() == 2
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    for t in (1, 3, 4, 5, 7, 8, 9, 16):  # the activation fragments are packed for 4, 8 or 16 tokens
        x = synth.activations(t, n_in, 12 + t, bf16=True)
        ref = oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t)
        # float-stored rows take the f32 path for every t (src/kernels.rs:1802)
        y = be.decode(w, x=dev(x)).cpu().numpy()
        assert np.isnan(y[:, 0]).all() and np.isnan(ref[:, 0]).all()  # row 0 holds the NaN bytes
        assert row_err(y[:, 1:], ref[:, 1:]) < TOL


def test_fp8_decode_on_a_fresh_stream_takes_the_one_pass_kernel(be, oxref):
    """A stream's decode scratch comes into being on first need, and FP8's one-pass decode kernel keeps its packed rows
    there: the first FP8 decode on a new stream must bring the scratch with it (device memory in use grows) and give the
    rows of the host surface's product, which runs the same kernel over the context's scratch, bit for bit. Without the
    scratch the call would fall back to the plain kernel: right within tolerance, three times slower, other bits."""
    import torch
    from oxinfer_amd import synth
    n_out, n_in, t = 512, 2048, 1
    data, scales = synth.fp8_e4m3(n_out, n_in, 91)
    w = be.upload_fp8(data, scales, n_out, n_in)
    x = synth.activations(t, n_in, 92, bf16=True)
    host = np.empty((t, n_out), np.float32)
    assert be.matmul(x, t, n_in, [(w, host)]), be.last_error()
    assert row_err(host, oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t)) < TOL
    xd = dev(x)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(side):
        y = be.decode(w, x=xd)
    side.synchronize()
    assert torch.cuda.mem_get_info()[0] <= free0 - (8 << 20), "the stream's decode scratch was not allocated"
    assert np.array_equal(y.cpu().numpy().view(np.uint32), host.view(np.uint32))
    assert be.stream_release(side.cuda_stream)


def test_fp8_rows_scale_blocks(oxref, be):
    """Scale rows change every 128 weight rows; the row-1 dequant check above would miss a wrong row index."""
    from oxinfer_amd import synth
    n_out, n_in = 260, 256
    data, scales = synth.fp8_e4m3(n_out, n_in, 21)
    w = be.upload_fp8(data, scales, n_out, n_in)
    x = synth.activations(2, n_in, 22, bf16=True)
    ref = oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, 2)
    assert row_err(be.decode(w, x=dev(x)).cpu().numpy(), ref) < TOL


@pytest.mark.parametrize("n_out,n_in", [(200, 512), (37, 1064), (4096, 4096)])
def test_bf16_weights(be, oxref, n_out, n_in):
    """WeightRef::Bf16 (src/gpu.rs:16): bf16 rows widen exactly (bf16_to_f32, src/kernels.rs:16-18) and the product
    accumulates in f32 over f32 activations (matmul_multi, src/kernels.rs:59-192): dequantized rows bit for bit, outputs
    within 1e-3 of the CPU's f32 product and of the f64 one, at every token count of the decode entry point, through
    the host surface past it, and declined where the reference's layout cannot be met."""
    from oxinfer_amd import synth
    rng = np.random.default_rng(n_out + n_in)
    wf = rng.normal(0.0, 0.02, (n_out, n_in)).astype(np.float32)
    wf[0, :8] = [0.0, -0.0, 1.0, -1.0, 3.3895314e38, -3.3895314e38, 1e-40, 9.1835e-41]  # the extremes of bf16, subnormals
    wf = synth.bf16_round(wf)
    wbits = (wf.view(np.uint32) >> 16).astype(np.uint16)
    w = be.upload_bf16(wbits, n_out, n_in)
    assert w is not None, be.last_error()
    got = be.dequantize(w, 0, min(n_out, 64)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), wf[:64].view(np.uint32))
    wf[0, :8] = 0.0  # (keep the products finite for the comparisons below)
    wbits = (wf.view(np.uint32) >> 16).astype(np.uint16)
    w = be.upload_bf16(wbits, n_out, n_in)
    for t in ((1, 2, 3, 4, 5, 7, 16) if n_out < 4096 else (1, 8)):
        x = lcg_input(t, n_in, 60 + t, oxref)
        y = be.decode(w, x=dev(x)).cpu().numpy()
        assert row_err(y, oxref.gemm_f32(wf, n_out, n_in, x, t)) < TOL
        assert row_err(y, (x.astype(np.float64) @ wf.astype(np.float64).T).astype(np.float32)) < TOL
    if n_out < 4096:
        t = 21  # the host surface walks longer batches 16 tokens at a time
        x = lcg_input(t, n_in, 99, oxref)
        yh = np.full((t, n_out), np.nan, np.float32)
        if n_in % 32 == 0:
            assert be.matmul(x, t, n_in, [(w, yh)]), be.last_error()
            assert row_err(yh, oxref.gemm_f32(wf, n_out, n_in, x, t)) < TOL
        else:
            assert not be.matmul(x, t, n_in, [(w, yh)]) and np.isnan(yh).all()
    assert be.upload_bf16(np.zeros((3, 12), np.uint16), 3, 12) is None  # rows must be whole 16-byte units


@pytest.mark.parametrize("n_out,n_in,scaled", [(37, 192, "none"), (64, 1024, "global"), (48, 4160, "blocks"), (200, 14336, "global")])
def test_nvfp4_upload_dequant_decode_gemm(be, oxref, n_out, n_in, scaled):
    """NVFP4 (ggml's blocks of 64 with an unsigned E4M3 scale per 16, src/ggml.rs:79-83, :936-947), float-stored like FP8
    (is_float, :219-224): dequantized rows bit-exact (with and without the matrix's scales on top, :420-432), decode at 1
    to 16 tokens within 1e-3 of the CPU's f32 product of those rows, the bf16 matrix-core GEMM past 16 tokens within 2e-2,
    and the host surface (Backend::matmul) routing both."""
    import torch
    from oxinfer_amd import synth
    raw, g = synth.gguf_nvfp4(n_out, n_in, 9000 + n_in)
    if scaled == "none":
        scales, block = None, None
    elif scaled == "global":
        scales, block = np.array([g], np.float32), (n_out, n_in)
    else:  # blocks of 16 rows x 128 columns, every scale different
        block = (16, 128)
        scales = np.abs(np.random.default_rng(5).normal(0.5, 0.2, (-(-n_out // 16), -(-n_in // 128)))).astype(np.float32) + 0.1
    w = be.upload_nvfp4(raw, n_out, n_in, scales, block)
    assert w is not None, be.last_error()
    assert w.bytes <= (n_out + 15) // 16 * 16 * (n_in + 127) // 128 * 128 * 0.5625 + 256 + (0 if scales is None else scales.size * 4 + 256)
    br, bc = block or (n_out, n_in)
    want = oxref.gguf_dequant_rows_scaled(oxref.NVFP4, raw, scales, n_out, n_in, br, bc)
    assert np.array_equal(be.dequantize(w).cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert np.array_equal(be.dequantize(w, 5, 21).cpu().numpy().view(np.uint32), want[5:21].view(np.uint32))
    for t in (1, 2, 3, 4, 7, 16):
        x = lcg_input(t, n_in, 77 + t, oxref)
        ref = oxref.gemm_quant(oxref.NVFP4, raw, scales, None, n_out, n_in, x, t, brows=br, bcols=bc)
        y = be.decode(w, x=dev(x)).cpu().numpy()
        assert row_err(y, ref) < TOL, (t, row_err(y, ref))
        yh = np.full((t, n_out), np.nan, np.float32)
        assert be.matmul(x, t, n_in, [(w, yh)]), be.last_error()
        assert np.array_equal(yh.view(np.uint32), y.view(np.uint32))
    for t in (17, 40, 130):
        x = synth.activations(t, n_in, 88 + t)
        ref = oxref.gemm_quant(oxref.NVFP4, raw, scales, None, n_out, n_in, x, t, brows=br, bcols=bc)
        y = be.gemm(w, dev(x), variant=0).cpu().numpy()
        assert row_err(y, ref) < 2e-2, (t, row_err(y, ref))
        # both operands rounded to bf16, as the kernel rounds them: tight against that product
        xb, wb = synth.bf16_round(x).astype(np.float64), synth.bf16_round(want).astype(np.float64)
        assert row_err(y, (xb @ wb.T).astype(np.float32)) < 1e-3, t
        yh = np.full((t, n_out), np.nan, np.float32)
        assert be.matmul(x, t, n_in, [(w, yh)]), be.last_error()
        assert row_err(yh, ref) < 2e-2
    # rows that are not whole blocks of 64, and scale blocks that cut through a tile: declined at upload
    assert be.lib.oxhip_upload(be.ctx, be.desc_gguf(40, raw[:36], 1, 32)[0]) is None and "64" in be.last_error()
    assert be.upload_nvfp4(raw, n_out, n_in, np.ones(n_out * (-(-n_in // 64)), np.float32), (1, 64)) is None


def test_host_matmul_matches_device_path_and_declines(be, oxref):
    from oxinfer_amd import synth
    n_in = 512
    raws = [(k, n, oxref.random_blocks(k, n * n_in // oxref.block_size(k), 31 + k)[0]) for k, n in ((Q4_K, 24), (Q6_K, 8), (Q8_0, 40))]
    ws = [be.upload_gguf(k, raw, n, n_in) for k, n, raw in raws]
    # up to 8 tokens the Q4_K and Q8_0 jobs share a launch; 9 to 16 run the decode kernels; past 16 every format takes
    # the prefill GEMM on the exact rows, as the CPU does past its decode limit (src/kernels.rs:1774-1847): bf16 matrix
    # cores, 2e-2 of the f32 product
    for t in (1, 3, 9, 16, 17, 40):
        x = lcg_input(t, n_in, 40 + t, oxref)
        ys = [np.full((t, n), np.nan, np.float32) for _, n, _ in raws]
        assert be.matmul(x, t, n_in, list(zip(ws, ys))), be.last_error()
        for (k, n, raw), y in zip(raws, ys):
            if t <= 16:
                assert row_err(y, oxref.gguf_decode(k, raw, n, n_in, x, t)) < TOL
            else:  # (a token has as few as 8 outputs here, all of which may cancel: the bound is on the terms' size)
                wf = oxref.dequantize_rows(k, raw, n, n_in)
                terms = (np.abs(x).astype(np.float64) @ np.abs(wf).astype(np.float64).T).max(axis=1)
                ref = oxref.gemm_quant(k, raw, None, None, n, n_in, x, t)
                assert float((np.abs(y - ref).max(axis=1) / terms).max()) < 2e-2 / 8
                xb, wb = synth.bf16_round(x).astype(np.float64), synth.bf16_round(wf).astype(np.float64)
                assert row_err(y, (xb @ wb.T).astype(np.float32)) < TOL
    # and so do MLX 4-bit and FP8 weights
    t, n_out = 40, 48
    wq, sc, bi = synth.mlx_q4(n_out, n_in, 3)
    q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, 64)
    data, scales = synth.fp8_e4m3(n_out, n_in, 4)
    wm, wf = be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in), be.upload_fp8(data, scales, n_out, n_in)
    x = synth.activations(t, n_in, 5)
    ym, yf = np.full((t, n_out), np.nan, np.float32), np.full((t, n_out), np.nan, np.float32)
    assert be.matmul(x, t, n_in, [(wm, ym), (wf, yf)]), be.last_error()
    assert row_err(ym, oxref.gemm_quant(-1, q, s16, off, n_out, n_in, x, t)) < 2e-2
    assert row_err(yf, oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t)) < 2e-2
    # a job whose weight has another n_in: declined, and nothing is written
    other = be.upload_gguf(Q8_0, oxref.random_blocks(Q8_0, 8 * 64 // 32, 1)[0], 8, 64)
    y0, y1 = np.full((1, 24), np.nan, np.float32), np.full((1, 8), np.nan, np.float32)
    assert not be.matmul(lcg_input(1, n_in, 1, oxref), 1, n_in, [(ws[0], y0), (other, y1)])
    assert np.isnan(y0).all() and np.isnan(y1).all() and "job 1" in be.last_error()
    assert "calls" in be.stats()


def test_upload_declines(be):
    assert be.upload_gguf(10, np.zeros(84, np.uint8), 1, 256) is None  # Q2_K: no device kernels
    assert "no device kernels" in be.last_error()
    assert be.upload_gguf(Q5_K, np.zeros(176, np.uint8), 1, 384) is None and "256" in be.last_error()
    assert be.upload_gguf(Q4_K, np.zeros(144, np.uint8), 1, 256) is not None


@pytest.mark.parametrize("kind,n_out,n_in", [(Q8_0, 14336, 4096), (Q8_0, 4096, 14336), (Q4_K, 14336, 4096), (Q4_K, 4096, 14336), (Q6_K, 14336, 4096), (Q6_K, 4096, 14336), (Q5_K, 4096, 14336), (MXFP4, 14336, 4096)])
def test_full_size_rows_against_oracle(be, oxref, kind, n_out, n_in):
    """The benchmark shapes: a sample of rows of the full-size product against the oracle, plus properties
    that hold at any size: the all-ones-activation row sums and batch invariance."""
    from oxinfer_amd import synth
    gen = {Q8_0: synth.gguf_q8_0, Q4_K: synth.gguf_q4_k, Q5_K: synth.gguf_q5_k, Q6_K: synth.gguf_q6_k, MXFP4: synth.gguf_mxfp4}[kind]
    raw = gen(n_out, n_in, 1000 + kind)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    assert w is not None, be.last_error()
    rb = oxref.row_bytes(kind, n_in)
    t = 8
    x = synth.activations(t, n_in, 2000 + kind)
    y = be.decode(w, xa=be.quantize_act(dev(x))).cpu().numpy()
    rows = np.r_[0:8, n_out // 2 - 3:n_out // 2 + 3, n_out - 8:n_out, np.random.default_rng(1).integers(0, n_out, 44)]
    sub = np.concatenate([raw[r * rb:(r + 1) * rb] for r in rows])
    ref = oxref.gguf_decode(kind, sub, len(rows), n_in, x, t)
    m = np.maximum(np.abs(y).max(axis=1), 1e-30)
    assert float((np.abs(y[:, rows] - ref).max(axis=1) / m).max()) < TOL
    y1 = be.decode(w, xa=be.quantize_act(dev(x[3:4]))).cpu().numpy()
    assert np.array_equal(y1[0].view(np.uint32), y[3].view(np.uint32))


def test_mlx_gemv_config_shape_against_oracle(be, oxref):
    """BASELINE configs[0] at its full size: MLX 4-bit g64 [4096, 4096] (bias = -8 scale), one token of N(0, 1). Every
    row: the int32 block sums bit for bit, the outputs within 1e-3 of the CPU decode product (from_mlx_q4 then the Q4
    decode kernel, src/quant.rs:518-563, src/kernels_x86.rs:447-474), the dequantized rows bit for bit; and the same
    rows from the shared launch of a layer's four 4096 x 4096 matmuls."""
    import torch
    from oxinfer_amd import synth
    n = k = 4096
    wq, sc, bi = synth.mlx_q4(n, k, 1)
    w = be.upload_mlx_q4(wq, sc, bi, 64, n, k)
    assert w is not None, be.last_error()
    q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n, k, 64)
    assert not off.any()  # bias = -8 scale: the offsets b + 8 s vanish exactly
    got = be.dequantize(w, 1000, 1064).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oxref.dequant_rows_q4(q, s16, off, 64, n, k, 1000, 1064).view(np.uint32))
    x = synth.activations(1, k, 2)
    xa = be.quantize_act(dev(x))
    ref, isums = oxref.q4_decode(q, s16, off, 64, n, k, x, 1, want_isums=True)
    assert np.array_equal(be.isums(w, xa, 32).cpu().numpy(), isums)
    y = be.decode(w, xa=xa).cpu().numpy()
    assert row_err(y, ref) < TOL
    # against the exact f32 product over the dequantized rows: the int8 activations' own bound (src/ggml.rs:1904)
    exact = (x.astype(np.float64) @ oxref.dequant_rows_q4(q, s16, off, 64, n, k).astype(np.float64).T).astype(np.float32)
    assert row_err(y, exact) < 3e-2
    ws = [w] + [be.upload_mlx_q4(*synth.mlx_q4(n, k, 10 + i), 64, n, k) for i in range(3)]
    ys = [torch.full((1, n), float("nan"), dtype=torch.float32, device="cuda") for _ in ws]
    be.decode_batch(be.decode_jobs([(wi, xa, None, 1, yi, None, None) for wi, yi in zip(ws, ys)]))
    torch.cuda.synchronize()
    assert np.array_equal(ys[0].cpu().numpy().view(np.uint32), y.view(np.uint32))
    for wi, yi in zip(ws[1:], ys[1:]):
        assert np.array_equal(yi.cpu().numpy().view(np.uint32), be.decode(wi, xa=xa).cpu().numpy().view(np.uint32))


def test_decode_batch_shares_a_launch_and_keeps_the_bits(be, oxref):
    """Independent matmuls handed over as one batch (the jobs of one Backend::matmul call, src/gpu.rs:160) run in one
    launch; every job's rows are bit-identical to its own launch, whatever its neighbours, formats and batch sizes."""
    import torch
    from oxinfer_amd import synth
    cases = [(Q8_0, 208, 512, 1), (Q4_K, 96, 1024, 8), (Q8_0, 64, 2048, 3), (Q4_K, 176, 512, 2), ("mlx", 80, 640, 5),
             (Q6_K, 48, 512, 2), (Q4_K, 33, 256, 4), ("mlx", 128, 128, 8),
             (Q8_0, 48, 14336, 8), (Q4_K, 32, 14336, 1), (Q6_K, 16, 14336, 5),  # these three slice K across workgroups
             (Q5_K, 72, 768, 7), (Q5_K, 40, 14336, 1), (MXFP4, 56, 1120, 6),
             (Q4_0, 48, 1056, 8), (Q4_0, 24, 14336, 2), ("q8", 88, 608, 3), ("q8", 16, 14336, 8)]
    jobs, alone = [], []
    for i, (kind, n_out, n_in, t) in enumerate(cases):
        if kind == "mlx":
            w = be.upload_mlx_q4(*synth.mlx_q4(n_out, n_in, 70 + i), 64, n_out, n_in)
        elif kind == "q8":
            w = be.upload_q8(*synth.q8_matrix(n_out, n_in, 70 + i), n_out, n_in)
        else:
            raw, _ = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 80 + i)
            w = be.upload_gguf(kind, raw, n_out, n_in)
        assert w is not None, be.last_error()
        xa = be.quantize_act(torch.from_numpy(synth.activations(t, n_in, 90 + i)).cuda())
        alone.append(be.decode(w, xa=xa).cpu().numpy())
        y = torch.full((t, n_out), float("nan"), dtype=torch.float32, device="cuda")
        jobs.append((w, xa, None, t, y, None, None))
    for order in (list(range(len(cases))), list(reversed(range(len(cases)))), [1, 3, 6], [4], [8, 0, 9, 10, 2], [11, 5, 12], [13, 4], [13],
                  [14, 16, 15, 17], [15], [17, 0]):  # (every format set on its own and beside others)
        for i in order:
            jobs[i][4].fill_(float("nan"))
        be.decode_batch(be.decode_jobs([jobs[i] for i in order]))
        torch.cuda.synchronize()
        for i in order:
            got = jobs[i][4].cpu().numpy()
            assert np.array_equal(got.view(np.uint32), alone[i].view(np.uint32)), (order, i, cases[i])


def test_decode_batch_of_full_size_jobs_keeps_the_bits(be, oxref):
    """A shared launch with work for every CU several times over maps runs to waves the fat way (a workgroup takes
    several K slices, a wave several runs): the benchmark's eight matmuls (Q8_0 and Q4_K, 4096 -> 14336 and 14336 -> 4096,
    1 and 8 tokens) and four Q6_K ones as one batch give every job the rows of its own launch bit for bit, and a sample
    of those rows is the CPU's within 1e-3."""
    import torch
    from oxinfer_amd import synth
    gens = {Q8_0: synth.gguf_q8_0, Q4_K: synth.gguf_q4_k, Q6_K: synth.gguf_q6_k}
    shapes = [(14336, 4096), (4096, 14336)]
    raws = {(kind, n): gens[kind](n, k, 40 + kind + i) for kind in gens for i, (n, k) in enumerate(shapes)}
    ws = {(kind, n): be.upload_gguf(kind, raws[(kind, n)], n, k) for kind in gens for n, k in shapes}
    jobs, alone, meta = [], [], []
    for kind in (Q8_0, Q4_K, Q6_K):
        for n, k in shapes:
            for t in (1, 8):
                xs = synth.activations(t, k, 50 + t)
                xa = be.quantize_act(torch.from_numpy(xs).cuda())
                alone.append(be.decode(ws[(kind, n)], xa=xa).cpu().numpy())
                jobs.append((ws[(kind, n)], xa, None, t, torch.full((t, n), float("nan"), dtype=torch.float32, device="cuda"), None, None))
                meta.append((kind, n, k, t, xs))
    for order in (list(range(8)), list(range(12)), [11, 3, 8, 0, 9, 5, 10, 6, 1, 7, 2, 4]):
        for i in order:
            jobs[i][4].fill_(float("nan"))
        be.decode_batch(be.decode_jobs([jobs[i] for i in order]))
        torch.cuda.synchronize()
        for i in order:
            assert np.array_equal(jobs[i][4].cpu().numpy().view(np.uint32), alone[i].view(np.uint32)), (order, i, meta[i][:4])
    rng = np.random.default_rng(5)
    for i in (1, 3, 5, 7, 9, 11):  # the eight-token jobs: 24 sampled rows each against the CPU's decode
        kind, n, k, t, xs = meta[i]
        rows = np.sort(rng.choice(n, 24, replace=False))
        rb = oxref.row_bytes(kind, k)
        sub = np.ascontiguousarray(np.asarray(raws[(kind, n)], np.uint8).reshape(n, rb)[rows])
        want = oxref.gguf_decode(kind, sub, len(rows), k, xs, t)
        assert row_err(alone[i][:, rows], want) < TOL, meta[i][:4]


def test_decode_batch_events(be, oxref):
    """Timing events of oxhip_dev_decode_batch: a lone job's launch and a shared launch carry them themselves, jobs of
    other kernels and split runs get them recorded around; either way the interval is positive and the rows unchanged."""
    import torch
    from oxinfer_amd import synth
    rng = np.random.default_rng(31)
    raw8, _ = oxref.random_blocks(Q8_0, 96 * 1024 // 32, 5)
    w8 = be.upload_gguf(Q8_0, raw8, 96, 1024)
    rawk, _ = oxref.random_blocks(Q4_K, 64 * 2048 // 256, 6)
    wk = be.upload_gguf(Q4_K, rawk, 64, 2048)
    q = rng.integers(0, 256, (10, 512 // 2), dtype=np.uint8)
    sc = np.abs(rng.normal(0, 0.01, (10, 512 // 32))).astype(np.float16).view(np.uint16)
    w4 = be.upload_q4(q, sc, None, 0, 10, 512)  # the planar kernel, not the matrix-core one
    assert w8 is not None and wk is not None and w4 is not None, be.last_error()
    xs = {1024: be.quantize_act(torch.from_numpy(synth.activations(13, 1024, 1)).cuda()),
          2048: be.quantize_act(torch.from_numpy(synth.activations(13, 2048, 2)).cuda()),
          512: be.quantize_act(torch.from_numpy(synth.activations(13, 512, 3)).cuda())}
    cases = [(w8, 1024, 96), (wk, 2048, 64), (w4, 512, 10)]
    for t in (1, 8, 13):  # 13: two launches for the matrix-core kernels
        plain = [be.decode(w, xa=xs[k], t=t).cpu().numpy() for w, k, _ in cases]
        # each job alone, with its own pair of events
        for (w, k, n), want in zip(cases, plain):
            y = torch.full((t, n), float("nan"), dtype=torch.float32, device="cuda")
            e0, e1 = be.event(), be.event()
            be.decode_batch(be.decode_jobs([(w, xs[k], None, t, y, e0, e1)]))
            torch.cuda.synchronize()
            assert be.elapsed_ms(e0, e1) > 0.0
            assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
        # all three in one call (the first two share a launch when t <= 8), events on the first and the last job
        ys = [torch.full((t, n), float("nan"), dtype=torch.float32, device="cuda") for _, _, n in cases]
        e0, e1, e2, e3 = be.event(), be.event(), be.event(), be.event()
        be.decode_batch(be.decode_jobs([(cases[0][0], xs[1024], None, t, ys[0], e0, None), (cases[1][0], xs[2048], None, t, ys[1], None, e1),
                                        (cases[2][0], xs[512], None, t, ys[2], e2, e3)]))
        torch.cuda.synchronize()
        assert be.elapsed_ms(e0, e1) > 0.0 and be.elapsed_ms(e2, e3) > 0.0 and be.elapsed_ms(e0, e3) > 0.0
        for y, want in zip(ys, plain):
            assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_works_from_another_thread_and_concurrent_calls_do_not_mix(be, oxref):
    """The Backend surface is Send + Sync (src/gpu.rs:151): a call from another thread, on weights uploaded here, and eight
    threads calling at once, each with its own input, get their own rows (src/cuda.rs:2048-2077, :2411-2439). A call's
    rows are a function of its inputs alone, so they must equal the rows of the same call made alone, bit for bit."""
    import threading
    from oxinfer_amd import synth
    n_out, n_in = 64, 512
    raw = oxref.random_blocks(Q4_K, n_out * n_in // 256, 91)[0]
    wq, sc, bi = synth.mlx_q4(n_out, n_in, 92)
    ws = [be.upload_gguf(Q4_K, raw, n_out, n_in), be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in)]
    cases = []
    for i in range(8):
        t = (3, 40)[i % 2]  # the shared decode launch, and the prefill GEMM with its scratch in the context
        x = synth.activations(t, n_in, 300 + i)
        ys = [np.full((t, n_out), np.nan, np.float32) for _ in ws]
        assert be.matmul(x, t, n_in, list(zip(ws, ys))), be.last_error()
        assert row_err(ys[0], oxref.gguf_decode(Q4_K, raw, n_out, n_in, x, t) if t <= 16 else oxref.gemm_quant(Q4_K, raw, None, None, n_out, n_in, x, t)) < 2e-2
        cases.append((t, x, ys))
    errors = []

    def worker(t, x, want, rounds):
        try:
            for _ in range(rounds):
                ys = [np.full((t, n_out), np.nan, np.float32) for _ in ws]
                if not be.matmul(x, t, n_in, list(zip(ws, ys))):
                    raise AssertionError("declined: " + be.last_error())
                for y, w0 in zip(ys, want):
                    if not np.array_equal(y.view(np.uint32), w0.view(np.uint32)):
                        raise AssertionError(f"rows of another call (t = {t})")
        except Exception as e:  # reported by the main thread
            errors.append(e)

    th = threading.Thread(target=worker, args=(*cases[0], 1))
    th.start()
    th.join()
    assert not errors, errors
    threads = [threading.Thread(target=worker, args=(*c, 8)) for c in cases]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
