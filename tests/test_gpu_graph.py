"""GPU parity of the device-resident decode-graph ops (Op::Norm / Linear / Glu / Route / Experts of the reference's
src/gpu_decode.rs) against compositions of the CPU oracle, through the C ABI. Everything stays on the device between
the ops; the bar is that of the decode path (1e-3 of a row's largest value, f32 accumulation)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
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


def rmsnorm_ref(x, w, eps):
    """rmsnorm of the reference (src/kernels.rs:2107-2123): squares summed one after the other in f32, r = ss^(-1/2),
    out = (x * r) * w."""
    out = np.empty_like(x)
    for i, row in enumerate(x):
        sq = (row * row).astype(np.float32)
        ss = np.add.accumulate(sq, dtype=np.float32)[-1] / np.float32(row.size) + np.float32(eps)
        r = np.float32(ss) ** np.float32(-0.5)
        out[i] = (row * r) * w if w is not None else row * r
    return out.astype(np.float32)


def weights(be, oxref, kind, n_out, n_in, seed):
    """(device weight, decode(x, t) on the oracle) for one storage format."""
    from oxinfer_amd import synth
    if kind == "mlx":
        wq, sc, bi = synth.mlx_q4(n_out, n_in, seed)
        rng = np.random.default_rng(seed + 1)
        sf = (sc.astype(np.uint32) << 16).view(np.float32)
        bi = synth.bf16_bits((np.float32(-8.0) * sf + 0.01 * rng.uniform(-1, 1, sc.shape)).astype(np.float32))
        q, s16, off = oxref.from_mlx_q4(wq, sc, bi, n_out, n_in, 64)
        return be.upload_mlx_q4(wq, sc, bi, 64, n_out, n_in), lambda x, t: oxref.q4_decode(q, s16, off, 64, n_out, n_in, x, t)
    if kind == "q4":  # planar Q4 without offsets: the v_dot4 kernel, whose output stage only stores
        rng = np.random.default_rng(seed)
        q = rng.integers(0, 256, (n_out, n_in // 2), dtype=np.uint8)
        sc = np.abs(rng.normal(0, 0.01, (n_out, n_in // 32))).astype(np.float16).view(np.uint16)
        sc[:, 1::2] = sc[:, 0::2] + 1  # scales differ inside a group: stays planar
        return be.upload_q4(q, sc, None, 0, n_out, n_in), lambda x, t: oxref.q4_decode(q, sc, None, 32, n_out, n_in, x, t)
    if kind == "bf16":
        wf = synth.bf16_round(np.random.default_rng(seed).normal(0.0, 0.02, (n_out, n_in)).astype(np.float32))
        return be.upload_bf16((wf.view(np.uint32) >> 16).astype(np.uint16), n_out, n_in), lambda x, t: oxref.gemm_f32(wf, n_out, n_in, x, t)
    if kind == "fp8":
        data, scales = synth.fp8_e4m3(n_out, n_in, seed)
        return be.upload_fp8(data, scales, n_out, n_in), lambda x, t: oxref.gemm_quant(oxref.F8E4M3, data, scales, None, n_out, n_in, x, t)
    raw, _ = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), seed)
    return be.upload_gguf(kind, raw, n_out, n_in), lambda x, t: oxref.gguf_decode(kind, raw, n_out, n_in, x, t)


@pytest.mark.parametrize("kind,n_out,n_in", [(Q4_K, 53, 768), (Q8_0, 40, 864), (Q6_K, 24, 512), (Q4_0, 33, 1120), ("mlx", 37, 640),
                                             (Q4_K, 32, 14336), (Q8_0, 48, 14336),  # K sliced across workgroups
                                             ("q4", 10, 512), ("bf16", 21, 520), ("fp8", 200, 512)])
def test_linear_store_add_gated(be, oxref, kind, n_out, n_in):
    """LinMode Store / Add / AddGated (src/gpu_decode.rs:37-50) over every storage format, 1 to 16 tokens."""
    import torch
    from oxinfer_amd import hip, synth
    w, ref_of = weights(be, oxref, kind, n_out, n_in, 500)
    assert w is not None, be.last_error()
    dense = kind in ("bf16", "fp8")
    for t in (1, 3, 8, 11, 16):
        x = synth.activations(t, n_in, 510 + t, bf16=dense)
        ref = ref_of(x, t)
        xd = dev(x)
        args = dict(x=xd) if dense else dict(xa=be.quantize_act(xd))
        y0 = synth.activations(t, n_out, 520 + t) * np.abs(ref).max()
        g = np.linspace(-3.0, 3.0, t).astype(np.float32)
        y = torch.full((t, n_out), float("nan"), device="cuda")
        assert be.linear(w, y, t=t, mode=hip.LIN_STORE, **args), be.last_error()
        assert row_err(y.cpu().numpy(), ref) < TOL, t
        y = dev(y0)
        assert be.linear(w, y, t=t, mode=hip.LIN_ADD, **args), be.last_error()
        assert row_err(y.cpu().numpy() - y0, ref) < TOL, t
        y = dev(y0)
        assert be.linear(w, y, t=t, mode=hip.LIN_ADD_GATED, gate=dev(g), **args), be.last_error()
        sig = (1.0 / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float32)[:, None]
        assert row_err(y.cpu().numpy() - y0, sig * ref) < TOL, t
    # the modes must come with their operands, and only with them
    xa1 = be.quantize_act(dev(synth.activations(1, n_in, 1))) if not dense else None
    x1 = dev(synth.activations(1, n_in, 1)) if dense else None
    y = torch.full((1, n_out), 7.0, device="cuda")
    assert not be.linear(w, y, xa=xa1, x=x1, t=1, mode=hip.LIN_ADD_GATED)
    assert not be.linear(w, y, xa=xa1, x=x1, t=1, mode=hip.LIN_STORE, gate=y)
    assert not be.linear(w, y, xa=xa1, x=x1, t=1, mode=hip.LIN_SILU_PAIR)
    assert not be.linear(w, y, xa=xa1, x=x1, t=17, mode=hip.LIN_STORE)
    assert float(y.min()) == 7.0 and float(y.max()) == 7.0  # declined: nothing written


@pytest.mark.parametrize("kind,n_out,n_in", [(Q4_K, 96, 512), (Q8_0, 40, 864), ("mlx", 80, 640), (Q4_K, 32, 14336), ("q4", 10, 512), ("bf16", 21, 520),
                                             (Q6_K, 48, 512), (Q4_K, 1000, 768), (Q8_0, 272, 14336), (Q4_0, 130, 1120), (Q6_K, 40, 14336)])
def test_linear_pairs(be, oxref, kind, n_out, n_in):
    """LinMode SiluPair / GeluPair: y = act(W x) * (W2 x) with silu_mul / gelu_mul (src/kernels.rs:2188-2198, :2234-2257). Over
    the matrix-core formats the pair is one launch whose workgroups hold the same rows' tiles of both matrices (the CUDA
    kernels' modes 2 and 3, src/cuda_decode.cu:131-167), with and without K slices, ragged last row groups, 1 to 13 tokens:
    the rows must equal Op::Glu of the two products computed apart, bit for bit."""
    import torch
    from oxinfer_amd import hip, synth
    w, ref_w = weights(be, oxref, kind, n_out, n_in, 600)
    u, ref_u = weights(be, oxref, kind, n_out, n_in, 601)
    dense = kind == "bf16"
    for t in (1, 4, 8, 13):
        x = synth.activations(t, n_in, 610 + t, bf16=dense) * np.float32(3.0)
        g_ref, u_ref = ref_w(x, t), ref_u(x, t)
        xd = dev(x)
        args = dict(x=xd) if dense else dict(xa=be.quantize_act(xd))
        y = torch.full((t, n_out), float("nan"), device="cuda")
        assert be.linear(w, y, t=t, mode=hip.LIN_SILU_PAIR, w2=u, **args), be.last_error()
        assert row_err(y.cpu().numpy(), oxref.silu_mul(g_ref, u_ref)) < TOL, t
        y = torch.full((t, n_out), float("nan"), device="cuda")
        assert be.linear(w, y, t=t, mode=hip.LIN_GELU_PAIR, w2=u, **args), be.last_error()
        g64 = g_ref.astype(np.float64)
        with np.errstate(over="ignore"):  # exp overflows to inf for very negative gates: the quotient is -0.0, as on the device
            gelu = g64 / (1.0 + np.exp(-2.0 * 0.7978846 * (g64 + 0.044715 * g64 ** 3))) * u_ref
        assert row_err(y.cpu().numpy(), gelu.astype(np.float32)) < TOL, t
        # Op::Glu on the two products computed apart gives the same rows as the pair
        gd, ud = torch.empty((t, n_out), device="cuda"), torch.empty((t, n_out), device="cuda")
        assert be.linear(w, gd, t=t, **args) and be.linear(u, ud, t=t, **args)
        assert np.array_equal(be.glu(gd, ud, gelu=True).cpu().numpy().view(np.uint32), y.cpu().numpy().view(np.uint32))
        ys = torch.full((t, n_out), float("nan"), device="cuda")
        assert be.linear(w, ys, t=t, mode=hip.LIN_SILU_PAIR, w2=u, **args), be.last_error()
        assert np.array_equal(be.glu(gd, ud, gelu=False).cpu().numpy().view(np.uint32), ys.cpu().numpy().view(np.uint32))
    if not dense:  # a second matrix of another storage format is not pairable: declined, nothing written
        other, _ = weights(be, oxref, Q8_0 if kind != Q8_0 else Q4_0, n_out, n_in, 602)
        y = torch.full((1, n_out), 7.0, device="cuda")
        assert not be.linear(w, y, t=1, mode=hip.LIN_SILU_PAIR, w2=other, xa=be.quantize_act(dev(synth.activations(1, n_in, 1))))
        assert float(y.min()) == 7.0 and float(y.max()) == 7.0


@pytest.mark.parametrize("n", [4096, 96, 14336])
def test_rmsnorm_quantize(be, oxref, n):
    """Op::Norm fused with the quantization of the next linear's input: the normed row within a few ulp of rmsnorm's
    (src/kernels.rs:2107-2123; its one-after-the-other sum of squares is not repeatable in parallel), and the QAct
    exactly quantize_act's of that row (src/quant.rs:243-343), bit for bit."""
    import torch
    from oxinfer_amd import synth
    t = 5
    v, _ = oxref.lcg_stream(n, t * n)
    x = ((v >> 7).astype(np.float64) / float(1 << 24) - 0.5).astype(np.float32).reshape(t, n)
    x *= np.array([1e-3, 1.0, 300.0, 2e5, 1.0], np.float32)[:, None]
    x[4] = 0.0  # an all-zero row: r = eps^(-1/2), every output 0
    rng = np.random.default_rng(n)
    wf = (1.0 + 0.1 * rng.normal(size=n)).astype(np.float32)
    wb = synth.bf16_round(wf)
    for eps in (1e-6, 1e-5):
        for w_host, w_dev in ((None, None), (wf, dev(wf)), (wb, dev(wb).to(torch.bfloat16))):
            out, qa = be.rmsnorm_quantize(dev(x), w_dev, eps)
            out = out.cpu().numpy()
            ref = rmsnorm_ref(x, w_host, eps)
            assert np.allclose(out, ref, rtol=2e-5, atol=0)  # (the f32 running sum of n squares is off by up to ~sqrt(n) ulp)
            q, scales, sums, fsums, hsums = oxref.quantize_act(out, t, n)
            assert np.array_equal(qa.q.cpu().numpy(), q)
            assert np.array_equal(qa.scales.cpu().numpy().view(np.uint32), scales.view(np.uint32))
            assert np.array_equal(qa.sums.cpu().numpy(), sums)
            assert np.array_equal(qa.fsums.cpu().numpy().view(np.uint32), fsums.view(np.uint32))
            assert np.array_equal(qa.hsums.cpu().numpy().view(np.uint32), hsums.view(np.uint32))
            assert np.array_equal(qa.sums16.cpu().numpy(), q.astype(np.int32).reshape(t, n // 16, 16).sum(axis=2))
            # without the f32 output the codes are the same
            _, qb = be.rmsnorm_quantize(dev(x), w_dev, eps, want_out=False)
            assert np.array_equal(qb.q.cpu().numpy(), q) and np.array_equal(qb.scales.cpu().numpy().view(np.uint32), scales.view(np.uint32))


def test_norm_with_all_fields(be, oxref):
    """Op::Norm as the reference defines it (src/gpu_decode.rs:53-66, src/cuda_decode.cu:314-327): rows with strides
    inside a larger buffer, the `pre` factor, `out +=`, and views that do not start on 16-byte boundaries. Against the f64
    definition out (+)= ((x pre) r) w, r = (mean((x pre)^2) + eps)^(-1/2); the quantized row is quantize_act of what `out`
    holds, bit for bit."""
    import torch
    rng = np.random.default_rng(9)
    n, rows, eps = 256, 3, 1e-5
    for x_off, o_off, xs, os_, pre, add in ((0, 0, 0, 0, 1.0, False), (4, 8, 320, 288, 0.5, True), (3, 1, 259, 261, 2.0, False), (1, 2, 256, 256, 1.5, True)):
        xsf, osf = xs or n, os_ or n
        xbuf = rng.normal(0, 2, x_off + rows * xsf + 7).astype(np.float32)
        obuf = rng.normal(0, 1, o_off + rows * osf + 7).astype(np.float32)
        w = rng.normal(1, 0.2, n + 1).astype(np.float32)
        xd, od, wd = dev(xbuf), dev(obuf), dev(w)
        w_view = wd[1:] if x_off % 4 else wd[:n]   # an unaligned weight view with the unaligned inputs
        w_host = w[1:] if x_off % 4 else w[:n]
        ok, qa = be.norm(xd[x_off:], n, rows, out=od[o_off:], w=w_view, pre=pre, x_stride=xs, out_stride=os_, eps=eps, add=add, want_q=True)
        assert ok, be.last_error()
        torch.cuda.synchronize()
        got = od.cpu().numpy()
        want = obuf.copy()
        for r in range(rows):
            xr = xbuf[x_off + r * xsf: x_off + r * xsf + n].astype(np.float64) * pre
            v = xr / np.sqrt((xr * xr).mean() + eps) * w_host.astype(np.float64)
            seg = slice(o_off + r * osf, o_off + r * osf + n)
            want[seg] = (obuf[seg] + v if add else v).astype(np.float32)
        assert np.abs(got - want).max() < 2e-6 * max(1.0, np.abs(want).max())
        # nothing outside the rows was touched
        mask = np.ones(obuf.size, bool)
        for r in range(rows):
            mask[o_off + r * osf: o_off + r * osf + n] = False
        assert np.array_equal(got[mask], obuf[mask])
        rows_out = np.stack([got[o_off + r * osf: o_off + r * osf + n] for r in range(rows)])
        q, sc, sums, fs, hs = oxref.quantize_act(rows_out, rows, n)
        assert np.array_equal(qa.q.cpu().numpy(), q) and np.array_equal(qa.scales.cpu().numpy().view(np.uint32), sc.view(np.uint32))
        assert np.array_equal(qa.sums.cpu().numpy(), sums) and np.array_equal(qa.fsums.cpu().numpy().view(np.uint32), fs.view(np.uint32))
    # `add` without an output, strides shorter than a row: declined
    assert not be.norm(xd, n, 1, out=None, add=True, want_q=True)[0]
    assert not be.norm(xd, n, 2, out=od, x_stride=n - 4)[0]


def test_decode_on_two_streams_overlaps_and_keeps_the_bits(be, oxref):
    """Calls on different streams keep separate scratch (partial rows and counters of K-sliced shapes), so they may
    overlap: matmuls issued alternately on two streams give, bit for bit, the rows of the same calls issued one after the
    other on one stream. A released stream's next call allocates its scratch again."""
    import torch
    n_out, n_in, t = 528, 14336, 8   # 14336 columns: K is sliced across workgroups, the slices meet through the scratch
    raws = [oxref.random_blocks(8, n_out * n_in // 32, 60 + i)[0] for i in range(2)]
    ws = [be.upload_gguf(8, r, n_out, n_in) for r in raws]
    xs = [np.random.default_rng(70 + i).normal(0, 1, (t, n_in)).astype(np.float32) for i in range(2)]
    xas = [be.quantize_act(dev(x)) for x in xs]
    serial = [be.decode(ws[i], xa=xas[i], t=t).cpu().numpy() for i in range(2)]
    for i in range(2):
        assert row_err(serial[i], oxref.gguf_decode(8, raws[i], n_out, n_in, xs[i], t)) < 1e-3
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ys = [[torch.empty((t, n_out), dtype=torch.float32, device="cuda") for _ in range(6)] for _ in range(2)]
    for rep in range(6):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                be.decode(ws[i], xa=xas[i], t=t, y=ys[i][rep])
    torch.cuda.synchronize()
    for i in range(2):
        for rep in range(6):
            assert np.array_equal(ys[i][rep].cpu().numpy().view(np.uint32), serial[i].view(np.uint32)), (i, rep)
    assert be.stream_release(streams[0].cuda_stream)
    with torch.cuda.stream(streams[0]):
        again = be.decode(ws[0], xa=xas[0], t=t)
    torch.cuda.synchronize()
    assert np.array_equal(again.cpu().numpy().view(np.uint32), serial[0].view(np.uint32))
    assert be.stream_release(streams[0].cuda_stream) and be.stream_release(streams[1].cuda_stream)


@pytest.mark.parametrize("ne,h,k", [(128, 2048, 8), (6, 256, 3), (300, 130, 6)])
def test_route(be, oxref, ne, h, k):
    """Op::Route (src/gpu_decode.rs:154-172): the router's logits (and the shared expert's gate logit behind them), then
    route_top_k over the experts' logits (src/moe.rs:180-193) into sel."""
    from oxinfer_amd import synth
    t = 3
    rng = np.random.default_rng(ne)
    router = rng.normal(0, 0.05, (ne, h)).astype(np.float32)
    gate = rng.normal(0, 0.05, h).astype(np.float32)
    scale = (0.5 + rng.uniform(size=ne)).astype(np.float32)
    x = synth.activations(t, h, 7)
    for with_gate, with_scale in ((False, False), (True, False), (True, True)):
        logits, sel = be.route(dev(x), dev(router), k, gate=dev(gate) if with_gate else None, expert_scale=dev(scale) if with_scale else None)
        logits, sel = logits.cpu().numpy(), sel.cpu().numpy()
        want = x.astype(np.float64) @ router.astype(np.float64).T
        assert np.abs(logits[:, :ne] - want).max() < 1e-5 * max(1.0, np.abs(want).max())
        if with_gate:
            assert np.abs(logits[:, ne] - x.astype(np.float64) @ gate.astype(np.float64)).max() < 1e-5
        ids, wts = sel[0].view(np.uint32), sel[1].view(np.float32)
        for i in range(t):
            ri, rw = oxref.route_top_k(np.ascontiguousarray(logits[i, :ne]), k)
            assert np.array_equal(ids[i], ri), i
            assert np.allclose(wts[i], rw * (scale[ri] if with_scale else 1.0), rtol=1e-6, atol=0), i


@pytest.mark.parametrize("ne,h,inter,k", [(6, 256, 128, 3), (16, 2048, 768, 8)])
def test_layer_chain_stays_on_the_device(be, oxref, ne, h, inter, k):
    """One token through residual linear (Add) -> RMSNorm + quantize -> Route -> Experts (add), every op on device
    buffers on one stream, against the same chain composed from the oracle's pieces."""
    import torch
    from oxinfer_amd import hip, synth
    raw_gu = [synth.mlx_q4(2 * inter, h, 3100 + e) for e in range(ne)]
    raw_dn = [synth.mlx_q4(h, inter, 3200 + e) for e in range(ne)]
    q_gu = [oxref.from_mlx_q4(*r, 2 * inter, h, 64) for r in raw_gu]
    q_dn = [oxref.from_mlx_q4(*r, h, inter, 64) for r in raw_dn]
    moe = be.upload_moe([be.desc_mlx_q4(*r, 64, 2 * inter, h) for r in raw_gu], [be.desc_mlx_q4(*r, 64, h, inter) for r in raw_dn], h, inter)
    assert moe is not None, be.last_error()
    wo_raw = synth.gguf_q4_k(h, h, 3300)
    wo = be.upload_gguf(Q4_K, wo_raw, h, h)
    rng = np.random.default_rng(3400 + ne)
    router = rng.normal(0, 0.2, (ne, h)).astype(np.float32)
    wn = (1.0 + 0.1 * rng.normal(size=h)).astype(np.float32)
    for t in (1, 4):
        x0 = synth.activations(t, h, 3500 + t)
        resid = synth.activations(t, h, 3600 + t)
        # device: four launches of the library per op group, nothing read back in between
        y = dev(resid)
        assert be.linear(wo, y, xa=be.quantize_act(dev(x0)), t=t, mode=hip.LIN_ADD), be.last_error()
        normed, qa = be.rmsnorm_quantize(y, dev(wn), 1e-6)
        logits, sel = be.route(normed, dev(router), k)
        assert be.experts(moe, normed, sel, y, add=True), be.last_error()
        torch.cuda.synchronize()
        # oracle
        y1 = resid + oxref.gguf_decode(Q4_K, wo_raw, h, h, x0, t)
        n1 = rmsnorm_ref(y1, wn, 1e-6)
        idx = np.zeros((t, k), np.uint32)
        w = np.zeros((t, k), np.float32)
        for i in range(t):
            idx[i], w[i] = oxref.route_top_k((n1[i].astype(np.float64) @ router.astype(np.float64).T).astype(np.float32), k)
        assert np.array_equal(sel[0].cpu().numpy().view(np.uint32), idx)
        y2 = oxref.moe_q4(q_gu, q_dn, 64, h, inter, n1, t, idx, w, y1, decode_path=True)
        assert row_err(y.cpu().numpy(), y2) < TOL, (t, row_err(y.cpu().numpy(), y2))
        # Experts with add = false writes the experts' sum alone
        only = torch.full((t, h), float("nan"), device="cuda")
        assert be.experts(moe, normed, sel, only, add=False)
        assert row_err(only.cpu().numpy(), y2 - y1) < TOL


@pytest.mark.parametrize("ne,h,inter,k,t", [(16, 2048, 768, 8, 1), (6, 256, 128, 3, 4)])
def test_plan_replays_a_layer_bit_for_bit(be, oxref, ne, h, inter, k, t):
    """A token's chain of ops recorded once and replayed (the matmul side of DecodePlan::step, src/gpu_decode.rs:572-587):
    quantize -> gate / up pair linear -> quantize -> down linear (Add) -> RMSNorm + quantize -> Route -> Experts (add) ->
    a K-sliced linear. Every replay, each on new contents of the same input buffer and with eager work and
    synchronizations between the replays, must equal the same chain issued call by call, bit for bit; and that chain is
    itself held to the oracle."""
    import torch
    from oxinfer_amd import hip, synth
    ffn = 512
    raw_gu = [synth.mlx_q4(2 * inter, h, 5100 + e) for e in range(ne)]
    raw_dn = [synth.mlx_q4(h, inter, 5200 + e) for e in range(ne)]
    q_gu = [oxref.from_mlx_q4(*r, 2 * inter, h, 64) for r in raw_gu]
    q_dn = [oxref.from_mlx_q4(*r, h, inter, 64) for r in raw_dn]
    moe = be.upload_moe([be.desc_mlx_q4(*r, 64, 2 * inter, h) for r in raw_gu], [be.desc_mlx_q4(*r, 64, h, inter) for r in raw_dn], h, inter)
    assert moe is not None, be.last_error()
    g_raw, u_raw, d_raw = synth.gguf_q4_k(ffn, h, 5300), synth.gguf_q4_k(ffn, h, 5301), synth.gguf_q8_0(h, ffn, 5302)
    wg, wu, wd = be.upload_gguf(Q4_K, g_raw, ffn, h), be.upload_gguf(Q4_K, u_raw, ffn, h), be.upload_gguf(Q8_0, d_raw, h, ffn)
    big_raw = synth.gguf_q8_0(272, 14336, 5303)                       # 14336 columns: its K slices meet through the stream's scratch
    wbig = be.upload_gguf(Q8_0, big_raw, 272, 14336)
    rng = np.random.default_rng(5400 + ne)
    router = dev(rng.normal(0, 0.2, (ne, h)).astype(np.float32))
    wn = dev((1.0 + 0.1 * rng.normal(size=h)).astype(np.float32))
    # the plan's buffers: allocated once, named by every recorded launch
    x_in = torch.zeros((t, h), device="cuda")
    xbig = torch.zeros((t, 14336), device="cuda")
    y = torch.zeros((t, h), device="cuda")
    a = torch.zeros((t, ffn), device="cuda")
    normed = torch.zeros((t, h), device="cuda")
    ybig = torch.zeros((t, 272), device="cuda")
    logits = torch.zeros((t, ne), device="cuda")
    sel = torch.zeros((2, t, k), dtype=torch.int32, device="cuda")
    qx, qa, qn, qbig = hip.QAct(t, h, "cuda"), hip.QAct(t, ffn, "cuda"), hip.QAct(t, h, "cuda"), hip.QAct(t, 14336, "cuda")
    C = __import__("ctypes")

    def chain():
        be.quantize_act(x_in, out=qx)
        assert be.linear(wg, a, xa=qx, t=t, mode=hip.LIN_SILU_PAIR, w2=wu), be.last_error()
        be.quantize_act(a, out=qa)
        assert be.linear(wd, y, xa=qa, t=t, mode=hip.LIN_ADD), be.last_error()
        ok = be.lib.oxhip_dev_rmsnorm_quantize(be.ctx, y.data_ptr(), wn.data_ptr(), None, 1e-6, t, h, normed.data_ptr(), C.byref(qn.c), be._stream())
        assert ok, be.last_error()
        ok = be.lib.oxhip_dev_route(be.ctx, normed.data_ptr(), router.data_ptr(), None, t, ne, h, k, logits.data_ptr(), sel.data_ptr(), None, be._stream())
        assert ok, be.last_error()
        assert be.experts(moe, normed, sel, y, add=True), be.last_error()
        be.quantize_act(xbig, out=qbig)
        assert be.linear(wbig, ybig, xa=qbig, t=t), be.last_error()

    stream = torch.cuda.Stream()
    inputs = [(synth.activations(t, h, 5500 + i), synth.activations(t, h, 5600 + i), synth.activations(t, 14336, 5700 + i)) for i in range(4)]

    def load(i):
        x_in.copy_(dev(inputs[i][0]))
        y.copy_(dev(inputs[i][1]))
        xbig.copy_(dev(inputs[i][2]))

    eager = []
    with torch.cuda.stream(stream):
        for i in range(4):   # call by call (the first pass also creates every scratch the chain needs)
            load(i)
            chain()
            stream.synchronize()
            eager.append((y.cpu().numpy().copy(), ybig.cpu().numpy().copy(), sel.cpu().numpy().copy(), a.cpu().numpy().copy()))
        # the call-by-call chain against the oracle (input 0)
        x0, r0, xb0 = inputs[0]
        gate = oxref.gguf_decode(Q4_K, g_raw, ffn, h, x0, t)
        act = oxref.silu_mul(gate, oxref.gguf_decode(Q4_K, u_raw, ffn, h, x0, t))
        assert row_err(eager[0][3], act) < TOL
        y1 = r0 + oxref.gguf_decode(Q8_0, d_raw, h, ffn, eager[0][3], t)
        n1 = rmsnorm_ref(y1, wn.cpu().numpy(), 1e-6)
        idx = eager[0][2][0].view(np.uint32)
        wts = eager[0][2][1].view(np.float32)
        y2 = oxref.moe_q4(q_gu, q_dn, 64, h, inter, n1, t, idx, wts, y1, decode_path=True)
        assert row_err(eager[0][0], y2) < 2 * TOL, row_err(eager[0][0], y2)
        assert row_err(eager[0][1], oxref.gguf_decode(Q8_0, big_raw, 272, 14336, xb0, t)) < TOL
        plan = be.plan_record(chain)
        assert plan.launches >= 9
        for rnd in range(2):
            for i in (2, 0, 3, 1):
                load(i)
                plan.replay()
                stream.synchronize()
                got = (y.cpu().numpy(), ybig.cpu().numpy(), sel.cpu().numpy(), a.cpu().numpy())
                for g_, e_ in zip(got, eager[i]):
                    assert np.array_equal(g_.view(np.uint32), e_.view(np.uint32)), (rnd, i)
                # eager work of the program's own between the replays (another matmul through the same scratch)
                be.quantize_act(xbig, out=qbig)
                assert be.linear(wbig, ybig, xa=qbig, t=t)
                torch.cuda.synchronize()
        del plan


def test_plan_recording_on_a_cold_stream_declines(be, oxref):
    """Recording on a stream whose scratch does not exist yet: the call that would have to allocate declines, the
    recording is refused as a whole (oxhip_plan_end returns 0, nothing is replayable) and the stream works again
    afterwards; once the chain has run there, the same recording succeeds. The null stream is refused."""
    import torch
    assert not be.lib.oxhip_plan_begin(be.ctx, None)
    raw, _ = oxref.random_blocks(8, 272 * 14336 // 32, 1)
    w = be.upload_gguf(8, raw, 272, 14336)
    x = torch.ones((1, 14336), device="cuda")
    stream = torch.cuda.Stream()   # a fresh stream: its K-slice scratch does not exist yet
    with torch.cuda.stream(stream):
        qa = be.quantize_act(x)
        y = torch.full((1, 272), 3.0, device="cuda")
        stream.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        with pytest.raises(RuntimeError, match="before recording"):
            be.plan_record(lambda: be.linear(w, y, xa=qa, t=1))
        stream.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0 and float(y.min()) == 3.0   # nothing allocated, nothing run
        assert be.linear(w, y, xa=qa, t=1), be.last_error()      # the same call outside a recording: allocates and runs
        stream.synchronize()
        want = y.cpu().numpy().copy()
        assert row_err(want, oxref.gguf_decode(8, raw, 272, 14336, np.ones((1, 14336), np.float32), 1)) < TOL
        plan = be.plan_record(lambda: be.linear(w, y, xa=qa, t=1))  # warmed now: recordable
        assert plan.launches >= 1
        y.zero_()
        plan.replay()
        stream.synchronize()
        assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
