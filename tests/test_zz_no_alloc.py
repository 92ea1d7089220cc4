"""The allocation-free decode entry point (oxhip_dev_decode_noalloc) against oxhip_dev_decode, through the C ABI.

Both run the same kernels with the same workgroup shape, so the rows must be equal bit for bit; the existing entry
point is itself held to the oracle (1e-3) here as well. Two calls in a row share the library's static scratch, the
second with a smaller input: what the first left behind (partial rows, counters) must not leak into it.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = 8, 12


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


def one_case(be, oxref, kind, n_out, n_in, t, seed):
    import torch
    raw, s2 = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), seed)
    w = be.upload_gguf(kind, raw, n_out, n_in)
    assert w is not None, be.last_error()
    v, _ = oxref.lcg_stream(s2, t * n_in)
    x = ((v % 2001).astype(np.float32) / np.float32(1000.0) - np.float32(1.0)).reshape(t, n_in)
    xa = be.quantize_act(dev(x))
    y = torch.full((t, n_out), float("nan"), dtype=torch.float32, device="cuda")
    got = be.decode_noalloc(w, xa, t=t, y=y)
    assert got is not None, be.last_error()
    want = be.decode(w, xa=xa, t=t)
    torch.cuda.synchronize()
    got, want = got.cpu().numpy(), want.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref = oxref.gguf_decode(kind, raw, n_out, n_in, x, t)
    assert row_err(got, ref) < 1e-3
    return w


def test_no_alloc_decode_matches_decode_twice(be, oxref):
    # rows of 14336 columns slice K across workgroups: partial rows and counters live in the static scratch
    w1 = one_case(be, oxref, Q8_0, 528, 14336, 11, 4101)
    # a smaller input right behind it, again K-sliced, then one whose K stays inside a workgroup
    w2 = one_case(be, oxref, Q4_K, 200, 8192, 3, 4102)
    w3 = one_case(be, oxref, Q4_K, 37, 768, 1, 4103)
    del w1, w2, w3


def test_no_alloc_call_leaves_device_memory_alone(be, oxref):
    """The property the entry point exists for: once the weight and the buffers are there, a call allocates and frees
    nothing on the device (free memory as the driver reports it is the same before and after), on a K-sliced shape and on
    one whose K stays inside a workgroup."""
    import torch
    for kind, n_out, n_in, t in ((Q8_0, 528, 14336, 8), (Q4_K, 64, 1024, 2)):
        raw, _ = oxref.random_blocks(kind, n_out * n_in // oxref.block_size(kind), 4200)
        w = be.upload_gguf(kind, raw, n_out, n_in)
        xa = be.quantize_act(torch.ones((t, n_in), dtype=torch.float32, device="cuda"))
        y = torch.empty((t, n_out), dtype=torch.float32, device="cuda")
        assert be.decode_noalloc(w, xa, t=t, y=y) is not None, be.last_error()   # warm: the kernel's code object is loaded
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        for _ in range(3):
            assert be.decode_noalloc(w, xa, t=t, y=y) is not None, be.last_error()
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        assert free1 == free0, (free0, free1)


def test_no_alloc_rejects_what_the_scratch_cannot_hold(be):
    n_out, n_in = 16640, 32768  # 8 K slices x 8 x 16640 floats of partial rows > 4 MiB
    raw = np.zeros(n_out * (n_in // 256) * 144, np.uint8)
    w = be.upload_gguf(Q4_K, raw, n_out, n_in)
    assert w is not None, be.last_error()
    import torch
    xa = be.quantize_act(torch.zeros((1, n_in), dtype=torch.float32, device="cuda"))
    y = torch.full((1, n_out), 7.0, dtype=torch.float32, device="cuda")
    assert be.decode_noalloc(w, xa, t=1, y=y) is None
    assert "static scratch" in be.last_error()
    torch.cuda.synchronize()
    assert float(y.min()) == 7.0 and float(y.max()) == 7.0  # declined: nothing written
    # bad arguments decline too
    assert be.decode_noalloc(w, xa, t=17, y=y) is None
