"""ctypes binding of liboxinfer_hip.so and `HipBackend`, the mirror of `trait Backend`
(src/gpu.rs:151-294 of the reference): name / wants / upload / matmul / stats with the reference's
conventions (False / None = declined, nothing written), plus the device-pointer entry points.

Device buffers are torch tensors (torch is plumbing for memory and streams only).
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboxinfer_hip.so")

W_BF16, W_Q8, W_Q4, W_GGUF, W_MLX_Q4 = 0, 1, 2, 3, 4
GGML_Q4_0, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_MXFP4, GGML_NVFP4, GGML_F8E4M3 = 2, 8, 12, 13, 14, 39, 40, 0x1000
GGML_BLOCK = {GGML_Q4_0: (32, 18), GGML_Q8_0: (32, 34), GGML_Q4_K: (256, 144), GGML_Q5_K: (256, 176), GGML_Q6_K: (256, 210), GGML_MXFP4: (32, 17), GGML_NVFP4: (64, 36)}


class WeightDesc(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("ggml_type", C.c_uint32), ("n_out", C.c_size_t), ("n_in", C.c_size_t),
                ("data", C.c_void_p), ("scales", C.c_void_p), ("offsets", C.c_void_p), ("group", C.c_uint32),
                ("block_scales", C.c_void_p), ("bs_rows", C.c_uint32), ("bs_cols", C.c_uint32)]


class Job(C.Structure):
    _fields_ = [("w", C.c_void_p), ("n_out", C.c_size_t), ("y", C.c_void_p)]


class DecodeJob(C.Structure):
    _fields_ = [("w", C.c_void_p), ("xa", C.c_void_p), ("x", C.c_void_p), ("t", C.c_size_t), ("y", C.c_void_p),
                ("ev_start", C.c_void_p), ("ev_stop", C.c_void_p)]


class GpuInfo(C.Structure):
    _fields_ = [("index", C.c_int), ("name", C.c_char * 256), ("arch", C.c_char * 64), ("memory_bytes", C.c_uint64),
                ("driver", C.c_char * 64), ("usable", C.c_int)]


class QuantJob(C.Structure):
    _fields_ = [("x", C.c_void_p), ("t", C.c_size_t), ("n_in", C.c_size_t), ("out", C.c_void_p)]


class RowsJob(C.Structure):
    _fields_ = [("w", C.c_void_p), ("up", C.c_void_p), ("n_out", C.c_size_t), ("y", C.c_void_p)]


class QActC(C.Structure):
    _fields_ = [("q", C.c_void_p), ("scales", C.c_void_p), ("sums", C.c_void_p), ("fsums", C.c_void_p),
                ("hsums", C.c_void_p), ("sums16", C.c_void_p), ("t", C.c_size_t), ("n_in", C.c_size_t)]


_lib = None


def library_path():
    return _SO


def load_library():
    """Loads liboxinfer_hip.so (built in-tree by `python -m oxinfer_amd.build`). Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        raise RuntimeError(f"{_SO} is not built: run `python -m oxinfer_amd.build` (hipcc, gfx950). "
                           "There is no CPU fallback in this package.")
    try:
        import torch  # noqa: F401  (its bundled HIP runtime must be the one this process uses)
    except ImportError:
        pass
    lib = C.CDLL(_SO)
    vp, sz = C.c_void_p, C.c_size_t
    sig = {
        "oxhip_probe": (C.c_int, [C.POINTER(GpuInfo), C.c_int]),
        "oxhip_open": (C.c_int, [C.c_int, C.POINTER(vp)]),
        "oxhip_close": (None, [vp]),
        "oxhip_name": (C.c_char_p, [vp]),
        "oxhip_last_error": (C.c_char_p, []),
        "oxhip_stats": (sz, [vp, C.c_char_p, sz]),
        "oxhip_wants": (C.c_int, [vp, sz, sz, sz]),
        "oxhip_upload": (vp, [vp, C.POINTER(WeightDesc)]),
        "oxhip_free_weight": (None, [vp, vp]),
        "oxhip_weight_bytes": (sz, [vp]),
        "oxhip_matmul": (C.c_int, [vp, vp, sz, sz, C.POINTER(Job), sz]),
        "oxhip_dev_quantize_act": (C.c_int, [vp, vp, sz, sz, C.POINTER(QActC), vp]),
        "oxhip_dev_quantize_act_batch": (C.c_int, [vp, C.POINTER(QuantJob), sz, vp]),
        "oxhip_dev_dequantize": (C.c_int, [vp, vp, sz, sz, vp, vp]),
        "oxhip_dev_decode": (C.c_int, [vp, vp, C.POINTER(QActC), vp, sz, vp, vp]),
        "oxhip_dev_decode_noalloc": (C.c_int, [vp, vp, C.POINTER(QActC), sz, vp, vp]),
        "oxhip_dev_isums": (C.c_int, [vp, vp, C.POINTER(QActC), vp, vp]),
        "oxhip_dev_decode_batch": (C.c_int, [vp, C.POINTER(DecodeJob), sz, vp]),
        "oxhip_dev_gemm": (C.c_int, [vp, vp, vp, C.c_int, sz, vp, C.c_int, C.c_int, vp]),
        "oxhip_dev_gemm_timed": (C.c_int, [vp, vp, vp, C.c_int, sz, vp, C.c_int, C.c_int, vp, vp, vp]),
        "oxhip_dev_gemm_isums": (C.c_int, [vp, vp, vp, C.c_int, sz, vp, vp]),
        "oxhip_matvec_rows": (C.c_int, [vp, vp, sz, sz, C.POINTER(RowsJob), sz]),
        "oxhip_upload_moe": (vp, [vp, C.POINTER(WeightDesc), C.POINTER(WeightDesc), C.POINTER(WeightDesc), sz, sz, sz, C.c_uint32, C.c_float]),
        "oxhip_free_moe": (None, [vp, vp]),
        "oxhip_moe_set_mode": (C.c_int, [vp, C.c_uint32]),
        "oxhip_moe_forward": (C.c_int, [vp, vp, sz, sz, sz, vp, vp, sz, vp, vp]),
        "oxhip_dev_route_top_k": (C.c_int, [vp, vp, sz, sz, sz, vp, vp, vp]),
        "oxhip_dev_moe": (C.c_int, [vp, vp, vp, sz, vp, vp, sz, vp, vp]),
        "oxhip_buf_alloc": (vp, [vp, sz]),
        "oxhip_buf_free": (None, [vp, vp]),
        "oxhip_buf_write": (C.c_int, [vp, vp, vp, sz, vp]),
        "oxhip_buf_read": (C.c_int, [vp, vp, vp, sz, vp]),
        "oxhip_dev_rmsnorm_quantize": (C.c_int, [vp, vp, vp, vp, C.c_float, sz, sz, vp, C.POINTER(QActC), vp]),
        "oxhip_dev_norm": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, sz, sz, sz, sz, C.c_float, C.c_int, C.POINTER(QActC), vp]),
        "oxhip_stream_release": (C.c_int, [vp, vp]),
        "oxhip_dev_linear": (C.c_int, [vp, vp, vp, C.POINTER(QActC), vp, sz, vp, C.c_uint32, vp, vp]),
        "oxhip_dev_glu": (C.c_int, [vp, vp, vp, sz, C.c_int, vp, vp]),
        "oxhip_dev_route": (C.c_int, [vp, vp, vp, vp, sz, sz, sz, sz, vp, vp, vp, vp]),
        "oxhip_dev_experts": (C.c_int, [vp, vp, vp, sz, vp, sz, vp, C.c_int, vp]),
        "oxhip_dev_moe_routed": (C.c_int, [vp, vp, vp, sz, vp, sz, sz, vp, vp, vp, C.c_int, vp]),
        "oxhip_plan_begin": (vp, [vp, vp]),
        "oxhip_plan_end": (C.c_int, [vp]),
        "oxhip_plan_launches": (sz, [vp]),
        "oxhip_plan_replay": (C.c_int, [vp, vp]),
        "oxhip_plan_free": (None, [vp]),
        "oxhip_event_create": (vp, []),
        "oxhip_event_destroy": (None, [vp]),
        "oxhip_event_elapsed_ms": (C.c_float, [vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def _np_ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def probe():
    """platform::gpu::cuda::probe for HIP devices (src/platform.rs:446-482): a list of dicts like `GpuInfo`."""
    lib = load_library()
    arr = (GpuInfo * 16)()
    n = lib.oxhip_probe(arr, 16)
    return [dict(kind="hip", index=g.index, name=g.name.decode(), arch=g.arch.decode(), memory_bytes=int(g.memory_bytes),
                 driver=g.driver.decode(), usable=bool(g.usable)) for g in arr[:min(n, 16)]]


class DeviceWeight:
    """`gpu::DeviceWeight` of one matrix (src/gpu.rs:57): freed when dropped."""

    def __init__(self, be, handle, n_out, n_in):
        self.be, self.handle, self.n_out, self.n_in = be, handle, n_out, n_in

    @property
    def bytes(self):
        return load_library().oxhip_weight_bytes(self.handle)

    def __del__(self):
        if getattr(self, "handle", None) and self.be.ctx:
            load_library().oxhip_free_weight(self.be.ctx, self.handle)
            self.handle = None


class DeviceMoe:
    """`DeviceWeight` of the routed experts of one MoE layer (Backend::upload_moe, src/gpu.rs:206-216)."""

    def __init__(self, be, handle, n_exp, h, inter):
        self.be, self.handle, self.n_exp, self.h, self.inter = be, handle, n_exp, h, inter

    def set_mode(self, mode):
        """MOE_AUTO: the reference's split by pass size; MOE_INT8: the integer kernels at every size."""
        if not load_library().oxhip_moe_set_mode(self.handle, mode):
            raise RuntimeError(self.be.last_error())

    def __del__(self):
        if getattr(self, "handle", None) and self.be.ctx:
            load_library().oxhip_free_moe(self.be.ctx, self.handle)
            self.handle = None


class Plan:
    """A recorded chain of device-pointer ops (oxhip_plan_*): the matmul side of `DecodePlan` (src/gpu_decode.rs:572-587)."""

    def __init__(self, be, handle):
        self.be, self.handle = be, handle

    @property
    def launches(self):
        return load_library().oxhip_plan_launches(self.handle)

    def replay(self, stream=None):
        if not load_library().oxhip_plan_replay(self.handle, C.c_void_p(stream) if stream else None):
            raise RuntimeError(self.be.last_error())

    def __del__(self):
        if getattr(self, "handle", None):
            load_library().oxhip_plan_free(self.handle)
            self.handle = None


ACT_SILU, ACT_GELU_TANH, ACT_SILU_CLAMP = 0, 1, 2
MOE_AUTO, MOE_INT8 = 0, 1
LIN_STORE, LIN_ADD, LIN_SILU_PAIR, LIN_GELU_PAIR, LIN_ADD_GATED = 0, 1, 2, 3, 4


class QAct:
    """`quant::QAct` (src/quant.rs:222-238) in device memory (torch tensors)."""

    def __init__(self, t, n_in, device):
        import torch
        self.t, self.n_in = t, n_in
        self.q = torch.empty((t, n_in), dtype=torch.int8, device=device)
        self.scales = torch.empty((t, n_in // 32), dtype=torch.float32, device=device)
        self.sums = torch.empty((t, n_in // 32), dtype=torch.int32, device=device)
        self.fsums = torch.empty((t, n_in // 32), dtype=torch.float32, device=device)
        self.hsums = torch.empty((t, n_in // 16), dtype=torch.float32, device=device)
        self.sums16 = torch.empty((t, n_in // 16), dtype=torch.int32, device=device)
        self.c = QActC(self.q.data_ptr(), self.scales.data_ptr(), self.sums.data_ptr(), self.fsums.data_ptr(),
                       self.hsums.data_ptr(), self.sums16.data_ptr(), t, n_in)


class HipBackend:
    """Mirror of `impl Backend for CudaBackend` (src/cuda.rs) over the HIP library."""

    def __init__(self, device=0):
        self.lib = load_library()
        ctx = C.c_void_p()
        if not self.lib.oxhip_open(device, C.byref(ctx)):
            raise RuntimeError("device hip: " + self.last_error())
        self.ctx = ctx
        self.device = device

    def close(self):
        if self.ctx:
            self.lib.oxhip_close(self.ctx)
            self.ctx = None

    def last_error(self):
        return (self.lib.oxhip_last_error() or b"").decode()

    # ---- Backend surface -------------------------------------------------------------------
    def name(self):
        return self.lib.oxhip_name(self.ctx).decode()

    def wants(self, n_out, n_in, t):
        return bool(self.lib.oxhip_wants(self.ctx, n_out, n_in, t))

    def stats(self):
        buf = C.create_string_buffer(256)
        self.lib.oxhip_stats(self.ctx, buf, 256)
        return buf.value.decode()

    def _upload(self, desc, keep):
        h = self.lib.oxhip_upload(self.ctx, C.byref(desc))
        del keep
        return DeviceWeight(self, h, desc.n_out, desc.n_in) if h else None

    @staticmethod
    def desc_gguf(ggml_type, data, n_out, n_in):
        data = np.ascontiguousarray(data, np.uint8)
        return WeightDesc(kind=W_GGUF, ggml_type=ggml_type, n_out=n_out, n_in=n_in, data=_np_ptr(data)), (data,)

    @staticmethod
    def desc_mlx_q4(w, scales, biases, group, n_out, n_in):
        w = np.ascontiguousarray(w, np.uint32)
        scales, biases = np.ascontiguousarray(scales, np.uint16), np.ascontiguousarray(biases, np.uint16)
        return (WeightDesc(kind=W_MLX_Q4, n_out=n_out, n_in=n_in, data=_np_ptr(w), scales=_np_ptr(scales), offsets=_np_ptr(biases),
                           group=group), (w, scales, biases))

    def upload_moe(self, gate_up, down, h, inter, up=None, act=ACT_SILU, act_param=0.0):
        """Backend::upload_moe: gate_up / down (/ up) are lists of (WeightDesc, keepalive) per expert."""
        n = len(gate_up)

        def arr(ds):
            a = (WeightDesc * n)()
            for i, (d, _) in enumerate(ds):
                a[i] = d
            return a
        hnd = self.lib.oxhip_upload_moe(self.ctx, arr(gate_up), arr(up) if up else None, arr(down), n, h, inter, act, act_param)
        return DeviceMoe(self, hnd, n, h, inter) if hnd else None

    def moe(self, x, t, h, inter, route_idx, route_w, k, dev, y):
        """Backend::moe: adds the routed experts' output into y ([t, h] f32, host). False = declined, y untouched."""
        x = np.ascontiguousarray(x, np.float32)
        ri, rw = np.ascontiguousarray(route_idx, np.uint32), np.ascontiguousarray(route_w, np.float32)
        assert y.dtype == np.float32 and y.flags.c_contiguous
        return bool(self.lib.oxhip_moe_forward(self.ctx, _np_ptr(x), t, h, inter, _np_ptr(ri), _np_ptr(rw), k, dev.handle, _np_ptr(y)))

    def dev_moe(self, dev, x, route_idx, route_w, y):
        """The same on device tensors: x [t, h] f32, route_idx [t, k] int32 (values as u32), route_w [t, k] f32, y += ."""
        t, k = route_idx.shape
        if not self.lib.oxhip_dev_moe(self.ctx, dev.handle, x.data_ptr(), t, route_idx.data_ptr(), route_w.data_ptr(), k,
                                      y.data_ptr(), self._stream()):
            raise RuntimeError(self.last_error())
        return y

    def route_top_k(self, logits, k):
        """moe::route_top_k on device logits [t, n_experts] -> (idx int32 [t, k], w f32 [t, k])."""
        import torch
        t, n = logits.shape
        idx = torch.empty((t, k), dtype=torch.int32, device=logits.device)
        w = torch.empty((t, k), dtype=torch.float32, device=logits.device)
        if not self.lib.oxhip_dev_route_top_k(self.ctx, logits.data_ptr(), t, n, k, idx.data_ptr(), w.data_ptr(), self._stream()):
            raise RuntimeError(self.last_error())
        return idx, w

    def matvec_rows(self, x, t, n_in, jobs):
        """Backend::matvec_rows: jobs = [(w, up or None, y ndarray [t, n_out])], 1 <= t <= 4."""
        x = np.ascontiguousarray(x, np.float32)
        arr = (RowsJob * len(jobs))()
        for i, (w, up, y) in enumerate(jobs):
            arr[i] = RowsJob(w.handle, up.handle if up is not None else None, w.n_out, y.ctypes.data)
        return bool(self.lib.oxhip_matvec_rows(self.ctx, _np_ptr(x), t, n_in, arr, len(jobs)))

    def upload_gguf(self, ggml_type, data, n_out, n_in):
        """WeightRef::Gguf: raw blocks, rows of `row_bytes` (src/ggml.rs:240-248)."""
        data = np.ascontiguousarray(data, np.uint8)
        bs, ts = GGML_BLOCK.get(ggml_type, (1, 0))
        if ts and data.size != n_out * (n_in // bs) * ts:
            raise ValueError("GGUF byte count does not match the shape")
        d = WeightDesc(kind=W_GGUF, ggml_type=ggml_type, n_out=n_out, n_in=n_in, data=_np_ptr(data))
        return self._upload(d, data)

    def upload_fp8(self, data, block_scales, n_out, n_in, block=(128, 128)):
        """GgufMatrix::fp8 (src/ggml.rs:325-341)."""
        data = np.ascontiguousarray(data, np.uint8)
        bs = np.ascontiguousarray(block_scales, np.float32)
        d = WeightDesc(kind=W_GGUF, ggml_type=GGML_F8E4M3, n_out=n_out, n_in=n_in, data=_np_ptr(data),
                       block_scales=_np_ptr(bs), bs_rows=block[0], bs_cols=block[1])
        return self._upload(d, (data, bs))

    def upload_nvfp4(self, data, n_out, n_in, scales=None, block=None):
        """GgufMatrix of NVFP4 blocks (src/ggml.rs:79-83) with, optionally, the matrix's scales on top (`block` = rows x
        columns per scale; default one scale for the matrix, as model::nvfp4_blocks builds it)."""
        data = np.ascontiguousarray(data, np.uint8)
        if data.size != n_out * (n_in // 64) * 36:
            raise ValueError("NVFP4 byte count does not match the shape")
        bs = None if scales is None else np.ascontiguousarray(np.atleast_1d(scales), np.float32)
        br, bc = block or (n_out, n_in)
        d = WeightDesc(kind=W_GGUF, ggml_type=GGML_NVFP4, n_out=n_out, n_in=n_in, data=_np_ptr(data), block_scales=_np_ptr(bs),
                       bs_rows=br if bs is not None else 0, bs_cols=bc if bs is not None else 0)
        return self._upload(d, (data, bs))

    def upload_q8(self, q, scales, n_out, n_in):
        """WeightRef::Q8 (QMatrix, src/quant.rs:128-133): int8 codes, one f32 scale per block of 32."""
        q, scales = np.ascontiguousarray(q, np.int8), np.ascontiguousarray(scales, np.float32)
        d = WeightDesc(kind=W_Q8, n_out=n_out, n_in=n_in, data=_np_ptr(q), scales=_np_ptr(scales))
        return self._upload(d, (q, scales))

    def upload_q4(self, q, scales, offsets, group, n_out, n_in):
        """WeightRef::Q4 (src/quant.rs:427-440): nibbles, f16 scales per 32, optional bf16 offsets."""
        q, scales = np.ascontiguousarray(q, np.uint8), np.ascontiguousarray(scales, np.uint16)
        offsets = None if offsets is None else np.ascontiguousarray(offsets, np.uint16)
        d = WeightDesc(kind=W_Q4, n_out=n_out, n_in=n_in, data=_np_ptr(q), scales=_np_ptr(scales),
                       offsets=_np_ptr(offsets), group=group if offsets is not None else 0)
        return self._upload(d, (q, scales, offsets))

    def upload_mlx_q4(self, w, scales, biases, group, n_out, n_in):
        """The MLX triplet; the device does what from_mlx_q4 does (src/quant.rs:518-563)."""
        w = np.ascontiguousarray(w, np.uint32)
        scales, biases = np.ascontiguousarray(scales, np.uint16), np.ascontiguousarray(biases, np.uint16)
        d = WeightDesc(kind=W_MLX_Q4, n_out=n_out, n_in=n_in, data=_np_ptr(w), scales=_np_ptr(scales),
                       offsets=_np_ptr(biases), group=group)
        return self._upload(d, (w, scales, biases))

    def upload_bf16(self, w, n_out, n_in):
        w = np.ascontiguousarray(w, np.uint16)
        d = WeightDesc(kind=W_BF16, n_out=n_out, n_in=n_in, data=_np_ptr(w))
        return self._upload(d, w)

    def matmul(self, x, t, n_in, jobs):
        """Backend::matmul: jobs = [(DeviceWeight, y ndarray [t, n_out] f32)]; True if every y was written."""
        x = np.ascontiguousarray(x, np.float32)
        arr = (Job * len(jobs))()
        for i, (w, y) in enumerate(jobs):
            assert y.dtype == np.float32 and y.flags.c_contiguous
            arr[i] = Job(w.handle, w.n_out, y.ctypes.data)
        return bool(self.lib.oxhip_matmul(self.ctx, _np_ptr(x), t, n_in, arr, len(jobs)))

    # ---- device-pointer entry points -------------------------------------------------------
    @staticmethod
    def _stream():
        import torch
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def quantize_act(self, x, out=None):
        """x: torch f32 [t, n_in] on the device -> QAct (device)."""
        t, n_in = x.shape
        out = out or QAct(t, n_in, x.device)
        if not self.lib.oxhip_dev_quantize_act(self.ctx, x.data_ptr(), t, n_in, C.byref(out.c), self._stream()):
            raise RuntimeError(self.last_error())
        return out

    def quantize_jobs(self, pairs):
        """A reusable job array for quantize_act_batch: pairs = [(x f32 [t, n_in] on the device, QAct)]."""
        arr = (QuantJob * len(pairs))()
        for i, (x, out) in enumerate(pairs):
            arr[i] = QuantJob(x.data_ptr(), x.shape[0], x.shape[1], C.addressof(out.c))
        return arr

    def quantize_act_batch(self, arr):
        if not self.lib.oxhip_dev_quantize_act_batch(self.ctx, arr, len(arr), self._stream()):
            raise RuntimeError(self.last_error())

    def dequantize(self, w, r0=0, r1=None):
        import torch
        r1 = w.n_out if r1 is None else r1
        out = torch.empty((r1 - r0, w.n_in), dtype=torch.float32, device=f"cuda:{self.device}")
        if not self.lib.oxhip_dev_dequantize(self.ctx, w.handle, r0, r1, out.data_ptr(), self._stream()):
            raise RuntimeError(self.last_error())
        return out

    def decode(self, w, xa=None, x=None, t=None, y=None):
        """The decode kernels on device buffers: xa (QAct) for quantized weights, x (f32) for float-stored ones."""
        import torch
        t = t or (xa.t if xa is not None else x.shape[0])
        if y is None:
            y = torch.empty((t, w.n_out), dtype=torch.float32, device=f"cuda:{self.device}")
        ok = self.lib.oxhip_dev_decode(self.ctx, w.handle, C.byref(xa.c) if xa is not None else None,
                                       x.data_ptr() if x is not None else None, t, y.data_ptr(), self._stream())
        if not ok:
            raise RuntimeError(self.last_error())
        return y

    def decode_noalloc(self, w, xa, t=None, y=None):
        """oxhip_dev_decode_noalloc: the decode kernels over the library's static scratch. False = declined."""
        import torch
        t = t or xa.t
        if y is None:
            y = torch.empty((t, w.n_out), dtype=torch.float32, device=f"cuda:{self.device}")
        ok = self.lib.oxhip_dev_decode_noalloc(self.ctx, w.handle, C.byref(xa.c), t, y.data_ptr(), self._stream())
        return y if ok else None

    # ---- decode-graph ops (device tensors; Op::Norm / Linear / Route / Experts of src/gpu_decode.rs) -----------
    def rmsnorm_quantize(self, x, w=None, eps=1e-6, want_out=True, want_q=True):
        """x [t, n] f32 -> (normed [t, n] f32 or None, QAct or None); w: f32 or bf16 device tensor [n], or None."""
        import torch
        t, n = x.shape
        out = torch.empty_like(x) if want_out else None
        q = QAct(t, n, x.device) if want_q else None
        wf = w.data_ptr() if w is not None and w.dtype == torch.float32 else None
        wb = w.data_ptr() if w is not None and w.dtype == torch.bfloat16 else None
        ok = self.lib.oxhip_dev_rmsnorm_quantize(self.ctx, x.data_ptr(), wf, wb, eps, t, n, out.data_ptr() if want_out else None,
                                                 C.byref(q.c) if want_q else None, self._stream())
        if not ok:
            raise RuntimeError(self.last_error())
        return out, q

    def norm(self, x, n, rows, out=None, w=None, pre=1.0, x_stride=0, out_stride=0, eps=1e-6, add=False, want_q=False):
        """Op::Norm with all its fields on device tensors (x, out: f32, any float offset into a larger buffer)."""
        import torch
        q = QAct(rows, n, x.device) if want_q else None
        wf = w.data_ptr() if w is not None and w.dtype == torch.float32 else None
        wb = w.data_ptr() if w is not None and w.dtype == torch.bfloat16 else None
        ok = self.lib.oxhip_dev_norm(self.ctx, x.data_ptr(), out.data_ptr() if out is not None else None, wf, wb, pre, n, rows, x_stride,
                                     out_stride, eps, int(add), C.byref(q.c) if want_q else None, self._stream())
        return (bool(ok), q)

    def stream_release(self, stream):
        return bool(self.lib.oxhip_stream_release(self.ctx, C.c_void_p(stream)))

    def linear(self, w, y, xa=None, x=None, t=None, mode=LIN_STORE, w2=None, gate=None):
        """Op::Linear on device tensors; y [t, n_out] f32 is written or added to according to `mode`. False = declined."""
        t = t or (xa.t if xa is not None else x.shape[0])
        return bool(self.lib.oxhip_dev_linear(self.ctx, w.handle, w2.handle if w2 is not None else None,
                                              C.byref(xa.c) if xa is not None else None, x.data_ptr() if x is not None else None, t,
                                              y.data_ptr(), mode, gate.data_ptr() if gate is not None else None, self._stream()))

    def glu(self, g, u, gelu=False):
        import torch
        y = torch.empty_like(g)
        if not self.lib.oxhip_dev_glu(self.ctx, g.data_ptr(), u.data_ptr(), g.numel(), int(gelu), y.data_ptr(), self._stream()):
            raise RuntimeError(self.last_error())
        return y

    def route(self, x, router, k, gate=None, expert_scale=None):
        """Op::Route: x [t, h], router [n_exp, h] f32 -> (logits [t, n_exp (+1)], sel int32 [2, t, k]: ids, then weight bits)."""
        import torch
        t, h = x.shape
        n_exp = router.shape[0]
        logits = torch.empty((t, n_exp + (1 if gate is not None else 0)), dtype=torch.float32, device=x.device)
        sel = torch.empty((2, t, k), dtype=torch.int32, device=x.device)
        ok = self.lib.oxhip_dev_route(self.ctx, x.data_ptr(), router.data_ptr(), gate.data_ptr() if gate is not None else None, t, n_exp, h, k,
                                      logits.data_ptr(), sel.data_ptr(), expert_scale.data_ptr() if expert_scale is not None else None, self._stream())
        if not ok:
            raise RuntimeError(self.last_error())
        return logits, sel

    def experts(self, dev, x, sel, y, add=True):
        """Op::Experts: the experts chosen in `sel` (as route() returns it) over x [t, h]; y += or y =."""
        _, t, k = sel.shape
        return bool(self.lib.oxhip_dev_experts(self.ctx, dev.handle, x.data_ptr(), t, sel.data_ptr(), k, y.data_ptr(), int(add), self._stream()))

    def moe_routed(self, dev, x, logits, k, y, sel=None, add=True, expert_scale=None):
        """Top-k of `logits` [t, n_exp (+...)] and the routed experts over x [t, h] in one call; returns sel [2, t, k]."""
        import torch
        t = x.shape[0]
        if sel is None:
            sel = torch.empty((2, t, k), dtype=torch.int32, device=x.device)
        ok = self.lib.oxhip_dev_moe_routed(self.ctx, dev.handle, x.data_ptr(), t, logits.data_ptr(), logits.shape[1], k,
                                           expert_scale.data_ptr() if expert_scale is not None else None, sel.data_ptr(), y.data_ptr(),
                                           int(add), self._stream())
        if not ok:
            raise RuntimeError(self.last_error())
        return sel

    def plan_record(self, chain):
        """Records chain() (device-pointer calls on the current torch stream, which must not be the null stream) and
        returns a Plan; raises when the recording fails. Run chain() once on that stream beforehand."""
        h = self.lib.oxhip_plan_begin(self.ctx, self._stream())
        if not h:
            raise RuntimeError(self.last_error())
        try:
            chain()
        except BaseException:
            self.lib.oxhip_plan_free(h)
            raise
        if not self.lib.oxhip_plan_end(h):
            msg = self.last_error()
            self.lib.oxhip_plan_free(h)
            raise RuntimeError(msg)
        return Plan(self, h)

    def decode_jobs(self, jobs):
        """Builds a reusable job array for decode_batch: jobs = [(DeviceWeight, QAct | None, x | None, t, y, ev0, ev1)]."""
        arr = (DecodeJob * len(jobs))()
        for i, (w, xa, x, t, y, e0, e1) in enumerate(jobs):
            arr[i] = DecodeJob(w.handle, C.addressof(xa.c) if xa is not None else None,
                               x.data_ptr() if x is not None else None, t, y.data_ptr(), e0, e1)
        return arr

    def decode_batch(self, arr):
        if not self.lib.oxhip_dev_decode_batch(self.ctx, arr, len(arr), self._stream()):
            raise RuntimeError(self.last_error())

    def event(self):
        e = self.lib.oxhip_event_create()
        if not e:
            raise RuntimeError(self.last_error())
        return e

    def elapsed_ms(self, a, b):
        return self.lib.oxhip_event_elapsed_ms(a, b)

    def gemm(self, w, x, variant=0, out_bf16=False, events=None):
        """Prefill GEMM on device tensors: x [t, n_in] f32 or bf16 -> y [t, n_out] f32 (or bf16). `events`: a pair from
        event() that the library records right before and after the variant's matrix kernel."""
        import torch
        t = x.shape[0]
        y = torch.empty((t, w.n_out), dtype=torch.bfloat16 if out_bf16 else torch.float32, device=x.device)
        xd = 1 if x.dtype == torch.bfloat16 else 0
        assert x.dtype in (torch.bfloat16, torch.float32) and x.is_contiguous()
        if events is None:
            ok = self.lib.oxhip_dev_gemm(self.ctx, w.handle, x.data_ptr(), xd, t, y.data_ptr(), int(out_bf16), variant, self._stream())
        else:
            ok = self.lib.oxhip_dev_gemm_timed(self.ctx, w.handle, x.data_ptr(), xd, t, y.data_ptr(), int(out_bf16), variant, self._stream(),
                                               events[0], events[1])
        if not ok:
            raise RuntimeError(self.last_error())
        return y

    def gemm_isums(self, w, x):
        """The int8 GEMM's exact block sums [t, n_out, n_in/32] (int32)."""
        import torch
        t = x.shape[0]
        out = torch.zeros((t, w.n_out, w.n_in // 32), dtype=torch.int32, device=x.device)
        xd = 1 if x.dtype == torch.bfloat16 else 0
        assert x.dtype in (torch.bfloat16, torch.float32) and x.is_contiguous()
        if not self.lib.oxhip_dev_gemm_isums(self.ctx, w.handle, x.data_ptr(), xd, t, out.data_ptr(), self._stream()):
            raise RuntimeError(self.last_error())
        return out

    def isums(self, w, xa, per):
        import torch
        out = torch.empty((xa.t, w.n_out, w.n_in // per), dtype=torch.int32, device=f"cuda:{self.device}")
        if not self.lib.oxhip_dev_isums(self.ctx, w.handle, C.byref(xa.c), out.data_ptr(), self._stream()):
            raise RuntimeError(self.last_error())
        return out
