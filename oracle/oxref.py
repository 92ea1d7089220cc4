"""ctypes binding of the CPU oracle (liboxref.so). TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this module; the product
package never does. All arrays are numpy, C-contiguous.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboxref.so")

F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0 = 0, 1, 2, 3, 6, 7, 8
Q2_K, Q4_K, Q5_K, Q6_K, BF16, MXFP4, NVFP4, F8E4M3 = 10, 12, 13, 14, 30, 39, 40, 0x1000
NAMES = {F32: "F32", F16: "F16", Q4_0: "Q4_0", Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q8_0: "Q8_0",
         Q2_K: "Q2_K", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", BF16: "BF16", MXFP4: "MXFP4"}


def build():
    """Compiles the oracle next to its sources."""
    subprocess.run(["make", "-s", "-C", _HERE, "-B"], check=True)


def _load():
    if not os.path.exists(_SO):
        build()
    lib = C.CDLL(_SO)
    u8p, i8p, u16p, u32p, i32p, f32p = (C.POINTER(t) for t in (C.c_uint8, C.c_int8, C.c_uint16, C.c_uint32, C.c_int32, C.c_float))
    sz, vp = C.c_size_t, C.c_void_p
    sig = {
        "oxref_f16_to_f32": (C.c_float, [C.c_uint16]),
        "oxref_f32_to_f16": (C.c_uint16, [C.c_float]),
        "oxref_f32_to_bf16": (C.c_uint16, [C.c_float]),
        "oxref_bf16_to_f32": (C.c_float, [C.c_uint16]),
        "oxref_block_size": (sz, [C.c_uint32]),
        "oxref_type_size": (sz, [C.c_uint32]),
        "oxref_row_bytes": (sz, [C.c_uint32, sz]),
        "oxref_lcg": (C.c_uint64, [C.POINTER(C.c_uint64)]),
        "oxref_random_blocks": (None, [C.c_uint32, sz, C.POINTER(C.c_uint64), vp]),
        "oxref_fnv1a_f32": (C.c_uint64, [vp, sz]),
        "oxref_dequantize_row": (None, [C.c_uint32, vp, sz, vp]),
        "oxref_decode_i8": (C.c_int, [C.c_uint32, vp, vp, vp, vp]),
        "oxref_e4m3_to_f32": (C.c_float, [C.c_uint8]),
        "oxref_ue4m3_half": (C.c_float, [C.c_uint8]),
        "oxref_gguf_dequant_rows_scaled": (None, [C.c_uint32, vp, vp, sz, sz, sz, sz, sz, vp]),
        "oxref_e4m3_scaled": (None, [vp, sz, C.c_float, vp]),
        "oxref_fp8_dequant_rows": (None, [vp, vp, sz, sz, sz, sz, sz, sz, vp]),
        "oxref_quantize_act": (None, [vp, sz, sz, vp, vp, vp, vp, vp]),
        "oxref_from_mlx_q4": (None, [vp, vp, vp, sz, sz, sz, vp, vp, vp]),
        "oxref_mlx_dequant_row": (None, [vp, vp, vp, sz, sz, sz, vp]),
        "oxref_dequant_rows_q4": (None, [vp, vp, vp, sz, sz, sz, sz, vp]),
        "oxref_q4_decode": (None, [vp, vp, vp, sz, sz, sz, vp, sz, vp, vp]),
        "oxref_q8_dequant_rows": (None, [vp, vp, sz, sz, sz, vp]),
        "oxref_q8_decode": (None, [vp, vp, sz, sz, vp, sz, vp, vp]),
        "oxref_q4_decode_avx2": (None, [vp, vp, vp, sz, sz, sz, vp, sz, vp, C.c_int]),
        "oxref_gguf_decode": (None, [C.c_uint32, vp, sz, sz, vp, sz, vp, vp]),
        "oxref_gguf_decode_avx2": (None, [C.c_uint32, vp, sz, sz, vp, sz, vp, C.c_int]),
        "oxref_gemm_f32": (None, [vp, sz, sz, vp, sz, vp, C.c_int]),
        "oxref_gemm_quant": (None, [C.c_int64, vp, vp, vp, sz, sz, sz, sz, sz, vp, sz, vp, C.c_int]),
        "oxref_i8gemm_q4": (None, [vp, vp, vp, sz, sz, sz, vp, sz, vp, vp]),
        "oxref_fast_exp": (C.c_float, [C.c_float]),
        "oxref_silu_mul": (None, [vp, vp, sz]),
        "oxref_route_top_k": (None, [vp, sz, sz, vp, vp]),
        "oxref_moe_q4": (None, [vp, vp, sz, sz, sz, sz, vp, sz, vp, vp, sz, vp, C.c_int]),
        "oxref_act_apply": (None, [C.c_uint32, C.c_float, vp, vp, sz]),
        "oxref_act_scalar": (C.c_float, [C.c_uint32, C.c_float, C.c_float, C.c_float]),
        "oxref_moe_q4_act": (None, [vp, vp, vp, sz, sz, sz, sz, vp, sz, vp, vp, sz, vp, C.c_int, C.c_uint32, C.c_float]),
        "oxref_moe_q4_avx2": (None, [vp, vp, sz, sz, sz, sz, vp, sz, vp, vp, sz, vp, C.c_int]),
        "oxref_hw_threads": (C.c_int, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


lib = _load()


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def block_size(kind):
    return lib.oxref_block_size(kind)


def type_size(kind):
    return lib.oxref_type_size(kind)


def row_bytes(kind, n):
    return lib.oxref_row_bytes(kind, n)


def hw_threads():
    return lib.oxref_hw_threads()


def random_blocks(kind, nb, seed):
    """Returns (bytes, new_seed): `nb` blocks of `kind` as the reference's fixture generator makes them."""
    s = C.c_uint64(seed)
    out = np.zeros(nb * type_size(kind), np.uint8)
    lib.oxref_random_blocks(kind, nb, C.byref(s), _p(out))
    return out, s.value


def lcg_stream(seed, n):
    s = C.c_uint64(seed)
    out = np.empty(n, np.uint64)
    for i in range(n):
        out[i] = lib.oxref_lcg(C.byref(s))
    return out, s.value


def fnv1a_f32(v):
    v = _c(v, np.float32)
    return lib.oxref_fnv1a_f32(_p(v), v.size)


def dequantize_row(kind, src, n):
    src = _c(src, np.uint8)
    out = np.empty(n, np.float32)
    lib.oxref_dequantize_row(kind, _p(src), n, _p(out))
    return out


def dequantize_rows(kind, data, n_out, n_in):
    return dequantize_row(kind, data, n_out * n_in).reshape(n_out, n_in)


def decode_i8(kind, blk):
    bs = block_size(kind)
    blk = _c(blk, np.uint8)
    q = np.zeros(bs, np.int8)
    s = np.zeros(bs // 16, np.float32)
    m = np.zeros(bs // 16, np.float32)
    has_min = lib.oxref_decode_i8(kind, _p(blk), _p(q), _p(s), _p(m))
    return q, s, m, bool(has_min)


def e4m3_to_f32(b):
    return lib.oxref_e4m3_to_f32(int(b))


def e4m3_scaled(src, s):
    src = _c(src, np.uint8)
    out = np.empty(src.size, np.float32)
    lib.oxref_e4m3_scaled(_p(src), src.size, float(s), _p(out))
    return out


def fp8_dequant_rows(data, scales, n_out, n_in, brows=128, bcols=128, r0=0, r1=None):
    r1 = n_out if r1 is None else r1
    data, scales = _c(data, np.uint8), _c(scales, np.float32)
    out = np.empty((r1 - r0, n_in), np.float32)
    lib.oxref_fp8_dequant_rows(_p(data), _p(scales), n_out, n_in, brows, bcols, r0, r1, _p(out))
    return out


def ue4m3_half(b):
    return lib.oxref_ue4m3_half(int(b))


def gguf_dequant_rows_scaled(kind, data, scales, n_out, n_in, brows=None, bcols=None, r0=0, r1=None):
    """GgufMatrix::dequantize_rows with block scales on top of the kind's own decoding (NVFP4's global scale)."""
    r1 = n_out if r1 is None else r1
    data = _c(data, np.uint8)
    scales = None if scales is None else _c(scales, np.float32)
    out = np.empty((r1 - r0, n_in), np.float32)
    lib.oxref_gguf_dequant_rows_scaled(kind, _p(data), _p(scales), n_in, brows or n_out, bcols or n_in, r0, r1, _p(out))
    return out


def quantize_act(x, t, n_in):
    x = _c(x, np.float32)
    assert x.size == t * n_in and n_in % 32 == 0
    q = np.empty((t, n_in), np.int8)
    scales = np.empty((t, n_in // 32), np.float32)
    sums = np.empty((t, n_in // 32), np.int32)
    fsums = np.empty((t, n_in // 32), np.float32)
    hsums = np.empty((t, n_in // 16), np.float32)
    lib.oxref_quantize_act(_p(x), t, n_in, _p(q), _p(scales), _p(sums), _p(fsums), _p(hsums))
    return q, scales, sums, fsums, hsums


def from_mlx_q4(w, scales, biases, n_out, n_in, group=64):
    w, scales, biases = _c(w, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    q = np.empty((n_out, n_in // 2), np.uint8)
    sc = np.empty((n_out, n_in // 32), np.uint16)
    off = np.empty((n_out, n_in // group), np.uint16)
    lib.oxref_from_mlx_q4(_p(w), _p(scales), _p(biases), n_out, n_in, group, _p(q), _p(sc), _p(off))
    return q, sc, off


def mlx_dequant_rows(w, scales, biases, n_out, n_in, bits=4, group=64):
    w, scales, biases = _c(w, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    out = np.empty((n_out, n_in), np.float32)
    wpr, gpr = n_in * bits // 32, n_in // group
    for r in range(n_out):
        lib.oxref_mlx_dequant_row(_p(w.reshape(-1)[r * wpr:]), _p(scales.reshape(-1)[r * gpr:]),
                                  _p(biases.reshape(-1)[r * gpr:]), bits, group, n_in, _p(out[r]))
    return out


def dequant_rows_q4(q, sc, off, group, n_out, n_in, r0=0, r1=None):
    r1 = n_out if r1 is None else r1
    q, sc = _c(q, np.uint8), _c(sc, np.uint16)
    off = None if off is None else _c(off, np.uint16)
    out = np.empty((r1 - r0, n_in), np.float32)
    lib.oxref_dequant_rows_q4(_p(q), _p(sc), _p(off), group, n_in, r0, r1, _p(out))
    return out


def q4_decode(q, sc, off, group, n_out, n_in, x, t, want_isums=False, avx2=False, threads=1):
    q, sc, x = _c(q, np.uint8), _c(sc, np.uint16), _c(x, np.float32)
    off = None if off is None else _c(off, np.uint16)
    y = np.empty((t, n_out), np.float32)
    if avx2:
        lib.oxref_q4_decode_avx2(_p(q), _p(sc), _p(off), group, n_out, n_in, _p(x), t, _p(y), threads)
        return y
    isums = np.empty((t, n_out, n_in // 32), np.int32) if want_isums else None
    lib.oxref_q4_decode(_p(q), _p(sc), _p(off), group, n_out, n_in, _p(x), t, _p(y), _p(isums))
    return (y, isums) if want_isums else y


def q8_dequant_rows(q, scales, n_out, n_in, r0=0, r1=None):
    """QMatrix rows as f32 (src/quant.rs:405-419)."""
    q, scales = _c(q, np.int8), _c(scales, np.float32)
    r1 = n_out if r1 is None else r1
    out = np.empty((r1 - r0, n_in), np.float32)
    lib.oxref_q8_dequant_rows(_p(q), _p(scales), n_in, r0, r1, _p(out))
    return out


def q8_decode(q, scales, n_out, n_in, x, t, want_isums=False):
    """QMatrix decode product (src/kernels.rs:1156-1167) and, on request, its int32 block sums [t, n_out, n_in/32]."""
    q, scales, x = _c(q, np.int8), _c(scales, np.float32), _c(x, np.float32)
    y = np.empty((t, n_out), np.float32)
    isums = np.empty((t, n_out, n_in // 32), np.int32) if want_isums else None
    lib.oxref_q8_decode(_p(q), _p(scales), n_out, n_in, _p(x), t, _p(y), _p(isums))
    return (y, isums) if want_isums else y


def gguf_decode(kind, data, n_out, n_in, x, t, want_isums=False, avx2=False, threads=1):
    data, x = _c(data, np.uint8), _c(x, np.float32)
    y = np.empty((t, n_out), np.float32)
    if avx2:
        lib.oxref_gguf_decode_avx2(kind, _p(data), n_out, n_in, _p(x), t, _p(y), threads)
        return y
    isums = np.empty((t, n_out, n_in // 16), np.int32) if want_isums else None
    lib.oxref_gguf_decode(kind, _p(data), n_out, n_in, _p(x), t, _p(y), _p(isums))
    return (y, isums) if want_isums else y


def gemm_f32(w, n_out, n_in, x, t, threads=None):
    w, x = _c(w, np.float32), _c(x, np.float32)
    y = np.empty((t, n_out), np.float32)
    lib.oxref_gemm_f32(_p(w), n_out, n_in, _p(x), t, _p(y), threads or hw_threads())
    return y


def gemm_quant(kind, data, aux0, aux1, n_out, n_in, x, t, group=64, brows=128, bcols=128, threads=None):
    """kind: a GGUF id, -1 for Q4 (data=q, aux0=f16 scales, aux1=bf16 offsets), or F8E4M3 (aux0=f32 block scales)."""
    x = _c(x, np.float32)
    y = np.empty((t, n_out), np.float32)
    lib.oxref_gemm_quant(kind, _p(data), _p(aux0), _p(aux1), group, brows, bcols, n_out, n_in, _p(x), t, _p(y),
                         threads or hw_threads())
    return y


def i8gemm_q4(q, sc, off, group, n_out, n_in, x, t, want_isums=False):
    q, sc, x = _c(q, np.uint8), _c(sc, np.uint16), _c(x, np.float32)
    off = None if off is None else _c(off, np.uint16)
    y = np.empty((t, n_out), np.float32)
    isums = np.empty((t, n_out, n_in // 32), np.int32) if want_isums else None
    lib.oxref_i8gemm_q4(_p(q), _p(sc), _p(off), group, n_out, n_in, _p(x), t, _p(y), _p(isums))
    return (y, isums) if want_isums else y


def fast_exp(x):
    return lib.oxref_fast_exp(float(x))


def silu_mul(a, b):
    a = np.array(a, np.float32, copy=True)
    b = _c(b, np.float32)
    lib.oxref_silu_mul(_p(a), _p(b), a.size)
    return a


def act_apply(kind, param, g, u):
    """Act::apply (src/moe.rs:18-37): act(g) * u elementwise; kind 0 SiLU, 1 GELU-tanh, 2 SiLU with clamp `param`."""
    g = np.array(g, np.float32, copy=True)
    u = _c(u, np.float32)
    lib.oxref_act_apply(kind, float(param), _p(g), _p(u), g.size)
    return g


def act_scalar(kind, param, g, u):
    """Act::scalar (src/moe.rs:39-46) of one pair."""
    return lib.oxref_act_scalar(kind, float(param), float(g), float(u))


def route_top_k(logits, k):
    logits = _c(logits, np.float32)
    idx = np.empty(k, np.uint32)
    w = np.empty(k, np.float32)
    lib.oxref_route_top_k(_p(logits), logits.size, k, _p(idx), _p(w))
    return idx, w


class _Q4Ref(C.Structure):
    _fields_ = [("q", C.c_void_p), ("sc", C.c_void_p), ("off", C.c_void_p)]


def moe_q4(gate_up, down, group, h, inter, x, t, route_idx, route_w, y, decode_path, avx2=False, threads=None, up=None, act=0, act_param=0.0):
    """gate_up / down: lists of (q, sc, off) numpy triples per expert. Adds into y ([t, h] f32) and returns it.
    avx2: the decode path scheduled and vectorized as the x86 CPU runs it (the timed baseline). up: split experts
    (gate_up then holds the gates). act / act_param: the layer's MoeAct (0 SiLU, 1 GELU-tanh, 2 SiLU clamp)."""
    ne = len(gate_up)
    keep = []

    def refs(ws):
        arr = (_Q4Ref * ne)()
        for i, (q, sc, off) in enumerate(ws):
            q, sc, off = _c(q, np.uint8), _c(sc, np.uint16), _c(off, np.uint16)
            keep.extend((q, sc, off))
            arr[i] = _Q4Ref(q.ctypes.data, sc.ctypes.data, off.ctypes.data)
        return arr

    gu, dn = refs(gate_up), refs(down)
    upr = refs(up) if up is not None else None
    x = _c(x, np.float32)
    route_idx, route_w = _c(route_idx, np.uint32), _c(route_w, np.float32)
    k = route_idx.size // t
    y = np.array(y, np.float32, copy=True)
    if avx2:
        assert decode_path
        lib.oxref_moe_q4_avx2(gu, dn, ne, group, h, inter, _p(x), t, _p(route_idx), _p(route_w), k, _p(y), threads or hw_threads())
        return y
    lib.oxref_moe_q4_act(gu, upr, dn, ne, group, h, inter, _p(x), t, _p(route_idx), _p(route_w), k, _p(y), int(decode_path), act, float(act_param))
    return y
