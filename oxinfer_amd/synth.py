"""Seeded synthetic tensors of the benchmark configurations (numpy on the host).

Weights are produced in the layouts the reference's loaders hand to a backend: the MLX triplet
(`weight` u32, `scales` / `biases` bf16), raw GGUF blocks, FP8 bytes with 128x128 f32 block scales.
"""
import numpy as np


def bf16_bits(x):
    """f32 -> bf16 bits, round to nearest even."""
    b = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_round(x):
    """f32 values rounded to bf16, as f32."""
    return (bf16_bits(x).astype(np.uint32) << 16).view(np.float32)


def mlx_q4(n_out, n_in, seed, group=64):
    """MLX affine 4-bit: nibbles uniform 0..15 (8 per little-endian u32, low nibble first), per group of 64
    bf16 scale = |N(0, 0.02)| / 7.5 and bf16 bias = -8 * scale. Returns (w u32, scales u16, biases u16)."""
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 1 << 32, (n_out, n_in // 8), dtype=np.uint64).astype(np.uint32)
    s = np.abs(rng.normal(0.0, 0.02, (n_out, n_in // group))).astype(np.float32) / np.float32(7.5)
    sb = bf16_bits(s)
    sf = (sb.astype(np.uint32) << 16).view(np.float32)
    bb = bf16_bits(np.float32(-8.0) * sf)  # exact: a power of two times a bf16
    return w, sb, bb


def q8_matrix(n_out, n_in, seed):
    """QMatrix (src/quant.rs:128-133): int8 codes uniform in [-127, 127], f32 scale ~ |N(0, 0.01)| per block of 32."""
    rng = np.random.default_rng(seed)
    q = rng.integers(-127, 128, (n_out, n_in), dtype=np.int8)
    scales = np.abs(rng.normal(0.0, 0.01, (n_out, n_in // 32))).astype(np.float32)
    return q, scales


def gguf_q4_0(n_out, n_in, seed):
    """Q4_0 blocks (18 B): f16 d ~ |N(0, 0.01)|, 32 nibbles uniform (byte j = elements j and j + 16)."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 32
    blk = np.empty((nb, 18), np.uint8)
    blk[:, :2] = np.abs(rng.normal(0.0, 0.01, nb)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blk[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    return blk.reshape(-1)


def gguf_q8_0(n_out, n_in, seed):
    """Q8_0 blocks (34 B): f16 d ~ |N(0, 0.01)|, 32 int8 uniform in [-127, 127]."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 32
    blk = np.empty((nb, 34), np.uint8)
    blk[:, :2] = np.abs(rng.normal(0.0, 0.01, nb)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blk[:, 2:] = rng.integers(-127, 128, (nb, 32), dtype=np.int8).view(np.uint8)
    return blk.reshape(-1)


def pack_k4_scales(sc, mn):
    """The 12 packed bytes of eight 6-bit (scale, min) pairs (inverse of get_scale_min_k4)."""
    sc, mn = sc.astype(np.uint8), mn.astype(np.uint8)
    q = np.empty(sc.shape[:-1] + (12,), np.uint8)
    q[..., 0:4] = sc[..., 0:4] | ((sc[..., 4:8] >> 4) << 6)
    q[..., 4:8] = mn[..., 0:4] | ((mn[..., 4:8] >> 4) << 6)
    q[..., 8:12] = (sc[..., 4:8] & 0xF) | ((mn[..., 4:8] & 0xF) << 4)
    return q


def gguf_q4_k(n_out, n_in, seed):
    """Q4_K super-blocks (144 B): f16 d, dmin ~ |N(0, 0.005)|, 6-bit scales / mins uniform, nibbles uniform."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 256
    blk = np.empty((nb, 144), np.uint8)
    blk[:, 0:2] = np.abs(rng.normal(0.0, 0.005, nb)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blk[:, 2:4] = np.abs(rng.normal(0.0, 0.005, nb)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blk[:, 4:16] = pack_k4_scales(rng.integers(0, 64, (nb, 8)), rng.integers(0, 64, (nb, 8)))
    blk[:, 16:] = rng.integers(0, 256, (nb, 128), dtype=np.uint8)
    return blk.reshape(-1)


def gguf_q5_k(n_out, n_in, seed):
    """Q5_K super-blocks (176 B): the Q4_K header, then 32 bytes of fifth bits and 128 of nibbles, uniform."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 256
    blk = np.empty((nb, 176), np.uint8)
    blk[:, 0:2] = np.abs(rng.normal(0.0, 0.005, nb)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blk[:, 2:4] = np.abs(rng.normal(0.0, 0.005, nb)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blk[:, 4:16] = pack_k4_scales(rng.integers(0, 64, (nb, 8)), rng.integers(0, 64, (nb, 8)))
    blk[:, 16:] = rng.integers(0, 256, (nb, 160), dtype=np.uint8)
    return blk.reshape(-1)


def gguf_mxfp4(n_out, n_in, seed):
    """MXFP4 blocks (17 B): an E8M0 scale byte 2^-12..2^-5 (as half values), 16 bytes of E2M1 codes, uniform."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 32
    blk = rng.integers(0, 256, (nb, 17), dtype=np.uint8)
    blk[:, 0] = rng.integers(116, 124, nb, dtype=np.uint8)
    return blk.reshape(-1)


def gguf_nvfp4(n_out, n_in, seed):
    """NVFP4 blocks of 64 in ggml's layout (36 B: four unsigned E4M3 scale bytes, one per 16 values, then 4 x 8 bytes of
    E2M1 codes, uniform; src/ggml.rs:936-947), scales 2^-9 .. 2^-3 with random mantissas (a few zero), and a global f32
    scale as compressed-tensors checkpoints carry it. Returns (bytes, global scale)."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 64
    blk = rng.integers(0, 256, (nb, 36), dtype=np.uint8)
    sc = (rng.integers(0, 7, (nb, 4)) << 3 | rng.integers(0, 8, (nb, 4))).astype(np.uint8)
    sc[rng.random((nb, 4)) < 0.01] = 0
    blk[:, :4] = sc
    return blk.reshape(-1), np.float32(abs(rng.normal(0.0, 0.5)) + 0.25)


def gguf_q6_k(n_out, n_in, seed):
    """Q6_K super-blocks (210 B): ql, qh uniform bits, int8 scales uniform, f16 d ~ +-|N(0, 0.005)|."""
    rng = np.random.default_rng(seed)
    nb = n_out * n_in // 256
    blk = rng.integers(0, 256, (nb, 210), dtype=np.uint8)
    blk[:, 208:210] = rng.normal(0.0, 0.005, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    return blk.reshape(-1)


def fp8_e4m3(n_out, n_in, seed, block=(128, 128)):
    """FP8 E4M3 weights: N(0, 1) rounded (RNE) and saturated to e4m3 (never a NaN byte), with f32 block scales
    ~ |N(0, 0.01)| per 128x128. Returns (bytes [n_out, n_in], scales [ceil(n_out/128), ceil(n_in/128)])."""
    import torch
    g = torch.Generator().manual_seed(seed)
    v = torch.randn((n_out, n_in), generator=g, dtype=torch.float32).clamp_(-448.0, 448.0)
    b = v.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    rng = np.random.default_rng(seed + 1)
    s = np.abs(rng.normal(0.0, 0.01, (-(-n_out // block[0]), -(-n_in // block[1])))).astype(np.float32)
    return b, s


def activations(t, n_in, seed, bf16=False):
    """[t, n_in] f32 ~ N(0, 1); bf16=True rounds them to bf16-representable values."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0.0, 1.0, (t, n_in)).astype(np.float32)
    return bf16_round(x) if bf16 else x


def router_logits(t, n_experts, seed):
    rng = np.random.default_rng(seed)
    return rng.normal(0.0, 1.0, (t, n_experts)).astype(np.float32)
