// Dequantization to f32 (bit-identical to the reference's CPU dequantizers) and the upload-time
// repacking kernels.
//
// Reference formulas, reproduced operation by operation (no fused multiply-add: this file is
// compiled with -ffp-contract=off):
//   Q4    ((nib - 8) as f32) * d + m                      src/quant.rs:586-606
//   Q8_0  (q as f32) * d                                  src/ggml.rs:707-712
//   Q4_K  (d * sc) * v - (dmin * mn), v the raw nibble    src/ggml.rs:750-773
//   Q6_K  (d * sc) * q, q = 6-bit code - 32               src/ggml.rs:774-793
//   FP8   e4m3(byte) * block scale                        src/ggml.rs:282-293, :433-444
//   MLX 4-bit -> Q4 + offsets                             src/quant.rs:518-563
#include "internal.hpp"

namespace oxhip {

__global__ __launch_bounds__(256) void dequantize_kernel(WeightView w, uint32_t r0, size_t total, float* __restrict__ out) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const uint32_t n = w.n_in;
    const uint32_t c = idx % n;
    const size_t r = r0 + idx / n;
    float v = 0.0f;
    switch (w.fmt) {
        case FMT_Q4: {
            uint32_t b = c / 32, j = c % 32;
            uint8_t byte = w.p0[r * (n / 2) + b * 16 + (j & 15)];
            int nib = j < 16 ? (byte & 0x0F) : (byte >> 4);
            float d = f16_bits_to_f32(reinterpret_cast<const uint16_t*>(w.p1)[r * (n / w.sgroup) + c / w.sgroup]);
            float m = w.group ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(w.p2)[r * (n / w.group) + c / w.group]) : 0.0f;
            v = (float)(nib - 8) * d + m;
            break;
        }
        case FMT_Q8_0: {
            float d = f16_bits_to_f32(reinterpret_cast<const uint16_t*>(w.p1)[r * (n / 32) + c / 32]);
            v = (float)reinterpret_cast<const int8_t*>(w.p0)[r * n + c] * d;
            break;
        }
        case FMT_Q4_K: {
            size_t nb = n / 256;
            uint32_t sb = c / 256, e = c % 256, j = e / 64, h = (e % 64) / 32, l = e % 32;
            uint8_t byte = w.p0[(r * nb + sb) * 128 + 32 * j + l];
            uint32_t q = (byte >> (4 * h)) & 0xF;
            uint4 mt = *reinterpret_cast<const uint4*>(w.p1 + (r * nb + sb) * 16);
            float d = f16_bits_to_f32((uint16_t)(mt.x & 0xFFFF)), dmin = f16_bits_to_f32((uint16_t)(mt.x >> 16));
            uint32_t sc, mn;
            scale_min_k4(2 * j + h, mt.y, mt.z, mt.w, sc, mn);
            float d1 = d * (float)sc, m1 = dmin * (float)mn;
            v = d1 * (float)q - m1;
            break;
        }
        case FMT_Q6_K: {
            size_t nb = n / 256;
            uint32_t sb = c / 256, e = c % 256, nn = e / 128, k = (e % 128) / 32, l = e % 32, is = l / 16;
            const uint8_t* ql = w.p0 + (r * nb + sb) * 128 + 64 * nn;
            uint8_t qh = w.p1[(r * nb + sb) * 64 + 32 * nn + l];
            uint8_t lo = ql[l + 32 * (k & 1)];
            int q = (int)((k < 2 ? (lo & 0xF) : (lo >> 4)) | (((qh >> (2 * k)) & 3) << 4)) - 32;
            float sc = (float)reinterpret_cast<const int8_t*>(w.p2)[(r * nb + sb) * 16 + 8 * nn + is + 2 * k];
            float d = f16_bits_to_f32(reinterpret_cast<const uint16_t*>(w.p3)[r * nb + sb]);
            v = d * sc * (float)q;
            break;
        }
        case FMT_FP8: {
            uint32_t ncb = (n + w.bc - 1) / w.bc;
            float s = reinterpret_cast<const float*>(w.p1)[(r / w.br) * ncb + c / w.bc];
            v = e4m3_to_f32(w.p0[r * n + c]) * s;
            break;
        }
        case FMT_BF16: v = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(w.p0)[r * n + c]); break;
        default: break;
    }
    out[idx] = v;
}

hipError_t launch_dequantize(const WeightView& w, size_t r0, size_t r1, float* out, hipStream_t s) {
    size_t total = (r1 - r0) * (size_t)w.n_in;
    if (!total) return hipSuccess;
    dequantize_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(w, (uint32_t)r0, total, out);
    return hipGetLastError();
}

// ---- upload-time repacking ---------------------------------------------------------------------
// One thread per source block; runs once per matrix.
__global__ __launch_bounds__(256) void repack_gguf_kernel(int fmt, const uint8_t* __restrict__ raw, size_t nblocks, uint8_t* p0,
                                                          uint8_t* p1, uint8_t* p2, uint8_t* p3) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    if (fmt == FMT_Q8_0) {
        const uint8_t* s = raw + b * 34;
        p1[2 * b] = s[0];
        p1[2 * b + 1] = s[1];
        for (int i = 0; i < 32; i++) p0[b * 32 + i] = s[2 + i];
    } else if (fmt == FMT_Q4_K) {
        const uint8_t* s = raw + b * 144;
        for (int i = 0; i < 16; i++) p1[b * 16 + i] = s[i];
        for (int i = 0; i < 128; i++) p0[b * 128 + i] = s[16 + i];
    } else if (fmt == FMT_Q6_K) {
        const uint8_t* s = raw + b * 210;
        for (int i = 0; i < 128; i++) p0[b * 128 + i] = s[i];
        for (int i = 0; i < 64; i++) p1[b * 64 + i] = s[128 + i];
        for (int i = 0; i < 16; i++) p2[b * 16 + i] = s[192 + i];
        p3[2 * b] = s[208];
        p3[2 * b + 1] = s[209];
    }
}

hipError_t launch_repack_gguf(int fmt, const uint8_t* raw, size_t n_out, size_t n_in, const WeightView& d, hipStream_t s) {
    size_t bs = fmt == FMT_Q8_0 ? 32 : 256;
    size_t nblocks = n_out * (n_in / bs);
    if (!nblocks) return hipSuccess;
    repack_gguf_kernel<<<(unsigned)((nblocks + 255) / 256), 256, 0, s>>>(fmt, raw, nblocks, const_cast<uint8_t*>(d.p0),
                                                                        const_cast<uint8_t*>(d.p1), const_cast<uint8_t*>(d.p2),
                                                                        const_cast<uint8_t*>(d.p3));
    return hipGetLastError();
}

// from_mlx_q4 (src/quant.rs:518-563): nibbles regrouped so byte j of a 32-block holds elements j and
// j+16; scale = f16(RNE) of the bf16 scale; offset = bf16(RNE) of bias + 8 * scale. One thread per
// block of 32; the first block of a group also writes the group's scale and offset.
__global__ __launch_bounds__(256) void repack_mlx_q4_kernel(const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
                                                            const uint16_t* __restrict__ biases, size_t nblocks, uint32_t bpr,
                                                            uint32_t bpg, uint8_t* __restrict__ q, uint16_t* __restrict__ sc,
                                                            uint16_t* __restrict__ off) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint4 words = *reinterpret_cast<const uint4*>(w + b * 4);
    uint32_t wd[4] = {words.x, words.y, words.z, words.w};
    uint32_t outw[4];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        uint32_t o = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int j = 4 * d + k;  // byte j: element j (low), j + 16 (high)
            uint32_t lo = (wd[j / 8] >> (4 * (j % 8))) & 15;
            uint32_t hi = (wd[(j + 16) / 8] >> (4 * ((j + 16) % 8))) & 15;
            o |= (lo | (hi << 4)) << (8 * k);
        }
        outw[d] = o;
    }
    *reinterpret_cast<uint4*>(q + b * 16) = make_uint4(outw[0], outw[1], outw[2], outw[3]);
    size_t r = b / bpr;
    uint32_t bi = b % bpr;
    if (bi % bpg == 0) {
        size_t g = r * (bpr / bpg) + bi / bpg;
        float s = bf16_bits_to_f32(scales[g]), bias = bf16_bits_to_f32(biases[g]);
        off[g] = f32_to_bf16_bits(bias + 8.0f * s);
        sc[g] = f32_to_f16_bits(s);
    }
}

hipError_t launch_repack_mlx_q4(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, size_t n_out, size_t n_in,
                                size_t group, const WeightView& d, hipStream_t s) {
    size_t nblocks = n_out * (n_in / 32);
    if (!nblocks) return hipSuccess;
    repack_mlx_q4_kernel<<<(unsigned)((nblocks + 255) / 256), 256, 0, s>>>(
        w, scales, biases, nblocks, (uint32_t)(n_in / 32), (uint32_t)(group / 32), const_cast<uint8_t*>(d.p0),
        reinterpret_cast<uint16_t*>(const_cast<uint8_t*>(d.p1)), reinterpret_cast<uint16_t*>(const_cast<uint8_t*>(d.p2)));
    return hipGetLastError();
}

// Q4Matrix scales are stored per block of 32; when every block of an offset group carries the
// same scale (always so after from_mlx_q4) one scale per group is kept. Sets *mismatch otherwise.
__global__ __launch_bounds__(256) void q4_scale_groups_kernel(const uint16_t* __restrict__ sc32, size_t ngroups, uint32_t bpg,
                                                              uint16_t* __restrict__ dst, int* mismatch) {
    size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= ngroups) return;
    uint16_t s = sc32[g * bpg];
    for (uint32_t i = 1; i < bpg; i++)
        if (sc32[g * bpg + i] != s) *mismatch = 1;
    dst[g] = s;
}

hipError_t launch_q4_scale_groups(const uint16_t* sc32, size_t n_out, size_t n_in, size_t sgroup, uint16_t* dst, int* mismatch,
                                  hipStream_t s) {
    size_t ngroups = n_out * (n_in / sgroup);
    if (!ngroups) return hipSuccess;
    q4_scale_groups_kernel<<<(unsigned)((ngroups + 255) / 256), 256, 0, s>>>(sc32, ngroups, (uint32_t)(sgroup / 32), dst, mismatch);
    return hipGetLastError();
}

}  // namespace oxhip
