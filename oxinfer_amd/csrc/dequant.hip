// Dequantization to f32 (bit-identical to the reference's CPU dequantizers) and the upload-time
// repacking kernels.
//
// Reference formulas, reproduced operation by operation (no fused multiply-add: this file is
// compiled with -ffp-contract=off):
//   Q4    ((nib - 8) as f32) * d + m                      src/quant.rs:586-606
//   Q8_0  (q as f32) * d                                  src/ggml.rs:707-712
//   Q4_K  (d * sc) * v - (dmin * mn), v the raw nibble    src/ggml.rs:750-773
//   Q5_K  the same with v = nibble + 16 * fifth bit       src/ggml.rs:750-773
//   Q6_K  (d * sc) * q, q = 6-bit code - 32               src/ggml.rs:774-793
//   MXFP4 2^(e - 128) * doubled E2M1 value               src/ggml.rs:922-928
//   NVFP4 (ue4m3(scale) / 2) * doubled E2M1 value, then * the matrix's scale   src/ggml.rs:936-947, :420-432
//   FP8   e4m3(byte) * block scale                        src/ggml.rs:282-293, :433-444
//   MLX 4-bit -> Q4 + offsets                             src/quant.rs:518-563
#include "internal.hpp"
#include "layout.hpp"

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
            v = (float)(nib - 8) * d;
            if (!w.br) v += m;  // Q4Matrix adds its offset, 0 without one (src/quant.rs:586-606); GGUF Q4_0 adds nothing (src/ggml.rs:675-683)
            break;
        }
        case FMT_Q8_0: {
            uint32_t tile = r >> 4, nn = r & 15, b = c >> 5, st = b >> 1, h = b & 1, e = c & 31, kq = e >> 3, j = e & 7;
            const uint8_t* rec = w.p0 + ((size_t)tile * t8_steps(n) + st) * T8_REC;
            float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + 1024 + 4 * nn + 2 * h));
            v = (float)(int8_t)rec[16 * (kq * 16 + nn) + 8 * h + j] * d;
            break;
        }
        case FMT_Q8F: {  // q as f32 * scale (src/quant.rs:405-419)
            uint32_t tile = r >> 4, nn = r & 15, b = c >> 5, st = b >> 1, h = b & 1, e = c & 31, kq = e >> 3, j = e & 7;
            const uint8_t* rec = w.p0 + ((size_t)tile * t8_steps(n) + st) * T8F_REC;
            float d = *reinterpret_cast<const float*>(rec + 1024 + 8 * nn + 4 * h);
            v = (float)(int8_t)rec[16 * (kq * 16 + nn) + 8 * h + j] * d;
            break;
        }
        case FMT_Q4_K:
        case FMT_Q5_K: {
            uint32_t tile = r >> 4, nn = r & 15, sb = c / 256, e = c % 256, pair = e / 64, hi = (e % 64) / 32, l = e % 32;
            uint32_t st = pair >> 1, jj = pair & 1, kq = l >> 3;
            const uint8_t* rec = w.p0 + ((size_t)tile * tk4_sbs(n) + sb) * (w.fmt == FMT_Q5_K ? TK5_REC : TK4_REC);
            uint8_t byte = rec[st * 1024 + 16 * (kq * 16 + nn) + 8 * jj + (l & 7)];
            uint32_t q = hi ? (byte >> 4) : (byte & 0xF);
            if (w.fmt == FMT_Q5_K) {  // the fifth bit adds 16 (src/ggml.rs:765-768)
                const uint32_t hb = *reinterpret_cast<const uint32_t*>(rec + TK4_REC + 256 * st + 4 * (kq * 16 + nn));
                q += 16 * ((hb >> (8 * (l & 3) + 4 * jj + 2 * hi + ((l & 7) >> 2))) & 1);
            }
            uint32_t sc = rec[2048 + 16 * nn + 2 * pair + hi], mn = rec[2048 + 16 * nn + 8 + 2 * pair + hi];
            float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + 2304 + 4 * nn));
            float dmin = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + 2304 + 4 * nn + 2));
            float d1 = d * (float)sc, m1 = dmin * (float)mn;
            v = d1 * (float)q - m1;
            break;
        }
        case FMT_Q4M: {
            uint32_t tile = r >> 4, nn = r & 15, b = c >> 5, st = b >> 2, bi = b & 3, e = c & 31, hi = e >> 4, pp = e & 15, kq = pp >> 2;
            const uint8_t* rec = w.p0 + ((size_t)tile * t4m_steps(n) + st) * T4M_REC;
            uint8_t byte = rec[16 * (kq * 16 + nn) + 4 * bi + (pp & 3)];
            int nib = hi ? (byte >> 4) : (byte & 0xF);
            float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + 1024 + 4 * nn + 2 * (bi >> 1)));
            float m = bf16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + 1088 + 4 * nn + 2 * (bi >> 1)));
            v = (float)(nib - 8) * d + m;
            break;
        }
        case FMT_MXFP4: {
            uint32_t tile = r >> 4, nn = r & 15, b = c >> 5, st = b >> 2, bi = b & 3, e = c & 31, hi = e >> 4, pp = e & 15, kq = pp >> 2;
            const uint8_t* rec = w.p0 + ((size_t)tile * t4m_steps(n) + st) * T4X_REC;
            uint8_t byte = rec[16 * (kq * 16 + nn) + 4 * bi + (pp & 3)];
            const uint32_t code = hi ? (byte >> 4) : (byte & 0xF);
            const int kv = (int)(int8_t)(mxfp4_values<0>(code) & 0xFF);
            v = e8m0_half(rec[1024 + 4 * nn + bi]) * (float)kv;
            break;
        }
        case FMT_NVFP4: {
            uint32_t tile = r >> 4, nn = r & 15, b = c >> 5, st = b >> 2, bi = b & 3, e = c & 31, hi = e >> 4, pp = e & 15, kq = pp >> 2;
            const uint8_t* rec = w.p0 + ((size_t)tile * t4m_steps(n) + st) * T4N_REC;
            uint8_t byte = rec[16 * (kq * 16 + nn) + 4 * bi + (pp & 3)];
            const uint32_t code = hi ? (byte >> 4) : (byte & 0xF);
            const int kv = (int)(int8_t)(mxfp4_values<0>(code) & 0xFF);
            v = ue4m3_half(rec[1024 + 8 * nn + 2 * bi + hi]) * (float)kv;
            if (w.br) v *= reinterpret_cast<const float*>(w.p1)[(r / w.br) * ((n + w.bc - 1) / w.bc) + c / w.bc];
            break;
        }
        case FMT_Q40: {  // (nib - 8) * d, no offset term (src/ggml.rs:675-683)
            uint32_t tile = r >> 4, nn = r & 15, b = c >> 5, st = b >> 2, bi = b & 3, e = c & 31, hi = e >> 4, pp = e & 15, kq = pp >> 2;
            const uint8_t* rec = w.p0 + ((size_t)tile * t4m_steps(n) + st) * T4M_REC;
            uint8_t byte = rec[16 * (kq * 16 + nn) + 4 * bi + (pp & 3)];
            int nib = hi ? (byte >> 4) : (byte & 0xF);
            float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + (bi < 2 ? 1024 : 1088) + 4 * nn + 2 * (bi & 1)));
            v = (float)(nib - 8) * d;
            break;
        }
        case FMT_Q6_K: {
            const uint32_t tile = r >> 4, nn = r & 15, st = c >> 7, wi = c & 127, h = wi >> 6, kq = (wi & 63) >> 4, j = wi & 15;
            const uint8_t* rec = w.p0 + ((size_t)tile * t6k_steps(n) + st) * T6K_REC;
            const uint32_t ln = 16 * kq + nn, bb = j & 3;
            const uint32_t dw = *reinterpret_cast<const uint32_t*>(rec + 16 * ln + 4 * (2 * h + (j >> 3)));
            const uint32_t hh = *reinterpret_cast<const uint32_t*>(rec + 1024 + 8 * ln + 4 * h);
            const uint32_t lo4 = (dw >> (8 * bb + 4 * ((j & 7) >> 2))) & 0xF, hi2 = (hh >> (8 * bb + 2 * (j >> 2))) & 3;
            int q = (int)(lo4 | (hi2 << 4)) - 32;
            float sc = (float)reinterpret_cast<const int8_t*>(rec + 1536 + 8 * nn)[4 * h + kq];
            float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(rec + 1664 + 2 * nn));
            v = d * sc * (float)q;
            break;
        }
        case FMT_FP8: {
            uint32_t ncb = (n + w.bc - 1) / w.bc;
            float s = reinterpret_cast<const float*>(w.p1)[(r / w.br) * ncb + c / w.bc];
            v = e4m3_to_f32(w.p0[fp8_offset(w, r, c)]) * s;
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
// Tile-packing of raw GGUF blocks (layout.hpp). One thread per 16-byte chunk of the destination;
// the threads of lane group kq = 0 also write the record's scales. Runs once per matrix.
__global__ __launch_bounds__(256) void pack_t8_kernel(const uint8_t* __restrict__ raw, uint32_t n_out, uint32_t n_in, uint8_t* __restrict__ dst) {
    const uint32_t nsteps = t8_steps(n_in), nblk = n_in / 32;
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    uint32_t l = idx & 63, nn = l & 15, kq = l >> 4;
    size_t ts = idx >> 6;
    uint32_t st = ts % nsteps;
    size_t tile = ts / nsteps;
    size_t row = tile * 16 + nn;
    uint8_t* rec = dst + ts * T8_REC;
    uint32_t out[4] = {0, 0, 0, 0};
    uint16_t d[2] = {0, 0};
    for (uint32_t h = 0; h < 2; h++) {
        uint32_t b = 2 * st + h;
        if (row < n_out && b < nblk) {
            const uint8_t* src = raw + (row * nblk + b) * 34;
            d[h] = (uint16_t)(src[0] | (src[1] << 8));
            for (int j = 0; j < 8; j++) out[2 * h + j / 4] |= (uint32_t)src[2 + 8 * kq + j] << (8 * (j & 3));
        }
    }
    *reinterpret_cast<uint4*>(rec + 16 * l) = make_uint4(out[0], out[1], out[2], out[3]);
    if (kq == 0) *reinterpret_cast<uint32_t*>(rec + 1024 + 4 * nn) = d[0] | ((uint32_t)d[1] << 16);
}

// FIVE: Q5_K blocks (d, dmin, scales[12], qh[32], qs[128]: src/ggml.rs:753-757) into TK5 records
template <bool FIVE>
__global__ __launch_bounds__(256) void pack_tk4_kernel(const uint8_t* __restrict__ raw, uint32_t n_out, uint32_t n_in, uint8_t* __restrict__ dst) {
    constexpr uint32_t REC = FIVE ? TK5_REC : TK4_REC, BLK = FIVE ? 176 : 144, QS = FIVE ? 48 : 16;
    const uint32_t nsb = tk4_sbs(n_in);
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)row_tiles(n_out) * nsb * 128;  // two steps of 64 chunks per super-block
    if (idx >= total) return;
    uint32_t l = idx & 63, nn = l & 15, kq = l >> 4, st = (idx >> 6) & 1;
    size_t tsb = idx >> 7;
    uint32_t sb = tsb % nsb;
    size_t tile = tsb / nsb;
    size_t row = tile * 16 + nn;
    uint8_t* rec = dst + tsb * REC;
    const uint8_t* src = raw + (row * nsb + sb) * BLK;
    uint32_t out[4] = {0, 0, 0, 0};
    if (row < n_out)
        for (uint32_t jj = 0; jj < 2; jj++)
            for (int j = 0; j < 8; j++) out[2 * jj + j / 4] |= (uint32_t)src[QS + 32 * (2 * st + jj) + 8 * kq + j] << (8 * (j & 3));
    *reinterpret_cast<uint4*>(rec + st * 1024 + 16 * l) = make_uint4(out[0], out[1], out[2], out[3]);
    if (FIVE) {  // qh[l'] bit 2 j' + h: the fifth bit of element l' of sub-block 2 j' + h (j' = 2 st + jj)
        uint32_t hb = 0;
        if (row < n_out)
            for (uint32_t jj = 0; jj < 2; jj++)
                for (uint32_t hi = 0; hi < 2; hi++)
                    for (uint32_t j = 0; j < 8; j++)
                        hb |= (((uint32_t)src[16 + 8 * kq + j] >> (2 * (2 * st + jj) + hi)) & 1u) << (8 * (j & 3) + 4 * jj + 2 * hi + (j >> 2));
        *reinterpret_cast<uint32_t*>(rec + TK4_REC + 256 * st + 4 * l) = hb;
    }
    if (kq == 0 && st == 0) {
        uint32_t sc[2] = {0, 0}, mn[2] = {0, 0}, dd = 0;
        if (row < n_out) {
            uint32_t d0 = src[4] | (src[5] << 8) | (src[6] << 16) | ((uint32_t)src[7] << 24);
            uint32_t d1 = src[8] | (src[9] << 8) | (src[10] << 16) | ((uint32_t)src[11] << 24);
            uint32_t d2 = src[12] | (src[13] << 8) | (src[14] << 16) | ((uint32_t)src[15] << 24);
            for (uint32_t i = 0; i < 8; i++) {
                uint32_t s, m;
                scale_min_k4(i, d0, d1, d2, s, m);
                sc[i >> 2] |= s << (8 * (i & 3));
                mn[i >> 2] |= m << (8 * (i & 3));
            }
            dd = src[0] | (src[1] << 8) | (src[2] << 16) | ((uint32_t)src[3] << 24);
        }
        *reinterpret_cast<uint4*>(rec + 2048 + 16 * nn) = make_uint4(sc[0], sc[1], mn[0], mn[1]);
        *reinterpret_cast<uint32_t*>(rec + 2304 + 4 * nn) = dd;
    }
}

// Planar Q4 with one scale and one offset per 64 -> tile-packed (layout.hpp).
__global__ __launch_bounds__(256) void pack_q4m_kernel(const uint8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                       const uint16_t* __restrict__ off, uint32_t n_out, uint32_t n_in,
                                                       uint8_t* __restrict__ dst) {
    const uint32_t nsteps = t4m_steps(n_in), nblk = n_in / 32;
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    uint32_t l = idx & 63, nn = l & 15, kq = l >> 4;
    size_t ts = idx >> 6;
    uint32_t st = ts % nsteps;
    size_t tile = ts / nsteps;
    size_t row = tile * 16 + nn;
    uint8_t* rec = dst + ts * T4M_REC;
    uint32_t out[4] = {0, 0, 0, 0};
    for (uint32_t b = 0; b < 4; b++) {
        uint32_t blk = 4 * st + b;
        if (row < n_out && blk < nblk) out[b] = *reinterpret_cast<const uint32_t*>(q + row * (n_in / 2) + blk * 16 + 4 * kq);
    }
    *reinterpret_cast<uint4*>(rec + 16 * l) = make_uint4(out[0], out[1], out[2], out[3]);
    if (kq == 0) {
        uint32_t d = 0, o = 0;
        for (uint32_t g = 0; g < 2; g++) {
            uint32_t grp = 2 * st + g;
            if (!off) {  // Q4_0: a scale per 32; d = blocks 0 and 1 of the step, o = blocks 2 and 3
                if (row < n_out && 4 * st + g < nblk) d |= (uint32_t)sc[row * nblk + 4 * st + g] << (16 * g);
                if (row < n_out && 4 * st + 2 + g < nblk) o |= (uint32_t)sc[row * nblk + 4 * st + 2 + g] << (16 * g);
            } else if (row < n_out && grp < n_in / 64) {
                d |= (uint32_t)sc[row * (n_in / 64) + grp] << (16 * g);
                o |= (uint32_t)off[row * (n_in / 64) + grp] << (16 * g);
            }
        }
        *reinterpret_cast<uint32_t*>(rec + 1024 + 4 * nn) = d;
        *reinterpret_cast<uint32_t*>(rec + 1088 + 4 * nn) = o;
    }
}

// GGUF MXFP4 blocks (scale byte, 16 code bytes: src/ggml.rs:922-928) -> T4X records; one thread per lane slot of a record.
__global__ __launch_bounds__(256) void pack_t4x_kernel(const uint8_t* __restrict__ raw, uint32_t n_out, uint32_t n_in, uint8_t* __restrict__ dst) {
    const uint32_t nsteps = t4m_steps(n_in), nblk = n_in / 32;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x, total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    const uint32_t l = idx & 63, nn = l & 15, kq = l >> 4;
    const size_t ts = idx >> 6, tile = ts / nsteps, row = tile * 16 + nn;
    const uint32_t st = (uint32_t)(ts % nsteps);
    uint8_t* rec = dst + ts * T4X_REC;
    uint32_t out[4] = {0, 0, 0, 0}, sc = 0;
    for (uint32_t b = 0; b < 4; b++) {
        const uint32_t blk = 4 * st + b;
        if (row < n_out && blk < nblk) {
            const uint8_t* src = raw + (row * nblk + blk) * 17;
            for (uint32_t j = 0; j < 4; j++) out[b] |= (uint32_t)src[1 + 4 * kq + j] << (8 * j);
            sc |= (uint32_t)src[0] << (8 * b);
        }
    }
    *reinterpret_cast<uint4*>(rec + 16 * l) = make_uint4(out[0], out[1], out[2], out[3]);
    if (kq == 0) *reinterpret_cast<uint32_t*>(rec + 1024 + 4 * nn) = sc;
}

// ggml NVFP4 blocks (four scale bytes, then per sub-block of 16 eight bytes: elements j low, j + 8 high; src/ggml.rs:936-947)
// -> T4N records; one thread per lane slot of a record.
__global__ __launch_bounds__(256) void pack_t4n_kernel(const uint8_t* __restrict__ raw, uint32_t n_out, uint32_t n_in, uint8_t* __restrict__ dst) {
    const uint32_t nsteps = t4m_steps(n_in), nb64 = n_in / 64;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x, total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    const uint32_t l = idx & 63, nn = l & 15, kq = l >> 4;
    const size_t ts = idx >> 6, tile = ts / nsteps, row = tile * 16 + nn;
    const uint32_t st = (uint32_t)(ts % nsteps);
    uint8_t* rec = dst + ts * T4N_REC;
    uint32_t out[4] = {0, 0, 0, 0}, sc[2] = {0, 0};
    for (uint32_t b = 0; b < 4; b++) {  // the step's 32-column group b: sub-blocks 2 (b & 1), 2 (b & 1) + 1 of block 2 st + b / 2
        const uint32_t blk = 2 * st + (b >> 1);
        if (row >= n_out || blk >= nb64) continue;
        const uint8_t* src = raw + ((size_t)row * nb64 + blk) * 36;
        const uint32_t s0 = 2 * (b & 1);
        for (uint32_t j = 0; j < 4; j++) {
            // element e of a sub-block: byte e % 8 of its eight, low nibble for e < 8
            const uint32_t e = 4 * kq + j;
            const uint32_t lo = (src[4 + 8 * s0 + (e & 7)] >> (4 * (e >> 3))) & 0xF;
            const uint32_t hi = (src[4 + 8 * (s0 + 1) + (e & 7)] >> (4 * (e >> 3))) & 0xF;
            out[b] |= (lo | (hi << 4)) << (8 * j);
        }
        sc[b >> 1] |= ((uint32_t)src[s0] | ((uint32_t)src[s0 + 1] << 8)) << (16 * (b & 1));
    }
    *reinterpret_cast<uint4*>(rec + 16 * l) = make_uint4(out[0], out[1], out[2], out[3]);
    if (kq == 0) *reinterpret_cast<uint2*>(rec + 1024 + 8 * nn) = make_uint2(sc[0], sc[1]);
}

hipError_t launch_pack_q4m(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t n_out, size_t n_in, uint8_t* dst,
                           hipStream_t s) {
    size_t total = (size_t)row_tiles((uint32_t)n_out) * t4m_steps((uint32_t)n_in) * 64;
    pack_q4m_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(q, sc, off, (uint32_t)n_out, (uint32_t)n_in, dst);
    return hipGetLastError();
}

// FP8 row-major -> tile-packed records (internal.hpp): one thread per lane slot of a record, 32 bytes.
__global__ __launch_bounds__(256) void pack_fp8_kernel(const uint8_t* __restrict__ raw, uint32_t n_out, uint32_t n_in, uint8_t* __restrict__ dst) {
    const uint32_t nsteps = n_in / 128;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x, total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    const uint32_t l = idx & 63, n = l & 15, kq = l >> 4;
    const size_t rec = idx >> 6, tile = rec / nsteps, st = rec % nsteps, row = tile * 16 + n;
    uint4 a = make_uint4(0u, 0u, 0u, 0u), b = a;
    if (row < n_out) {
        const uint4* src = reinterpret_cast<const uint4*>(raw + row * n_in + 128 * st + 32 * kq);
        a = src[0];
        b = src[1];
    }
    uint4* out = reinterpret_cast<uint4*>(dst + rec * 2048 + 16 * l);
    out[0] = a;
    out[64] = b;
}

hipError_t launch_pack_fp8(const uint8_t* raw, size_t n_out, size_t n_in, uint8_t* dst, hipStream_t s) {
    const size_t total = (size_t)row_tiles((uint32_t)n_out) * (n_in / 128) * 64;
    if (!total) return hipSuccess;
    pack_fp8_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, dst);
    return hipGetLastError();
}

// Q6_K (210-byte blocks of 256: ql[128], qh[64], 16 int8 scales, f16 d; element 128 nn + 32 k + l of a block has its low
// nibble in ql[64 nn + l + 32 (k & 1)] (high half for k >= 2) and its two high bits at bit 2 k of qh[32 nn + l],
// src/ggml.rs:774-793) -> T6K records; one thread per lane slot of a record.
__global__ __launch_bounds__(256) void pack_t6k_kernel(const uint8_t* __restrict__ raw, uint32_t n_out, uint32_t n_in, uint8_t* __restrict__ dst) {
    const uint32_t nsteps = t6k_steps(n_in), nb = n_in / 256;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x, total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    const uint32_t l = idx & 63, n = l & 15, kq = l >> 4;
    const size_t recno = idx >> 6, tile = recno / nsteps, st = recno % nsteps, row = tile * 16 + n;
    uint8_t* rec = dst + recno * T6K_REC;
    uint32_t lo[4] = {0, 0, 0, 0}, hi[2] = {0, 0};
    const bool live = row < n_out;
    const uint8_t* blk = raw + ((live ? row : 0) * nb + st / 2) * 210;
    const uint32_t nn = st & 1;
    if (live) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const uint32_t wi = 64 * h + 16 * kq + j, k = wi >> 5, e = wi & 31;
                const uint8_t qb = blk[64 * nn + e + 32 * (k & 1)];
                const uint32_t lo4 = k < 2 ? (qb & 0xFu) : (qb >> 4), hi2 = (blk[128 + 32 * nn + e] >> (2 * k)) & 3u;
                lo[2 * h + (j >> 3)] |= lo4 << (8 * (j & 3) + 4 * ((j & 7) >> 2));
                hi[h] |= hi2 << (8 * (j & 3) + 2 * (j >> 2));
            }
    }
    *reinterpret_cast<uint4*>(rec + 16 * l) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    *reinterpret_cast<uint2*>(rec + 1024 + 8 * l) = make_uint2(hi[0], hi[1]);
    if (kq == 0) {
        uint32_t s0 = 0, s1 = 0;
        uint16_t d = 0;
        if (live) {
            for (int i = 0; i < 4; i++) {
                s0 |= (uint32_t)blk[192 + 8 * nn + i] << (8 * i);
                s1 |= (uint32_t)blk[192 + 8 * nn + 4 + i] << (8 * i);
            }
            d = (uint16_t)(blk[208] | (blk[209] << 8));
        }
        *reinterpret_cast<uint2*>(rec + 1536 + 8 * n) = make_uint2(s0, s1);
        *reinterpret_cast<uint16_t*>(rec + 1664 + 2 * n) = d;
    }
}

// QMatrix (q i8 [n_out][n_in], scales f32 [n_out][n_in/32]) -> T8F records; one thread per lane slot of a record.
__global__ __launch_bounds__(256) void pack_t8f_kernel(const int8_t* __restrict__ q, const float* __restrict__ scales, uint32_t n_out, uint32_t n_in,
                                                       uint8_t* __restrict__ dst) {
    const uint32_t nsteps = t8_steps(n_in), nblk = n_in / 32;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x, total = (size_t)row_tiles(n_out) * nsteps * 64;
    if (idx >= total) return;
    const uint32_t l = idx & 63, nn = l & 15, kq = l >> 4;
    const size_t ts = idx >> 6, tile = ts / nsteps, row = tile * 16 + nn;
    const uint32_t st = (uint32_t)(ts % nsteps);
    uint8_t* rec = dst + ts * T8F_REC;
    uint2 c[2] = {make_uint2(0u, 0u), make_uint2(0u, 0u)};
    float d[2] = {0.0f, 0.0f};
    for (uint32_t h = 0; h < 2; h++) {
        const uint32_t b = 2 * st + h;
        if (row < n_out && b < nblk) {
            c[h] = *reinterpret_cast<const uint2*>(q + row * n_in + 32 * b + 8 * kq);
            d[h] = scales[row * nblk + b];
        }
    }
    *reinterpret_cast<uint4*>(rec + 16 * l) = make_uint4(c[0].x, c[0].y, c[1].x, c[1].y);
    if (kq == 0) *reinterpret_cast<float2*>(rec + 1024 + 8 * nn) = make_float2(d[0], d[1]);
}

hipError_t launch_pack_q8f(const int8_t* q, const float* scales, size_t n_out, size_t n_in, uint8_t* dst, hipStream_t s) {
    const size_t total = (size_t)row_tiles((uint32_t)n_out) * t8_steps((uint32_t)n_in) * 64;
    if (!total) return hipSuccess;
    pack_t8f_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(q, scales, (uint32_t)n_out, (uint32_t)n_in, dst);
    return hipGetLastError();
}

hipError_t launch_repack_gguf(int fmt, const uint8_t* raw, size_t n_out, size_t n_in, const WeightView& d, hipStream_t s) {
    uint8_t* p0 = const_cast<uint8_t*>(d.p0);
    if (fmt == FMT_Q8_0) {
        size_t total = (size_t)row_tiles((uint32_t)n_out) * t8_steps((uint32_t)n_in) * 64;
        pack_t8_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, p0);
    } else if (k45_format(fmt)) {
        size_t total = (size_t)row_tiles((uint32_t)n_out) * tk4_sbs((uint32_t)n_in) * 128;
        if (!total) return hipSuccess;
        if (fmt == FMT_Q5_K) pack_tk4_kernel<true><<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, p0);
        else pack_tk4_kernel<false><<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, p0);
    } else if (fmt == FMT_MXFP4) {
        size_t total = (size_t)row_tiles((uint32_t)n_out) * t4m_steps((uint32_t)n_in) * 64;
        if (!total) return hipSuccess;
        pack_t4x_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, p0);
    } else if (fmt == FMT_NVFP4) {
        size_t total = (size_t)row_tiles((uint32_t)n_out) * t4m_steps((uint32_t)n_in) * 64;
        if (!total) return hipSuccess;
        pack_t4n_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, p0);
    } else if (fmt == FMT_Q6_K) {
        size_t total = (size_t)row_tiles((uint32_t)n_out) * t6k_steps((uint32_t)n_in) * 64;
        if (!total) return hipSuccess;
        pack_t6k_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(raw, (uint32_t)n_out, (uint32_t)n_in, p0);
    } else {
        return hipErrorInvalidValue;
    }
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
