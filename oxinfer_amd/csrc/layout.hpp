// Tile-packed device layouts of the quantized formats, shared by the upload repackers, the
// dequantizers and the MFMA kernels.
//
// A matrix is cut into row tiles of 16 rows; a tile is a sequence of K-steps, and each K-step is
// stored as one record so that a wavefront reads it with one fully coalesced 16-byte-per-lane
// load: lane l = 16 * kq + n holds bytes [16 l, 16 l + 16) of the record, which are the codes of
// row n of the tile at the K positions MFMA lane group kq consumes. Scales (and mins / offsets) of
// the 16 rows follow the codes in the same record. Rows past n_out and blocks past n_in are zero.
// The bytes are those of the source format (Q4_K: its 12 packed scale bytes are stored unpacked as
// 16 bytes, 2.8 % more), only rearranged.
//
//   Q8_0 (T8)   step = 2 blocks of 32 (64 K), record 1088 B:
//               codes[16 l + 8 h + j] = q[row n][block 2 s + h][8 kq + j]          1024 B
//               d[n][h] f16                                                          64 B
//   Q4_K (TK4)  super-block record 2368 B = 2 steps of 128 K + metadata:
//               codes[1024 t + 16 l + 8 jj + j] = qs[32 (2 t + jj) + 8 kq + j]     2048 B
//                  (low nibble: sub-block 2 (2 t + jj), high nibble: the next one)
//               sc[n][8], mn[n][8] bytes (the 6-bit scales and mins, unpacked)       256 B
//               d[n], dmin[n] f16                                                     64 B
//   Q5_K (TK5)  the TK4 record followed by the fifth bits, 2880 B:
//               hbit[256 t + 4 l] (a dword): bit 8 k + i = fifth bit of the code in byte k of the lane's operand dword i
//                  of step t, i = 4 jj + 2 (high nibble) + (j / 4), k = j % 4, for the codes byte 8 jj + j    512 B
//   Q4 with one scale and one offset per 64 (MLX; T4M)  step = 4 blocks (128 K), record 1152 B:
//               codes[16 l + 4 b + j] = q[row n][block 4 s + b][4 kq + j]           1024 B
//                  (low nibble: element 4 kq + j, high nibble: element 16 + 4 kq + j)
//               d[n][2] f16 (blocks 0-1, blocks 2-3)                                  64 B
//               off[n][2] bf16                                                        64 B
//   GGUF Q4_0 in the same records: d[n][4] f16, the scales of blocks 0-1 where MLX has its scales and of blocks 2-3
//   where it has its offsets.
//   MXFP4 (T4X) the T4M codes (byte j of a block: elements j and j + 16, as in the file) followed by the four E8M0 scale
//               bytes of each row's blocks, record 1088 B
//   NVFP4 (T4N) the T4M code geometry over ggml's blocks of 64 (sub-block s of 16: scale byte s, then 8 bytes whose byte j
//               holds elements j and j + 8): byte j of a lane's dword b holds the step's elements 32 b + 4 kq + j (low
//               nibble) and 32 b + 16 + 4 kq + j (high), followed by the eight unsigned-E4M3 scale bytes of each row's
//               sub-blocks of 16 (sub-block 2 b + high), record 1152 B: 4.5 bit per weight, as in the file
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace oxhip {

constexpr uint32_t T8_REC = 1088;
// QMatrix (int8 codes, f32 scale per 32): the T8 codes followed by the two f32 block scales of each of the 16 rows.
constexpr uint32_t T8F_REC = 1152;
constexpr uint32_t TK4_REC = 2368;
constexpr uint32_t TK5_REC = TK4_REC + 512;
constexpr uint32_t T4M_REC = 1152;
constexpr uint32_t T4X_REC = 1088;
constexpr uint32_t T4N_REC = 1152;
// Q6_K, 16 rows x 128 columns (half a super-block), lane = 16 kq + n, code j of half h = row n, column 64 h + 16 kq + j:
//   [0, 1024)    low nibbles, 16 bytes per lane: dword 2 h + j / 8, byte j % 4, low nibble if j % 8 < 4, else high
//   [1024, 1536) the two high bits, 8 bytes per lane: dword h, bits 8 (j % 4) + 2 (j / 4)
//   [1536, 1664) the 8 int8 scales of row n's 16-column sub-blocks (sub-block 4 h + kq), 8 bytes per row
//   [1664, 1696) f16 d of row n's super-block
// so (dword >> 4 i) & 0x0F0F0F0F | ((high >> 2 r) & 0x03030303) << 4 are the four int8 operand dwords of a lane.
constexpr uint32_t T6K_REC = 1696;

__host__ __device__ inline uint32_t t8_steps(uint32_t n_in) { return (n_in / 32 + 1) / 2; }
__host__ __device__ inline uint32_t tk4_sbs(uint32_t n_in) { return n_in / 256; }
__host__ __device__ inline uint32_t t4m_steps(uint32_t n_in) { return (n_in / 32 + 3) / 4; }
__host__ __device__ inline uint32_t t6k_steps(uint32_t n_in) { return n_in / 128; }
__host__ __device__ inline uint32_t row_tiles(uint32_t n_out) { return (n_out + 15) / 16; }

__host__ __device__ inline size_t t8_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * t8_steps(n_in) * T8_REC; }
__host__ __device__ inline size_t t8f_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * t8_steps(n_in) * T8F_REC; }
__host__ __device__ inline size_t tk4_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * tk4_sbs(n_in) * TK4_REC; }
__host__ __device__ inline size_t tk5_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * tk4_sbs(n_in) * TK5_REC; }
__host__ __device__ inline size_t t4x_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * t4m_steps(n_in) * T4X_REC; }
__host__ __device__ inline size_t t4n_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * t4m_steps(n_in) * T4N_REC; }
__host__ __device__ inline size_t t4m_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * t4m_steps(n_in) * T4M_REC; }

__host__ __device__ inline size_t t6k_bytes(uint32_t n_out, uint32_t n_in) { return (size_t)row_tiles(n_out) * t6k_steps(n_in) * T6K_REC; }

}  // namespace oxhip
