// quantize_act of one block of 32 (src/quant.rs:267-292 of the reference), by one lane: shared by the stand-alone
// kernel and the MoE front kernel.
#pragma once
#include "internal.hpp"

namespace oxhip {

__device__ __forceinline__ void quantize_act_block(const float* __restrict__ x, size_t b, int8_t* __restrict__ q, float* __restrict__ scales,
                                                   int32_t* __restrict__ sums, float* __restrict__ fsums, float* __restrict__ hsums,
                                                   int32_t* __restrict__ sums16) {
    const float4* src = reinterpret_cast<const float4*>(x + b * 32);
    float v[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float4 f = src[i];
        v[4 * i] = f.x;
        v[4 * i + 1] = f.y;
        v[4 * i + 2] = f.z;
        v[4 * i + 3] = f.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    // Rust's iter().sum() starts from -0.0 (an all -0.0 block sums to -0.0).
    float h0 = -0.0f, h1 = -0.0f, f = -0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) h0 += v[i];
#pragma unroll
    for (int i = 16; i < 32; i++) h1 += v[i];
#pragma unroll
    for (int i = 0; i < 32; i++) f += v[i];
    int s0 = 0, s1 = 0;
    uint32_t packed[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t w = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float r = roundf(v[4 * i + k] * inv);  // half away from zero
            int iv = r != r ? 0 : (int)fminf(fmaxf(r, -128.0f), 127.0f);
            if (i < 4) s0 += iv; else s1 += iv;
            w |= ((uint32_t)iv & 0xFF) << (8 * k);
        }
        packed[i] = w;
    }
    uint4* dst = reinterpret_cast<uint4*>(q + b * 32);
    dst[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    dst[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
    scales[b] = amax / 127.0f;
    sums[b] = s0 + s1;
    fsums[b] = f;
    hsums[2 * b] = h0;
    hsums[2 * b + 1] = h1;
    sums16[2 * b] = s0;
    sums16[2 * b + 1] = s1;
}

}  // namespace oxhip
