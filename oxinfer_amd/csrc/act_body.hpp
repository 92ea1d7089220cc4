// quantize_act of one block of 32 (src/quant.rs:267-292 of the reference), by one lane: shared by the stand-alone
// kernel and the MoE front kernel.
#pragma once
#include "internal.hpp"

namespace oxhip {

// (the block's 32 values already in registers: block b of the output arrays)
__device__ __forceinline__ void quantize_act_values(const float* v, size_t b, int8_t* __restrict__ q, float* __restrict__ scales,
                                                    int32_t* __restrict__ sums, float* __restrict__ fsums, float* __restrict__ hsums,
                                                    int32_t* __restrict__ sums16) {
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
    quantize_act_values(v, b, q, scales, sums, fsums, hsums, sums16);
}

// fast_exp of the reference (src/kernels.rs:2225-2231): clamp, Cody-Waite reduction, degree-6 polynomial,
// scale by 2^fx through the exponent bits; every operation unfused as written there.
__device__ __forceinline__ float fast_exp(float x) {
    x = fminf(fmaxf(x, -87.0f), 88.0f);
    const float fx = roundf(x * 1.44269504088896340736f);
    const float r = (x - fx * 0.693359375f) - fx * -2.12194440e-4f;
    const float p = 1.0f + r * (1.0f + r * (0.5f + r * (0.16666667f + r * (0.041666668f + r * (0.008333334f + r * 0.0013888889f)))));
    return __int_as_float(((int)fx + 127) << 23) * p;
}

// Act::apply of one pair (src/moe.rs:18-37, silu_mul / gelu_mul): kind 0 SiLU, 1 GELU-tanh, 2 SiLU with clamp `param`.
__device__ __forceinline__ float gated_act(float g, float u, uint32_t kind, float param) {
    if (kind == 1) {
        const float K2 = 2.0f * 0.7978846f;
        const float t = K2 * (g + 0.044715f * g * g * g);
        return g / (1.0f + fast_exp(-t)) * u;
    }
    if (kind == 2) {
        g = fminf(g, param);
        u = fminf(fmaxf(u, -param), param);
    }
    return g / (1.0f + fast_exp(-g)) * u;
}

// Act::scalar (src/moe.rs:39-46), what the reference's grouped prefill path applies: the exponential of the SiLU
// kinds is the library's, not fast_exp (GELU-tanh goes through fast_exp in both, src/kernels.rs:2235-2239).
__device__ __forceinline__ float gated_act_scalar(float g, float u, uint32_t kind, float param) {
    if (kind == 1) return gated_act(g, u, kind, param);
    if (kind == 2) {
        g = fminf(g, param);
        u = fminf(fmaxf(u, -param), param);
    }
    return g / (1.0f + expf(-g)) * u;
}

}  // namespace oxhip
