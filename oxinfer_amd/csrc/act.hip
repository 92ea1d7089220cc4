// Activation quantization on the device: quant::quantize_act (src/quant.rs:243-343 of the reference).
//
// Per block of 32: amax = max |x|, inv = 127 / amax (0 for an all-zero block),
// q = round-half-away(x * inv) as int8, scale = amax / 127, the integer block sum, and the f32 sums
// of the block and of each half in element order. Every output is bit-identical to the CPU's, so
// the sums are sequential: one lane owns one block and walks its 32 values (eight 16-byte loads).
// The work is a few hundred KB at most; it is latency, not bandwidth, that matters here.
#include "internal.hpp"

namespace oxhip {

__global__ __launch_bounds__(64) void quantize_act_kernel(const float* __restrict__ x, size_t nblocks, int8_t* __restrict__ q,
                                                          float* __restrict__ scales, int32_t* __restrict__ sums,
                                                          float* __restrict__ fsums, float* __restrict__ hsums,
                                                          int32_t* __restrict__ sums16) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
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

hipError_t launch_quantize_act(const float* x, size_t t, size_t n_in, const oxhip_qact& o, hipStream_t s) {
    size_t nblocks = t * n_in / 32;
    if (nblocks == 0) return hipSuccess;
    dim3 grid((unsigned)((nblocks + 63) / 64));
    quantize_act_kernel<<<grid, 64, 0, s>>>(x, nblocks, o.q, o.scales, o.sums, o.fsums, o.hsums, o.sums16);
    return hipGetLastError();
}

}  // namespace oxhip
