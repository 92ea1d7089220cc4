// Activation quantization on the device: quant::quantize_act (src/quant.rs:243-343 of the reference).
//
// Per block of 32: amax = max |x|, inv = 127 / amax (0 for an all-zero block),
// q = round-half-away(x * inv) as int8, scale = amax / 127, the integer block sum, and the f32 sums
// of the block and of each half in element order. Every output is bit-identical to the CPU's, so
// the sums are sequential: one lane owns one block and walks its 32 values (eight 16-byte loads).
// The work is a few hundred KB at most; it is latency, not bandwidth, that matters here.
#include "act_body.hpp"
#include "internal.hpp"

namespace oxhip {

__global__ __launch_bounds__(64) void quantize_act_kernel(const float* __restrict__ x, size_t nblocks, int8_t* __restrict__ q,
                                                          float* __restrict__ scales, int32_t* __restrict__ sums,
                                                          float* __restrict__ fsums, float* __restrict__ hsums,
                                                          int32_t* __restrict__ sums16) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    quantize_act_block(x, b, q, scales, sums, fsums, hsums, sums16);
}

hipError_t launch_quantize_act(const float* x, size_t t, size_t n_in, const oxhip_qact& o, hipStream_t s) {
    size_t nblocks = t * n_in / 32;
    if (nblocks == 0) return hipSuccess;
    dim3 grid((unsigned)((nblocks + 63) / 64));
    quantize_act_kernel<<<grid, 64, 0, s>>>(x, nblocks, o.q, o.scales, o.sums, o.fsums, o.hsums, o.sums16);
    return hipGetLastError();
}

}  // namespace oxhip
