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

// Several activation matrices in one launch (a decode step quantizes the input of every group of matmuls; each launch
// is a few microseconds of latency whatever its size).
struct QuantBatchArgs {
    uint32_t njobs;
    uint32_t first[QUANT_BATCH_MAX + 1];  // first lane-block of job j; first[njobs] = total
    const float* x[QUANT_BATCH_MAX];
    int8_t* q[QUANT_BATCH_MAX];
    float* scales[QUANT_BATCH_MAX];
    int32_t* sums[QUANT_BATCH_MAX];
    float* fsums[QUANT_BATCH_MAX];
    float* hsums[QUANT_BATCH_MAX];
    int32_t* sums16[QUANT_BATCH_MAX];
};

__global__ __launch_bounds__(64) void quantize_act_batch_kernel(QuantBatchArgs a) {
    const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= a.first[a.njobs]) return;
    uint32_t j = 0;
    while (j + 1 < a.njobs && b >= a.first[j + 1]) j++;
    quantize_act_block(a.x[j], (size_t)(b - a.first[j]), a.q[j], a.scales[j], a.sums[j], a.fsums[j], a.hsums[j], a.sums16[j]);
}

hipError_t launch_quantize_act_batch(const float* const* x, const size_t* t, const size_t* n_in, const oxhip_qact* o, size_t n, hipStream_t s) {
    for (size_t i0 = 0; i0 < n; i0 += QUANT_BATCH_MAX) {
        QuantBatchArgs a{};
        a.njobs = (uint32_t)(n - i0 < (size_t)QUANT_BATCH_MAX ? n - i0 : (size_t)QUANT_BATCH_MAX);
        uint32_t total = 0;
        for (uint32_t j = 0; j < a.njobs; j++) {
            const size_t nb = t[i0 + j] * n_in[i0 + j] / 32;
            if (total + nb > 0x7FFFFFFFu) return hipErrorInvalidValue;
            a.first[j] = total;
            total += (uint32_t)nb;
            a.x[j] = x[i0 + j];
            a.q[j] = o[i0 + j].q;
            a.scales[j] = o[i0 + j].scales;
            a.sums[j] = o[i0 + j].sums;
            a.fsums[j] = o[i0 + j].fsums;
            a.hsums[j] = o[i0 + j].hsums;
            a.sums16[j] = o[i0 + j].sums16;
        }
        a.first[a.njobs] = total;
        if (!total) continue;
        quantize_act_batch_kernel<<<(total + 63) / 64, 64, 0, s>>>(a);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_quantize_act(const float* x, size_t t, size_t n_in, const oxhip_qact& o, hipStream_t s) {
    size_t nblocks = t * n_in / 32;
    if (nblocks == 0) return hipSuccess;
    dim3 grid((unsigned)((nblocks + 63) / 64));
    quantize_act_kernel<<<grid, 64, 0, s>>>(x, nblocks, o.q, o.scales, o.sums, o.fsums, o.hsums, o.sums16);
    return hipGetLastError();
}

}  // namespace oxhip
