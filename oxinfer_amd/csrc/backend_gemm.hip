// The prefill GEMM entry points over gemm.hip.
#include "backend.hpp"

using namespace oxhip;

namespace oxhip {

// Packs x and runs the bf16 GEMM; the packed activations live in ctx scratch.
int gemm_bf16_run(oxhip_ctx* c, const oxhip_weight* w, const void* x, bool x_bf16, size_t t, void* y, bool y_bf16, hipStream_t s) {
    if (w->v.fmt != FMT_Q4M) {
        set_error("gemm: the bf16 variant runs MLX 4-bit weights");
        return 0;
    }
    const size_t mtiles = (t + 15) / 16, kblocks = 4 * (size_t)t4m_steps(w->v.n_in);
    const size_t pack_bytes = align_up(mtiles * kblocks * 64 * 16, 256);
    const uint32_t slices = gemm_k_slices(w->v, mtiles);
    const size_t bytes = pack_bytes + (slices > 1 ? (size_t)slices * t * w->v.n_out * 4 : 0);
    if (c->gemm_ws.cap < bytes) {
        (void)hipStreamSynchronize(s);  // an earlier GEMM may still read the old scratch
        if (!c->gemm_ws.grow(bytes)) {
            set_error("gemm: device memory short");
            return 0;
        }
    }
    HIP_TRY(launch_pack_a(x, x_bf16, true, t, w->v.n_in, mtiles, kblocks, c->gemm_ws.p, s), "gemm pack launch");
    float* partial = reinterpret_cast<float*>(static_cast<uint8_t*>(c->gemm_ws.p) + pack_bytes);
    HIP_TRY(launch_gemm_bf16(w->v, c->gemm_ws.p, t, mtiles, y, y_bf16, partial, s), "gemm launch");
    return 1;
}

}  // namespace oxhip

extern "C" {

int oxhip_dev_gemm(oxhip_ctx* c, const oxhip_weight* w, const void* x, int x_dtype, size_t t, void* y, int y_dtype, int variant,
                   void* stream) {
    if (!c || !w || !x || !y || !t || x_dtype < 0 || x_dtype > 1 || y_dtype < 0 || y_dtype > 1) {
        set_error("gemm: bad arguments");
        return 0;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (variant) {
        case OXHIP_GEMM_BF16: return gemm_bf16_run(c, w, x, x_dtype == OXHIP_BF16, t, y, y_dtype == OXHIP_BF16, s);
        default: set_error("gemm: unknown variant"); return 0;
    }
}

}  // extern "C"
