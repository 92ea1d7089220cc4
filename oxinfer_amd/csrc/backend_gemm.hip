// The prefill GEMM entry points over gemm.hip.
#include "backend.hpp"

using namespace oxhip;

namespace oxhip {

thread_local KernelSpan g_kernel_span;

// The GEMMs' packed activations grow on first use (with a wait for the stream): not while a plan records on the stream.
static bool grow_ws(DevBuf& ws, size_t bytes, hipStream_t s) {
    if (ws.cap >= bytes) return true;
    if (stream_recording(s)) {
        set_error("gemm: this call would have to allocate device memory while a plan records on its stream (run the chain once before recording)");
        return false;
    }
    (void)hipStreamSynchronize(s);  // an earlier GEMM may still read the old scratch
    if (!ws.grow(bytes)) {
        set_error("gemm: device memory short");
        return false;
    }
    return true;
}

// Packs x and runs the bf16 GEMM; the packed activations live in `ws` (the calling stream's scratch: grown on first use).
int gemm_bf16_run(DevBuf& ws, const oxhip_weight* w, const void* x, bool x_bf16, size_t t, void* y, bool y_bf16, hipStream_t s) {
    const bool fp8 = w->v.fmt == FMT_FP8;
    if (!gemm_bf16_ok(w->v)) {
        set_error("gemm: the bf16 variant runs MLX 4-bit, Q8, Q8_0, Q4_K, Q5_K and Q6_K weights and FP8 weights whose rows are multiples of 128");
        return 0;
    }
    if (fp8 && skinny_fp8_ok(w->v, t)) {  // up to 32 tokens: bandwidth-bound, one pass over the weights
        const size_t need = skinny_fp8_pack_bytes(w->v, t, 1);
        if (!grow_ws(ws, need, s)) return 0;
        span_start(s);  // (the skinny kernel and its packing launch count as one)
        HIP_TRY(launch_skinny_fp8(w->v, x, x_bf16, false, t, y, y_bf16, ws.p, s), "fp8 skinny launch");
        span_stop(s);
        return 1;
    }
    const size_t mtiles = (t + 15) / 16, kblocks = 4 * (size_t)((w->v.n_in + 127) / 128);
    const size_t pack_bytes = align_up(mtiles * kblocks * 64 * 16, 256);
    const uint32_t slices = gemm_k_slices(w->v, mtiles);
    const size_t bytes = pack_bytes + (slices > 1 ? (size_t)slices * t * w->v.n_out * 4 : 0);
    if (!grow_ws(ws, bytes, s)) return 0;
    HIP_TRY(launch_pack_a(x, x_bf16, gemm_bf16_pack_mode(w->v), t, w->v.n_in, mtiles, kblocks, ws.p, s), "gemm pack launch");
    float* partial = reinterpret_cast<float*>(static_cast<uint8_t*>(ws.p) + pack_bytes);
    HIP_TRY(launch_gemm_bf16(w->v, ws.p, t, mtiles, y, y_bf16, partial, s), "gemm launch");
    return 1;
}

// FP8 block-scaled weights: activations quantized to e4m3 per 1 x 128 tile, fp8 MFMA.
int gemm_fp8_run(DevBuf& ws, const oxhip_weight* w, const void* x, bool x_bf16, size_t t, void* y, bool y_bf16, hipStream_t s) {
    if (w->v.fmt != FMT_FP8 || w->v.br != 128 || w->v.bc != 128 || w->v.n_in % 128) {
        set_error("gemm: the fp8 variant runs FP8 weights with 128 x 128 block scales and rows that are multiples of 128");
        return 0;
    }
    const size_t mtiles = (t + 15) / 16, kblocks = w->v.n_in / 128;
    const size_t pack_bytes = align_up(mtiles * kblocks * 64 * 32, 256), sx_bytes = align_up(kblocks * mtiles * 16 * 4, 256);
    const uint32_t slices = gemm_fp8_k_slices(w->v, mtiles);
    const size_t bytes = pack_bytes + sx_bytes + (slices > 1 ? (size_t)slices * t * w->v.n_out * 4 : 0);
    if (!grow_ws(ws, bytes, s)) return 0;
    uint8_t* base = static_cast<uint8_t*>(ws.p);
    float* sx = reinterpret_cast<float*>(base + pack_bytes);
    float* partial = reinterpret_cast<float*>(base + pack_bytes + sx_bytes);
    HIP_TRY(launch_quantize_act_fp8(x, x_bf16, t, w->v.n_in, mtiles, kblocks, base, sx, s), "fp8 activation quantization launch");
    HIP_TRY(launch_gemm_fp8(w->v, base, sx, t, mtiles, y, y_bf16, partial, s), "fp8 gemm launch");
    return 1;
}

// MLX 4-bit weights on the int8 matrix cores: activations quantized per token and block of 32, exact int32 block
// sums, f32 rescale (the reference's int8 GEMM, src/kernels_i8gemm.rs:160-315). `dump` (optional) receives the sums.
int gemm_i8_run(DevBuf& ws, const oxhip_weight* w, const void* x, bool x_bf16, size_t t, void* y, bool y_bf16, int32_t* dump,
                hipStream_t s) {
    if (w->v.fmt != FMT_Q4M) {
        set_error("gemm: the int8 variant runs MLX 4-bit weights (group 64)");
        return 0;
    }
    size_t slots, ngrp;
    gemm_i8_geometry(w->v, t, &slots, &ngrp);
    const size_t frag_bytes = align_up(slots / 16 * ngrp * 64 * 16, 256), xs_bytes = align_up(slots * ngrp * 8, 256),
                 fs_bytes = align_up(slots * ngrp * 4, 256);
    const uint32_t slices = gemm_i8_k_slices(w->v, t);
    const bool direct = slices == 1 && !y_bf16 && y;
    const size_t bytes = frag_bytes + xs_bytes + fs_bytes + (direct ? 0 : (size_t)slices * t * w->v.n_out * 4);
    if (!grow_ws(ws, bytes, s)) return 0;
    uint8_t* base = static_cast<uint8_t*>(ws.p);
    void *frag = base, *xs = base + frag_bytes, *fs = base + frag_bytes + xs_bytes;
    float* partial = reinterpret_cast<float*>(base + frag_bytes + xs_bytes + fs_bytes);
    HIP_TRY(launch_quantize_pack_i8(x, x_bf16, t, w->v, frag, xs, fs, s), "int8 activation quantization launch");
    HIP_TRY(launch_gemm_i8(w->v, frag, xs, fs, t, direct ? static_cast<float*>(y) : partial, dump, s), "int8 gemm launch");
    if (!direct && y) HIP_TRY(launch_gemm_reduce(partial, t * (size_t)w->v.n_out, slices, y, y_bf16, s), "gemm reduce launch");
    return 1;
}

}  // namespace oxhip

extern "C" {

int oxhip_dev_gemm_isums(oxhip_ctx* c, const oxhip_weight* w, const void* x, int x_dtype, size_t t, int32_t* out, void* stream) {
    if (!c || !w || !x || !out || !t || x_dtype < 0 || x_dtype > 1) {
        set_error("gemm_isums: bad arguments");
        return 0;
    }
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    StreamScratch* sc = scratch_for(c, static_cast<hipStream_t>(stream), false);
    if (!sc) {
        set_error("gemm_isums: device memory short");
        return 0;
    }
    return gemm_i8_run(sc->gemm_ws, w, x, x_dtype == OXHIP_BF16, t, nullptr, false, out, static_cast<hipStream_t>(stream));
}

int oxhip_dev_gemm(oxhip_ctx* c, const oxhip_weight* w, const void* x, int x_dtype, size_t t, void* y, int y_dtype, int variant,
                   void* stream) {
    if (!c || !w || !x || !y || !t || x_dtype < 0 || x_dtype > 1 || y_dtype < 0 || y_dtype > 1) {
        set_error("gemm: bad arguments");
        return 0;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    StreamScratch* sc = scratch_for(c, s, false);
    if (!sc) {
        set_error("gemm: device memory short");
        return 0;
    }
    DevBuf& ws = sc->gemm_ws;
    int rc = 0;
    switch (variant) {
        case OXHIP_GEMM_BF16: rc = gemm_bf16_run(ws, w, x, x_dtype == OXHIP_BF16, t, y, y_dtype == OXHIP_BF16, s); break;
        case OXHIP_GEMM_I8: rc = gemm_i8_run(ws, w, x, x_dtype == OXHIP_BF16, t, y, y_dtype == OXHIP_BF16, nullptr, s); break;
        case OXHIP_GEMM_FP8: rc = gemm_fp8_run(ws, w, x, x_dtype == OXHIP_BF16, t, y, y_dtype == OXHIP_BF16, s); break;
        default: set_error("gemm: unknown variant"); return 0;
    }
    if (!rc && stream_recording(s)) {  // a declined call leaves a hole in a recording: the plan must not be replayable
        std::lock_guard<std::mutex> g(c->smu);
        c->record_failed.insert(s);
    }
    return rc;
}

int oxhip_dev_gemm_timed(oxhip_ctx* c, const oxhip_weight* w, const void* x, int x_dtype, size_t t, void* y, int y_dtype, int variant,
                         void* stream, void* ev_start, void* ev_stop) {
    g_kernel_span.start = static_cast<hipEvent_t>(ev_start);
    g_kernel_span.stop = static_cast<hipEvent_t>(ev_stop);
    const int ok = oxhip_dev_gemm(c, w, x, x_dtype, t, y, y_dtype, variant, stream);
    g_kernel_span = KernelSpan{};
    return ok;
}

}  // extern "C"
