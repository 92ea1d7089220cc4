// Device-resident ops of the reference's single-token decode graph (src/gpu_decode.rs:52-340), so that a token's
// linears and its MoE layer run back to back on buffers that stay in HBM: Op::Linear with its LinMode, Op::Norm fused
// with the quantization of the next linear's input, Op::Route, Op::Experts, Op::Glu, and the arena they work in.
#include <algorithm>

#include "backend.hpp"

using namespace oxhip;

namespace oxhip {

// The scratch of the device-pointer entry points, one set per stream: launches on one stream are ordered, so they may
// share; launches on different streams may overlap and must not. A stream's entry holds no device memory until a call
// needs some: the partial rows and arrival counters of the decode kernels (16 MiB + 2 MiB) come with the first launch on
// that stream whose shape slices K across workgroups (`slices`), their counters cleared by a kernel on that same stream
// (ordered before the launch that follows, and no wait for the rest of the device).
StreamScratch* scratch_for(oxhip_ctx* c, hipStream_t s, bool slices) {
    std::lock_guard<std::mutex> g(c->smu);
    StreamScratch* sc;
    auto it = c->per_stream.find(s);
    if (it != c->per_stream.end()) {
        sc = it->second;
    } else {
        sc = new StreamScratch();
        c->per_stream.emplace(s, sc);
    }
    if (slices && !sc->dec.partial) {
        if (stream_recording(s)) {  // (smu is held: the failure is noted here, not through may_allocate)
            c->record_failed.insert(s);
            return nullptr;
        }
        DecodeScratch d;
        d.partial_floats = c->dec.partial_floats;
        d.ncounters = c->dec.ncounters;
        if (hipMalloc(reinterpret_cast<void**>(&d.partial), d.partial_floats * 4) != hipSuccess ||
            hipMalloc(reinterpret_cast<void**>(&d.counters), d.ncounters * 4) != hipSuccess ||
            launch_fill_zero(d.counters, d.ncounters, s) != hipSuccess) {
            if (d.partial) (void)hipFree(d.partial);
            if (d.counters) (void)hipFree(d.counters);
            return nullptr;
        }
        sc->dec = d;
    }
    return sc;
}

static void release_scratch(StreamScratch* sc) {
    if (sc->dec.partial) (void)hipFree(sc->dec.partial);
    if (sc->dec.counters) (void)hipFree(sc->dec.counters);
    sc->tmp.release();
    sc->gemm_ws.release();
    delete sc;
}

void free_stream_scratch(oxhip_ctx* c) {
    std::lock_guard<std::mutex> g(c->smu);
    for (auto& kv : c->per_stream) release_scratch(kv.second);
    c->per_stream.clear();
}

bool needs_slices(const oxhip_weight* w) {
    if (w->v.fmt == FMT_FP8) return skinny_fp8_ok(w->v, 1);  // (its one-pass decode kernel keeps its packed rows in the same scratch)
    size_t p = 0, n = 0;
    decode_scratch_need(w->v, &p, &n);
    return p != 0;
}

}  // namespace oxhip

extern "C" {

int oxhip_stream_release(oxhip_ctx* c, void* stream) {
    if (!c) {
        set_error("stream_release: null context");
        return 0;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    HIP_TRY(hipStreamSynchronize(s), "stream_release: the stream's work failed");  // its launches may still use the scratch
    std::lock_guard<std::mutex> g(c->smu);
    auto it = c->per_stream.find(s);
    if (it == c->per_stream.end()) return 1;
    release_scratch(it->second);
    c->per_stream.erase(it);
    return 1;
}

void* oxhip_buf_alloc(oxhip_ctx* c, size_t bytes) {
    if (!c || !bytes) {
        set_error("buf_alloc: bad arguments");
        return nullptr;
    }
    void* p = nullptr;
    if (hipSetDevice(c->device) != hipSuccess || hipMalloc(&p, bytes) != hipSuccess) {
        set_error("buf_alloc: device memory short");
        return nullptr;
    }
    if (hipMemset(p, 0, bytes) != hipSuccess) {
        (void)hipFree(p);
        set_error("buf_alloc: clearing failed");
        return nullptr;
    }
    return p;
}

void oxhip_buf_free(oxhip_ctx* c, void* p) {
    if (!p) return;
    if (c) (void)hipSetDevice(c->device);
    (void)hipFree(p);
}

int oxhip_buf_write(oxhip_ctx* c, void* dst, const void* src, size_t bytes, void* stream) {
    if (!c || !dst || !src) {
        set_error("buf_write: null argument");
        return 0;
    }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)), "buf_write");
    HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "buf_write");  // the host buffer may be reused at once
    return 1;
}

int oxhip_buf_read(oxhip_ctx* c, void* dst, const void* src, size_t bytes, void* stream) {
    if (!c || !dst || !src) {
        set_error("buf_read: null argument");
        return 0;
    }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)), "buf_read");
    HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "buf_read");
    return 1;
}

int oxhip_dev_rmsnorm_quantize(oxhip_ctx* c, const float* x, const float* w_f32, const uint16_t* w_bf16, float eps, size_t t, size_t n,
                               float* out, const oxhip_qact* q, void* stream) {
    if (!c || !x || (!out && !q) || n % 32 || (w_f32 && w_bf16) || (q && (q->n_in != n || q->t < t))) {
        set_error("rmsnorm_quantize: bad arguments (n must be a multiple of 32, one kind of weights, outputs of the input's shape)");
        return 0;
    }
    HIP_TRY(launch_rmsnorm_quantize(x, w_f32, w_bf16, eps, t, n, out, q, static_cast<hipStream_t>(stream)), "rmsnorm_quantize launch");
    return 1;
}

int oxhip_dev_norm(oxhip_ctx* c, const float* x, float* out, const float* w_f32, const uint16_t* w_bf16, float pre, size_t n, size_t rows,
                   size_t x_stride, size_t out_stride, float eps, int add, const oxhip_qact* q, void* stream) {
    if (!c || !x || (!out && !q) || n % 32 || !n || (w_f32 && w_bf16) || (q && (q->n_in != n || q->t < rows)) || (add && !out) ||
        (x_stride && x_stride < n) || (out_stride && out_stride < n)) {
        set_error("norm: bad arguments (n a multiple of 32, one kind of weights, strides of at least n floats, `add` needs `out`)");
        return 0;
    }
    HIP_TRY(launch_rmsnorm_quantize(x, w_f32, w_bf16, eps, rows, n, out, q, static_cast<hipStream_t>(stream), pre, add != 0, x_stride, out_stride),
            "norm launch");
    return 1;
}

int oxhip_dev_glu(oxhip_ctx* c, const float* g, const float* u, size_t n, int gelu, float* y, void* stream) {
    if (!c || !g || !u || !y) {
        set_error("glu: null argument");
        return 0;
    }
    HIP_TRY(launch_glu(g, u, n, gelu != 0, y, static_cast<hipStream_t>(stream)), "glu launch");
    return 1;
}

int oxhip_dev_linear(oxhip_ctx* c, const oxhip_weight* w, const oxhip_weight* w2, const oxhip_qact* xa, const float* x, size_t t, float* y,
                     uint32_t mode, const float* gate, void* stream) {
    if (!c || !w || !y || t == 0 || t > 16 || mode > OXHIP_LIN_ADD_GATED) {
        set_error("linear: bad arguments (1 <= t <= 16)");
        return 0;
    }
    const bool pair = mode == OXHIP_LIN_SILU_PAIR || mode == OXHIP_LIN_GELU_PAIR;
    if (pair != (w2 != nullptr) || (mode == OXHIP_LIN_ADD_GATED) != (gate != nullptr)) {
        set_error("linear: the pair modes take a second matrix, the gated mode a gate, the others neither");
        return 0;
    }
    if (pair && (w2->v.n_in != w->v.n_in || w2->v.n_out != w->v.n_out || w2->v.fmt != w->v.fmt)) {
        set_error("linear: the matrices of a pair share shape and storage format (pairable, src/gpu_decode.rs:340-349)");
        return 0;
    }
    QActView v{};
    if (is_dense(w)) {
        if (!x) {
            set_error("linear: float-stored weights take f32 rows");
            return 0;
        }
    } else {
        if (!xa || xa->n_in != w->v.n_in || xa->t < t) {
            set_error("linear: quantized activations missing or of another shape");
            return 0;
        }
        v = view_of(*xa);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    StreamScratch* sc = scratch_for(c, s, needs_slices(w));
    if (!sc) {
        set_error(stream_recording(s) ? "linear: the stream's K-slice scratch does not exist yet and a plan records on it (run the chain once before recording)"
                                      : "linear: device memory short");
        return 0;
    }
    const size_t n_out = w->v.n_out;
    Epi epi;
    epi.mode = mode == OXHIP_LIN_ADD ? EPI_ADD : mode == OXHIP_LIN_ADD_GATED ? EPI_ADD_GATED : EPI_STORE;
    epi.gate = gate;
    if (!pair) {
        if (mfma_decode_format(w->v.fmt)) {
            HIP_TRY(launch_decode_mfma(w->v, v, t, y, sc->dec, s, nullptr, nullptr, epi), "linear launch");
            return 1;
        }
        if (epi.mode == EPI_STORE) {
            HIP_TRY(launch_decode(w->v, v, x, t, y, s, sc->dec), "linear launch");
            return 1;
        }
        // formats whose kernels only store: the product goes to scratch, the mode is a small kernel of its own
        if (sc->tmp.cap < t * n_out * 4 && !may_allocate(c, s, "linear")) return 0;
        if (!sc->tmp.grow(t * n_out * 4)) {
            set_error("linear: device memory short");
            return 0;
        }
        float* tmp = static_cast<float*>(sc->tmp.p);
        HIP_TRY(launch_decode(w->v, v, x, t, tmp, s, sc->dec), "linear launch");
        HIP_TRY(launch_epilogue(tmp, t, n_out, y, epi, s), "linear epilogue launch");
        return 1;
    }
    // y = act(W x) * (W2 x). The matrix-core decode kernel pairs the two matrices' tiles of the same rows in one workgroup and
    // applies the gate in its output stage: one launch, no intermediate rows (bit-identical to the two products and Op::Glu)
    if (decode_pair_ok(w->v)) {
        Epi pe;
        pe.pair_p0 = w2->v.p0;
        pe.pair_act = mode == OXHIP_LIN_GELU_PAIR ? 1u : 0u;
        HIP_TRY(launch_decode_mfma(w->v, v, t, y, sc->dec, s, nullptr, nullptr, pe), "linear pair launch");
        return 1;
    }
    // the other formats: both products into scratch, then the gate
    if (sc->tmp.cap < 2 * t * n_out * 4 && !may_allocate(c, s, "linear")) return 0;
    if (!sc->tmp.grow(2 * t * n_out * 4)) {
        set_error("linear: device memory short");
        return 0;
    }
    float* g = static_cast<float*>(sc->tmp.p);
    float* u = g + t * n_out;
    HIP_TRY(launch_decode(w->v, v, x, t, g, s, sc->dec), "linear launch");
    HIP_TRY(launch_decode(w2->v, v, x, t, u, s, sc->dec), "linear launch");
    HIP_TRY(launch_glu(g, u, t * n_out, mode == OXHIP_LIN_GELU_PAIR, y, s), "linear gate launch");
    return 1;
}

int oxhip_dev_route(oxhip_ctx* c, const float* x, const float* router, const float* gate, size_t t, size_t n_exp, size_t h, size_t k,
                    float* logits, uint32_t* sel, const float* expert_scale, void* stream) {
    if (!c || !x || !router || !logits || !sel || !t || !k || k > 32 || k > n_exp || n_exp > 1024 || !h) {
        set_error("route: bad arguments (k <= 32, k <= n_experts <= 1024)");
        return 0;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(launch_router_logits(x, router, gate, t, n_exp, h, logits, s), "router launch");
    // sel: the k ids of every token, then their k weights (for one token: k ids then k weights, src/gpu_decode.rs:158-160)
    HIP_TRY(launch_route_top_k(logits, t, n_exp, k, sel, reinterpret_cast<float*>(sel + t * k), s, n_exp + (gate ? 1 : 0), expert_scale),
            "route_top_k launch");
    return 1;
}

}  // extern "C"
