// Definitions shared by the files that implement the C ABI: the context, the device weight, staging.
#pragma once
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "internal.hpp"
#include "layout.hpp"

namespace oxhip {

#define HIP_TRY(expr, what)                                                              \
    do {                                                                                 \
        hipError_t e__ = (expr);                                                         \
        if (e__ != hipSuccess) {                                                         \
            oxhip::set_error(std::string(what) + ": " + hipGetErrorString(e__));         \
            return 0;                                                                    \
        }                                                                                \
    } while (0)

constexpr size_t VRAM_RESERVE = 512ull << 20;  // kept free for activations (src/cuda.rs:573-588)

struct DevBuf {
    void* p = nullptr;
    size_t cap = 0;
    bool grow(size_t need) {
        if (cap >= need && p) return true;
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
        size_t want = (need < 256 ? 256 : need) * 2;
        if (hipMalloc(&p, want) != hipSuccess) {
            p = nullptr;
            return false;
        }
        cap = want;
        return true;
    }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
    }
};

// Scratch of the device-pointer entry points on one stream: the decode kernels' K-slice rows and counters, the
// products of a gate / up pair (and of formats whose kernels only store) before their epilogue, the prefill GEMMs'
// packed activations.
struct StreamScratch {
    DecodeScratch dec;
    DevBuf tmp;
    DevBuf gemm_ws;
};

}  // namespace oxhip

struct oxhip_weight {
    oxhip::WeightView v{};
    void* base = nullptr;
    size_t bytes = 0;
};

#include <set>

struct oxhip_ctx {
    int device = 0;
    std::string name;
    hipStream_t stream = nullptr;
    std::mutex mu;  // serializes the host-pointer surface (staging is shared), as Mutex<Staging> does
    oxhip::DevBuf x, xq, y;
    oxhip::DevBuf gemm_ws;  // packed activations of the prefill GEMMs
    oxhip::DecodeScratch dec;  // partial rows and counters of the decode kernels that split K across workgroups (host surface, on `stream`)
    std::mutex smu;            // guards per_stream
    std::map<hipStream_t, oxhip::StreamScratch*> per_stream;  // the device-pointer entry points' scratch, by calling stream
    std::set<hipStream_t> record_failed;  // streams whose plan recording met a call that had to allocate (guarded by smu)
    double ms_in = 0, ms_gpu = 0, ms_out = 0;
    size_t calls = 0;
};

namespace oxhip {

// backend_gemm.hip: packs x into `ws` and runs the bf16-matrix-core GEMM (1 = done, 0 = declined with the error set)
int gemm_bf16_run(DevBuf& ws, const oxhip_weight* w, const void* x, bool x_bf16, size_t t, void* y, bool y_bf16, hipStream_t s);
// backend_graph.hip: the calling stream's scratch (nullptr when memory is short). `slices`: the launch that follows may
// slice K across workgroups, so the entry must hold the decode kernels' partial rows and counters (allocated on first need).
StreamScratch* scratch_for(oxhip_ctx* c, hipStream_t s, bool slices);
void free_stream_scratch(oxhip_ctx* c);
bool needs_slices(const oxhip_weight* w);  // a decode launch of this weight alone uses the stream's decode scratch (K slices across workgroups, FP8's packed rows)

// True while `s` records a plan (stream capture): a call must then not allocate, free, wait or clear with a memset.
inline bool stream_recording(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return s && hipStreamIsCapturing(s, &st) == hipSuccess && st == hipStreamCaptureStatusActive;
}
// Called before a device-pointer entry point allocates on behalf of stream `s`: false (error set, the recording marked
// failed so that oxhip_plan_end declines) while a plan records there.
inline bool may_allocate(oxhip_ctx* c, hipStream_t s, const char* who) {
    if (!stream_recording(s)) return true;
    {
        std::lock_guard<std::mutex> g(c->smu);
        c->record_failed.insert(s);
    }
    set_error(std::string(who) + ": this call would have to allocate device memory while a plan records on its stream (run the chain once before recording)");
    return false;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline QActView view_of(const oxhip_qact& a) { return QActView{a.q, a.scales, a.sums, a.fsums, a.hsums, a.sums16}; }

// A QAct for t rows of n_in carved out of one buffer.
inline size_t qact_bytes(size_t t, size_t n_in) {
    size_t b32 = t * n_in / 32, b16 = t * n_in / 16;
    return align_up(t * n_in, 256) + 3 * align_up(b32 * 4, 256) + 2 * align_up(b16 * 4, 256);
}
inline oxhip_qact carve_qact(void* base, size_t t, size_t n_in) {
    uint8_t* p = static_cast<uint8_t*>(base);
    size_t b32 = t * n_in / 32, b16 = t * n_in / 16;
    oxhip_qact a{};
    if (!p) return a;
    a.q = reinterpret_cast<int8_t*>(p);
    p += align_up(t * n_in, 256);
    a.scales = reinterpret_cast<float*>(p);
    p += align_up(b32 * 4, 256);
    a.sums = reinterpret_cast<int32_t*>(p);
    p += align_up(b32 * 4, 256);
    a.fsums = reinterpret_cast<float*>(p);
    p += align_up(b32 * 4, 256);
    a.hsums = reinterpret_cast<float*>(p);
    p += align_up(b16 * 4, 256);
    a.sums16 = reinterpret_cast<int32_t*>(p);
    a.t = t;
    a.n_in = n_in;
    return a;
}

// float-stored matrices (is_float, src/ggml.rs:219-224): f32 activations at decode sizes
inline bool is_dense(const oxhip_weight* w) { return w->v.fmt == FMT_FP8 || w->v.fmt == FMT_BF16 || w->v.fmt == FMT_NVFP4; }

}  // namespace oxhip
