// Backend::upload_moe / moe / matvec_rows (src/gpu.rs:165, :206-248 of the reference) over the grouped
// decode kernel, plus their device-pointer forms.
#include <cstdlib>
#include <cstring>
#include <vector>

#include "backend.hpp"

using namespace oxhip;

struct oxhip_moe {
    std::vector<oxhip_weight*> gate_up, up, down;  // up empty when gate/up are fused
    size_t n_exp = 0, h = 0, inter = 0;
    uint32_t act_kind = 0;
    float act_param = 0;
    const uint8_t** bases_gu = nullptr;  // device arrays of tile-packed bases
    const uint8_t** bases_up = nullptr;
    const uint8_t** bases_dn = nullptr;
    DevBuf ws;                           // scratch of one pass
    size_t ws_pairs = 0, ws_t = 0;
    uint32_t mode = OXHIP_MOE_AUTO;      // oxhip_moe_set_mode
    bool counters_dirty = false;         // a pass failed part-way: the arrival counters may not be back at zero
};

namespace {

bool mfma_format(const oxhip_weight* w) { return w->v.fmt == FMT_Q8_0 || w->v.fmt == FMT_Q4_K || t4m_format(w->v.fmt); }

size_t up256(size_t v) { return (v + 255) / 256 * 256; }

constexpr size_t COMB_GROUPS = 4096;  // row groups of the down projection that may meet through counters (h <= 65536)

// The scratch of one pass, carved from one allocation.
struct Scratch {
    int* row_of;
    int* src;
    int4* chunks;
    int* nchunks;
    oxhip_qact xa;  // x quantized, [t][h]
    float* gu;      // [pairs][2 inter] (fused) or g [pairs][inter] then u [pairs][inter]
    float* a;       // [pairs][inter]
    oxhip_qact aq;  // a quantized
    float* o;       // [pairs][h]
    void* fx;       // bf16 fragments of the chunks' rows of x, and of a (the prefill form: chunks of up to 16 rows)
    void* fa;
    uint32_t* counters;  // arrival counters of the down launch's row groups (zero between launches)
    uint32_t max_chunks;
    size_t bytes;
};

// The chunk table holds the most chunks any plan can cut: an expert with c routed rows yields ceil(c / rows per chunk)
// chunks, at most c of them (chunks of one row, a one-token pass) plus one per expert in use. Every part grows with t
// and pairs, so a buffer sized for the largest of each serves any smaller pass.
Scratch carve(uint8_t* base, size_t t, size_t pairs, size_t n_exp, size_t h, size_t inter) {
    Scratch s{};
    s.max_chunks = (uint32_t)((pairs < n_exp ? pairs : n_exp) + pairs + 1);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        uint8_t* p = base ? base + off : nullptr;
        off += up256(bytes);
        return p;
    };
    // (the counters first: their place must not depend on the pass's size, they stay zero from one pass to the next)
    s.counters = reinterpret_cast<uint32_t*>(take((size_t)COMB_GROUPS * CTR_STRIDE * 4));
    s.row_of = reinterpret_cast<int*>(take(pairs * 4));
    s.src = reinterpret_cast<int*>(take(pairs * 4));
    s.chunks = reinterpret_cast<int4*>(take((size_t)s.max_chunks * 16));
    s.nchunks = reinterpret_cast<int*>(take(4));
    s.xa = carve_qact(take(qact_bytes(t, h)), t, h);
    s.gu = reinterpret_cast<float*>(take(pairs * 2 * inter * 4));
    s.a = reinterpret_cast<float*>(take(pairs * inter * 4));
    s.aq = carve_qact(take(qact_bytes(pairs, inter)), pairs, inter);
    s.o = reinterpret_cast<float*>(take(pairs * h * 4));
    const size_t chunks16 = (pairs < n_exp ? pairs : n_exp) + pairs / 16 + 1;
    const bool prefill = pairs / n_exp >= 6 && h % 128 == 0 && inter % 128 == 0;
    s.fx = take(prefill ? moe_bf16_frag_bytes(chunks16, h) : 0);
    s.fa = take(prefill ? moe_bf16_frag_bytes(chunks16, inter) : 0);
    s.bytes = off;
    return s;
}

// Routing inside the pass: with `logits` ([t] rows `logit_stride` apart) the top-k of every token is formed first, into
// route_idx / route_w (then outputs: [t, k] each).
struct RouteIn {
    const float* logits = nullptr;
    size_t stride = 0;
    const float* expert_scale = nullptr;
};

int moe_pass(oxhip_ctx* c, oxhip_moe* m, const float* x, size_t t, const uint32_t* route_idx, const float* route_w, size_t k,
             float* y, hipStream_t s, bool add, const RouteIn& rin) {
    const size_t pairs = t * k, h = m->h, inter = m->inter;
    if (!pairs) return 1;
    uint32_t* ridx_out = const_cast<uint32_t*>(route_idx);
    float* rw_out = const_cast<float*>(route_w);
    bool routed = rin.logits == nullptr;  // the routes are there (given, or already formed)
    if (pairs > m->ws_pairs || t > m->ws_t) {
        if (!may_allocate(c, s, "moe")) return 0;
        (void)hipStreamSynchronize(s);  // an earlier pass may still read the old scratch
        const size_t np = pairs > m->ws_pairs ? pairs : m->ws_pairs, nt = t > m->ws_t ? t : m->ws_t;
        Scratch probe = carve(nullptr, nt, np, m->n_exp, h, inter);
        if (!m->ws.grow(probe.bytes)) {
            m->ws_pairs = m->ws_t = 0;
            set_error("moe: device memory short");
            return 0;
        }
        m->ws_pairs = np;
        m->ws_t = nt;
        // the arrival counters start at zero (every launch leaves them so); the buffer moved, and its layout with it
        HIP_TRY(hipMemsetAsync(m->ws.p, 0, m->ws.cap, s), "moe scratch clear");
    }
    Scratch sc = carve(static_cast<uint8_t*>(m->ws.p), t, pairs, m->n_exp, h, inter);
    if (m->counters_dirty) {
        // an earlier pass ended in an error after its down launch may have started: the last workgroup of each row group
        // puts its counter back to zero, which a failed launch may not have done
        HIP_TRY(launch_fill_zero(sc.counters, (size_t)COMB_GROUPS * CTR_STRIDE, s), "moe counter clear launch");
        m->counters_dirty = false;
    }
    // Rows per chunk: one pass over an expert's weights serves a whole chunk, so chunks grow with the rows an expert
    // gets on average (8 rows per matrix-core instruction, up to 4 instructions per weight record).
    uint32_t max_rows = (uint32_t)(t < 8 ? t : 8);
    const size_t avg = pairs / m->n_exp;
    if (avg >= 6 && mfma_format(m->gate_up[0])) max_rows = avg >= 20 ? 32 : 16;
#ifdef OXHIP_TUNING  // tuning builds only: rows per chunk in OXHIP_MOE_CHUNK
    if (const char* e = getenv("OXHIP_MOE_CHUNK")) {
        const int v = atoi(e);
        if ((v == 8 || v == 16 || v == 32) && t >= 8) max_rows = (uint32_t)v;
    }
#endif
    // Prefill passes over MLX 4-bit experts (six or more routed rows per expert on average) take the bf16 form: see
    // moe_bf16.hip. OXHIP_MOE_INT8 (oxhip_moe_set_mode) keeps the integer path (the 1e-3 accuracy class) at any size.
    const bool fused = m->up.empty();
    const size_t grid_chunks16 = (pairs < m->n_exp ? pairs : m->n_exp) + pairs / 16 + 1;
    const bool bf16_form = avg >= 6 && fused && moe_bf16_ok(m->gate_up[0]->v) && moe_bf16_ok(m->down[0]->v) && m->mode != OXHIP_MOE_INT8 &&
                           reinterpret_cast<uintptr_t>(x) % 16 == 0 && grid_chunks16 <= 65535;
    if (bf16_form) max_rows = 16;
    if (!bf16_form) {
        // The grouped integer kernel stages a chunk's activations in LDS, one set per group of 8 rows: long rows take
        // smaller chunks (checked for every projection before anything is launched).
        auto fits = [&](uint32_t rows) {
            return decode_grouped_fits(m->gate_up[0]->v, rows) && decode_grouped_fits(m->down[0]->v, rows) &&
                   (fused || decode_grouped_fits(m->up[0]->v, rows));
        };
        while (max_rows > 8 && !fits(max_rows)) max_rows /= 2;
        if (!fits(max_rows)) {
            set_error("moe: rows of these experts are too long for the grouped kernel's staging");
            return 0;
        }
    }
    const uint32_t grid_chunks = (uint32_t)((pairs < m->n_exp ? pairs : m->n_exp) + pairs / max_rows + 1);
    GroupView g{};
    g.chunks = sc.chunks;
    g.nchunks = sc.nchunks;
    // One token over fused gate / up experts needs no plan: chunk j is route j (see GroupView::direct); its routing
    // and the quantization of x share a launch, and the pass is three launches.
    const bool direct = !bf16_form && t == 1 && fused && decode_grouped_glu_ok(m->gate_up[0]->v, inter) && row_tiles((uint32_t)h) <= COMB_GROUPS;
    if (!routed && !(direct && m->n_exp <= 256)) {
        HIP_TRY(launch_route_top_k(rin.logits, t, m->n_exp, k, ridx_out, rw_out, s, rin.stride, rin.expert_scale), "route_top_k launch");
        routed = true;
    }
    if (bf16_form) {
        HIP_TRY(launch_moe_plan(route_idx, pairs, k, m->n_exp, max_rows, sc.row_of, sc.src, sc.chunks, sc.nchunks, s), "moe plan launch");
        HIP_TRY(launch_moe_pack_bf16(x, h, sc.src, sc.chunks, sc.nchunks, grid_chunks, sc.fx, s, moe_bf16_std_geometry(m->gate_up[0]->v)), "moe pack launch");
        g.bases = m->bases_gu;
        if (moe_bf16_glu_ok(m->gate_up[0]->v, inter, grid_chunks)) {
            // the gate / up launch pairs gate and up tiles per workgroup, applies the activation and writes the down projection's fragments
            HIP_TRY(launch_moe_bf16(m->gate_up[0]->v, g, grid_chunks, sc.fx, nullptr, s, inter, m->act_kind, m->act_param, moe_bf16_std_geometry(m->down[0]->v),
                                    sc.fa),
                    "moe gate launch");
        } else {
            HIP_TRY(launch_moe_bf16(m->gate_up[0]->v, g, grid_chunks, sc.fx, sc.gu, s), "moe gate launch");
            HIP_TRY(launch_moe_act_pack_bf16(sc.gu, sc.gu + inter, 2 * inter, inter, m->act_kind, m->act_param, sc.chunks, sc.nchunks, grid_chunks, sc.fa, s,
                                             moe_bf16_std_geometry(m->down[0]->v)),
                    "moe act launch");
        }
        g.bases = m->bases_dn;
        HIP_TRY(launch_moe_bf16(m->down[0]->v, g, grid_chunks, sc.fa, sc.o, s), "moe down launch");
    } else {
        if (direct) {
            if (!routed) HIP_TRY(launch_route_quantize(rin.logits, 1, m->n_exp, k, ridx_out, rw_out, rin.stride, rin.expert_scale, x, h, sc.xa, s), "route + quantize launch");
            else HIP_TRY(launch_quantize_act(x, 1, h, sc.xa, s), "moe quantize launch");
            g.direct = route_idx;
            g.direct_n = (uint32_t)k;
            g.direct_x0 = 1;
        } else {
            HIP_TRY(launch_moe_front(route_idx, pairs, k, m->n_exp, max_rows, sc.row_of, sc.src, sc.chunks, sc.nchunks, x, t, h, sc.xa, s), "moe plan launch");
        }
        // gate / up over the routed rows of x (row i of the gathered order is token src[i])
        g.rowmap = direct ? nullptr : sc.src;
        g.bases = m->bases_gu;
        // fused gate / up experts whose launch pairs gate and up tiles: the activation and the quantization of its output
        // are the launch's own output stage; the down launch then also combines (the last workgroup of a row group to
        // finish adds the routed rows in route order): three launches for a decode-sized pass
        // (decode-sized passes only: a large pass has enough rows to fill launches of their own, and its combination is
        // too much work for the one workgroup per row group that would do it)
        const bool small = t <= 8;
        const bool glu_fused = small && fused && decode_grouped_glu_ok(m->gate_up[0]->v, inter);
        const bool comb_fused = small && row_tiles((uint32_t)h) <= COMB_GROUPS;
        if (glu_fused) {
            GroupView gg = g;
            gg.glu_inter = (uint32_t)inter;
            gg.act_kind = m->act_kind;
            gg.act_param = m->act_param;
            gg.aq_q = sc.aq.q;
            gg.aq_scales = sc.aq.scales;
            gg.aq_sums = sc.aq.sums;
            gg.aq_fsums = sc.aq.fsums;
            gg.aq_hsums = sc.aq.hsums;
            gg.aq_sums16 = sc.aq.sums16;
            HIP_TRY(launch_decode_mfma_grouped(m->gate_up[0]->v, view_of(sc.xa), gg, grid_chunks, max_rows, sc.gu, s), "moe gate launch");
        } else {
        HIP_TRY(launch_decode_mfma_grouped(m->gate_up[0]->v, view_of(sc.xa), g, grid_chunks, max_rows, sc.gu, s), "moe gate launch");
        const float* up_out = sc.gu + inter;
        size_t stride = 2 * inter;
        if (!fused) {
            g.bases = m->bases_up;
            float* u = sc.gu + pairs * inter;
            HIP_TRY(launch_decode_mfma_grouped(m->up[0]->v, view_of(sc.xa), g, grid_chunks, max_rows, u, s), "moe up launch");
            up_out = u;
            stride = inter;
        }
        if (inter % 32 == 0 && stride % 4 == 0) {
            HIP_TRY(launch_moe_act_quantize(sc.gu, up_out, stride, pairs, inter, m->act_kind, m->act_param, sc.aq, s), "moe act launch");
        } else {
            HIP_TRY(launch_moe_act(sc.gu, up_out, stride, pairs, inter, m->act_kind, m->act_param, sc.a, s), "moe act launch");
            HIP_TRY(launch_quantize_act(sc.a, pairs, inter, sc.aq, s), "moe quantize launch");
        }
        }
        g.rowmap = nullptr;
        g.bases = m->bases_dn;
        g.direct_x0 = 0;
        if (comb_fused) {
            g.comb_y = y;
            g.row_of = direct ? nullptr : sc.row_of;
            g.route_w = route_w;
            g.comb_t = (uint32_t)t;
            g.comb_k = (uint32_t)k;
            g.comb_add = add ? 1u : 0u;
            g.comb_counters = sc.counters;
        }
        HIP_TRY(launch_decode_mfma_grouped(m->down[0]->v, view_of(sc.aq), g, grid_chunks, max_rows, sc.o, s), "moe down launch");
        if (comb_fused) return 1;
    }
    HIP_TRY(launch_moe_combine(sc.o, sc.row_of, route_w, t, k, h, y, s, add), "moe combine launch");
    return 1;
}

// A pass that fails part-way (a launch error) may leave the down launch's arrival counters above zero; the next pass on
// this layer clears them first.
int moe_run(oxhip_ctx* c, oxhip_moe* m, const float* x, size_t t, const uint32_t* route_idx, const float* route_w, size_t k,
            float* y, hipStream_t s, bool add = true, const RouteIn& rin = RouteIn{}) {
    const int rc = moe_pass(c, m, x, t, route_idx, route_w, k, y, s, add, rin);
    if (!rc) m->counters_dirty = true;
    return rc;
}

}  // namespace

extern "C" {

void oxhip_free_moe(oxhip_ctx* c, oxhip_moe* m) {
    if (!m) return;
    if (c) {
        (void)hipSetDevice(c->device);
        (void)hipDeviceSynchronize();
    }
    for (auto* w : m->gate_up) oxhip_free_weight(c, w);
    for (auto* w : m->up) oxhip_free_weight(c, w);
    for (auto* w : m->down) oxhip_free_weight(c, w);
    if (m->bases_gu) (void)hipFree(m->bases_gu);
    if (m->bases_up) (void)hipFree(m->bases_up);
    if (m->bases_dn) (void)hipFree(m->bases_dn);
    m->ws.release();
    delete m;
}

oxhip_moe* oxhip_upload_moe(oxhip_ctx* c, const oxhip_weight_desc* gate_up, const oxhip_weight_desc* up, const oxhip_weight_desc* down,
                            size_t n_experts, size_t h, size_t inter, uint32_t act_kind, float act_param) {
    if (!c || !gate_up || !down || !n_experts || !h || !inter) {
        set_error("upload_moe: null argument");
        return nullptr;
    }
    if (act_kind > OXHIP_ACT_SILU_CLAMP) {
        set_error("upload_moe: this activation runs on the CPU only");
        return nullptr;
    }
    if (h % 32 || inter % 32) {
        set_error("upload_moe: h and inter must be multiples of 32");
        return nullptr;
    }
    auto* m = new oxhip_moe();
    m->n_exp = n_experts;
    m->h = h;
    m->inter = inter;
    m->act_kind = act_kind;
    m->act_param = act_param;
    auto fail = [&](const std::string& why) -> oxhip_moe* {
        const std::string msg = "upload_moe: " + why;
        oxhip_free_moe(c, m);
        set_error(msg);
        return nullptr;
    };
    const size_t gu_rows = up ? inter : 2 * inter;
    for (size_t e = 0; e < n_experts; e++) {
        if (gate_up[e].n_out != gu_rows || gate_up[e].n_in != h || down[e].n_out != h || down[e].n_in != inter ||
            (up && (up[e].n_out != inter || up[e].n_in != h)))
            return fail("expert " + std::to_string(e) + " has another shape");
        oxhip_weight* w = oxhip_upload(c, &gate_up[e]);
        if (!w) return fail(oxhip_last_error());
        m->gate_up.push_back(w);
        if (up) {
            w = oxhip_upload(c, &up[e]);
            if (!w) return fail(oxhip_last_error());
            m->up.push_back(w);
        }
        w = oxhip_upload(c, &down[e]);
        if (!w) return fail(oxhip_last_error());
        m->down.push_back(w);
    }
    auto same = [&](const std::vector<oxhip_weight*>& v) {
        for (auto* w : v)
            if (w->v.fmt != v[0]->v.fmt || !mfma_format(w)) return false;
        return true;
    };
    if (!same(m->gate_up) || !same(m->down) || (up && !same(m->up))) return fail("experts must share one of the formats the grouped kernel runs (Q8_0, Q4_K, Q4_0, MXFP4, MLX Q4)");
    auto table = [&](const std::vector<oxhip_weight*>& v, const uint8_t*** out) {
        std::vector<const uint8_t*> host(v.size());
        for (size_t i = 0; i < v.size(); i++) host[i] = v[i]->v.p0;
        if (hipMalloc(reinterpret_cast<void**>(out), host.size() * sizeof(void*)) != hipSuccess) return false;
        return hipMemcpy(*out, host.data(), host.size() * sizeof(void*), hipMemcpyHostToDevice) == hipSuccess;
    };
    if (!table(m->gate_up, &m->bases_gu) || !table(m->down, &m->bases_dn) || (up && !table(m->up, &m->bases_up)))
        return fail("device memory short");
    return m;
}

int oxhip_moe_set_mode(oxhip_moe* m, uint32_t mode) {
    if (!m || mode > OXHIP_MOE_INT8) {
        set_error("moe_set_mode: bad arguments");
        return 0;
    }
    m->mode = mode;
    return 1;
}

int oxhip_dev_route_top_k(oxhip_ctx* c, const float* logits, size_t t, size_t n_experts, size_t k, uint32_t* idx, float* w, void* stream) {
    if (!c || !logits || !idx || !w || !k || k > 32 || k > n_experts || n_experts > 1024) {
        set_error("route_top_k: bad arguments (k <= 32, k <= n_experts <= 1024)");
        return 0;
    }
    HIP_TRY(launch_route_top_k(logits, t, n_experts, k, idx, w, static_cast<hipStream_t>(stream)), "route_top_k launch");
    return 1;
}

int oxhip_dev_moe(oxhip_ctx* c, oxhip_moe* m, const float* x, size_t t, const uint32_t* route_idx, const float* route_w, size_t k,
                  float* y, void* stream) {
    if (!c || !m || !x || !route_idx || !route_w || !y || !k) {
        set_error("moe: null argument");
        return 0;
    }
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    return moe_run(c, m, x, t, route_idx, route_w, k, y, static_cast<hipStream_t>(stream));
}

int oxhip_dev_experts(oxhip_ctx* c, oxhip_moe* m, const float* x, size_t t, const uint32_t* sel, size_t k, float* y, int add, void* stream) {
    if (!c || !m || !x || !sel || !y || !k || !t || k > 32) {
        set_error("experts: bad arguments (1 <= k <= 32)");
        return 0;
    }
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    return moe_run(c, m, x, t, sel, reinterpret_cast<const float*>(sel + t * k), k, y, static_cast<hipStream_t>(stream), add != 0);
}

int oxhip_dev_moe_routed(oxhip_ctx* c, oxhip_moe* m, const float* x, size_t t, const float* logits, size_t logit_stride, size_t k,
                         const float* expert_scale, uint32_t* sel, float* y, int add, void* stream) {
    if (!c || !m || !x || !logits || !sel || !y || !k || !t || k > 32 || k > m->n_exp || m->n_exp > 1024 || (logit_stride && logit_stride < m->n_exp)) {
        set_error("moe_routed: bad arguments (k <= 32, k <= n_experts <= 1024)");
        return 0;
    }
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    RouteIn rin;
    rin.logits = logits;
    rin.stride = logit_stride;
    rin.expert_scale = expert_scale;
    return moe_run(c, m, x, t, sel, reinterpret_cast<const float*>(sel + t * k), k, y, static_cast<hipStream_t>(stream), add != 0, rin);
}

int oxhip_moe_forward(oxhip_ctx* c, const float* x, size_t t, size_t h, size_t inter, const uint32_t* route_idx, const float* route_w,
                      size_t k, oxhip_moe* m, float* y) {
    if (!c || !m || !x || !route_idx || !route_w || !y || !t || !k || h != m->h || inter != m->inter) {
        set_error("moe: bad arguments");
        return 0;
    }
    for (size_t i = 0; i < t * k; i++)
        if (route_idx[i] >= m->n_exp) {  // bad routes decline (src/cuda.rs:803-813)
            set_error("moe: route to expert " + std::to_string(route_idx[i]) + " of " + std::to_string(m->n_exp));
            return 0;
        }
    std::lock_guard<std::mutex> g(c->mu);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    hipStream_t s = c->stream;
    const size_t xb = t * h * 4, rb = t * k * 4;
    if (!c->x.grow(xb + 2 * up256(rb)) || !c->y.grow(xb)) {
        set_error("moe: device memory short");
        return 0;
    }
    uint8_t* xd = static_cast<uint8_t*>(c->x.p);
    uint32_t* ri = reinterpret_cast<uint32_t*>(xd + up256(xb));
    float* rw = reinterpret_cast<float*>(xd + up256(xb) + up256(rb));
    HIP_TRY(hipMemcpyAsync(xd, x, xb, hipMemcpyHostToDevice, s), "moe copy-in");
    HIP_TRY(hipMemcpyAsync(ri, route_idx, rb, hipMemcpyHostToDevice, s), "moe copy-in");
    HIP_TRY(hipMemcpyAsync(rw, route_w, rb, hipMemcpyHostToDevice, s), "moe copy-in");
    HIP_TRY(hipMemcpyAsync(c->y.p, y, xb, hipMemcpyHostToDevice, s), "moe copy-in");  // y is added to
    if (!moe_run(c, m, reinterpret_cast<const float*>(xd), t, ri, rw, k, static_cast<float*>(c->y.p), s)) {
        (void)hipStreamSynchronize(s);
        return 0;
    }
    std::vector<float> host(t * h);
    HIP_TRY(hipMemcpyAsync(host.data(), c->y.p, xb, hipMemcpyDeviceToHost, s), "moe copy-out");
    HIP_TRY(hipStreamSynchronize(s), "moe");
    std::memcpy(y, host.data(), xb);
    c->calls++;
    return 1;
}

// Backend::matvec_rows: y = W x, or y = silu(W x) * (U x) (silu_mul's fast_exp form), 1 <= t <= 4.
int oxhip_matvec_rows(oxhip_ctx* c, const float* x, size_t t, size_t n_in, oxhip_rows_job* jobs, size_t n_jobs) {
    if (!c || !x || !jobs || !n_jobs || t < 1 || t > 4 || n_in % 32) {
        set_error("matvec_rows: bad arguments (1 <= t <= 4)");
        return 0;
    }
    size_t y_total = 0;
    bool any_q = false;
    for (size_t j = 0; j < n_jobs; j++) {
        const oxhip_rows_job& jb = jobs[j];
        if (!jb.w || !jb.y || jb.w->v.n_in != n_in || jb.w->v.n_out != jb.n_out ||
            (jb.up && (jb.up->v.n_in != n_in || jb.up->v.n_out != jb.n_out))) {
            set_error("matvec_rows: job " + std::to_string(j) + " does not match its weights");
            return 0;
        }
        y_total += t * jb.n_out * (jb.up ? 2 : 1);
        any_q |= !is_dense(jb.w) || (jb.up && !is_dense(jb.up));
    }
    std::lock_guard<std::mutex> g(c->mu);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    hipStream_t s = c->stream;
    if (!c->x.grow(t * n_in * 4) || !c->y.grow(y_total * 4) || (any_q && !c->xq.grow(qact_bytes(t, n_in)))) {
        set_error("matvec_rows: device memory short");
        return 0;
    }
    HIP_TRY(hipMemcpyAsync(c->x.p, x, t * n_in * 4, hipMemcpyHostToDevice, s), "matvec_rows copy-in");
    oxhip_qact xa{};
    if (any_q) {
        xa = carve_qact(c->xq.p, t, n_in);
        HIP_TRY(launch_quantize_act(static_cast<const float*>(c->x.p), t, n_in, xa, s), "quantize_act launch");
    }
    float* yd = static_cast<float*>(c->y.p);
    size_t off = 0;
    std::vector<size_t> at(n_jobs);
    // The jobs the matrix-core decode kernel takes share ONE launch (they all read the same x): a plain job as it is, a
    // gate / up job as a pair whose workgroups hold the tiles of the same rows of both matrices and store silu(W x) * (U x)
    // themselves (src/cuda_decode.cu:131-167). The others launch one by one, a pair as two products and the gate.
    std::vector<DecodeBatchItem> fused;
    for (size_t j = 0; j < n_jobs; j++) {
        const oxhip_rows_job& jb = jobs[j];
        const size_t n = t * jb.n_out;
        at[j] = off;
        const bool pairable = !jb.up || (jb.up->v.fmt == jb.w->v.fmt && decode_pair_ok(jb.w->v));
        if (pairable && !is_dense(jb.w) && decode_batchable(jb.w->v, t)) {
            Epi e;
            if (jb.up) e.pair_p0 = jb.up->v.p0;
            fused.push_back(DecodeBatchItem{jb.w->v, view_of(xa), yd + off, (uint32_t)t, e});
        } else {
            HIP_TRY(launch_decode(jb.w->v, view_of(xa), static_cast<const float*>(c->x.p), t, yd + off, s, c->dec), "decode launch");
            if (jb.up) {
                HIP_TRY(launch_decode(jb.up->v, view_of(xa), static_cast<const float*>(c->x.p), t, yd + off + n, s, c->dec), "decode launch");
                HIP_TRY(launch_moe_act(yd + off, yd + off + n, jb.n_out, t, jb.n_out, OXHIP_ACT_SILU, 0.0f, yd + off, s), "act launch");
            }
        }
        off += n * (jb.up ? 2 : 1);
    }
    if (!fused.empty()) {
        hipError_t e = launch_decode_mfma_batch(fused.data(), fused.size(), c->dec, s);
        if (e == hipErrorOutOfMemory) {  // the scratch does not hold these jobs' K slices together: one launch each
            for (auto& it : fused) HIP_TRY(launch_decode_mfma(it.w, it.xa, t, it.y, c->dec, s, nullptr, nullptr, it.epi), "decode launch");
        } else {
            HIP_TRY(e, "decode batch launch");
        }
    }
    std::vector<float> host(y_total);
    HIP_TRY(hipMemcpyAsync(host.data(), yd, y_total * 4, hipMemcpyDeviceToHost, s), "matvec_rows copy-out");
    HIP_TRY(hipStreamSynchronize(s), "matvec_rows");
    for (size_t j = 0; j < n_jobs; j++) std::memcpy(jobs[j].y, host.data() + at[j], t * jobs[j].n_out * 4);
    c->calls++;
    return 1;
}

}  // extern "C"
