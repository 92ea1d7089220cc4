// CPU oracle for the quantized-weight matmul path: TEST INFRASTRUCTURE ONLY (see oxref.h).
//
// Every function restates the algorithm of the cited reference lines (paths relative to the
// reference tree). Build with -ffp-contract=off: the reference never fuses a multiply with an
// add unless it writes an explicit fused multiply-add, and neither does this file.
#include "oxref.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#if defined(__AVX2__)
#include <immintrin.h>
#endif

namespace {

inline float bits_f32(uint32_t b) {
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}
inline uint32_t f32_bits(float f) {
    uint32_t b;
    std::memcpy(&b, &f, 4);
    return b;
}
inline uint16_t u16at(const uint8_t* b, size_t i) { return (uint16_t)(b[i] | (b[i + 1] << 8)); }
inline uint32_t u32at(const uint8_t* b, size_t i) {
    return (uint32_t)b[i] | ((uint32_t)b[i + 1] << 8) | ((uint32_t)b[i + 2] << 16) | ((uint32_t)b[i + 3] << 24);
}
inline float f16at(const uint8_t* b, size_t i) { return oxref_f16_to_f32(u16at(b, i)); }

constexpr size_t QBLOCK = 32;  // src/quant.rs: activation / Q8 / Q4 block
constexpr size_t QK_K = 256;   // src/ggml.rs:36

// ---------------------------------------------------------------------------------------------
// A small persistent pool for the timed CPU baseline (the reference uses a spin pool,
// src/pool.rs; only its scheduling shape matters here, not its code).
// ---------------------------------------------------------------------------------------------
class Pool {
   public:
    explicit Pool(int n) : n_(n) {
        for (int i = 1; i < n_; i++) th_.emplace_back([this] { worker(); });
    }
    ~Pool() {
        {
            std::lock_guard<std::mutex> g(m_);
            stop_ = true;
            gen_++;
        }
        cv_.notify_all();
        for (auto& t : th_) t.join();
    }
    int threads() const { return n_; }
    void run(size_t jobs, const std::function<void(size_t)>& f) {
        if (jobs == 0) return;
        if (n_ == 1 || jobs == 1) {
            for (size_t i = 0; i < jobs; i++) f(i);
            return;
        }
        {
            std::lock_guard<std::mutex> g(m_);
            f_ = &f;
            jobs_ = jobs;
            next_.store(0);
            active_ = n_ - 1;
            gen_++;
        }
        cv_.notify_all();
        drain();
        std::unique_lock<std::mutex> g(m_);
        done_.wait(g, [this] { return active_ == 0; });
        f_ = nullptr;
    }

   private:
    void drain() {
        for (;;) {
            size_t i = next_.fetch_add(1);
            if (i >= jobs_) break;
            (*f_)(i);
        }
    }
    void worker() {
        uint64_t seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> g(m_);
                cv_.wait(g, [&] { return gen_ != seen; });
                seen = gen_;
                if (stop_) return;
            }
            drain();
            {
                std::lock_guard<std::mutex> g(m_);
                active_--;
            }
            done_.notify_one();
        }
    }
    int n_;
    std::vector<std::thread> th_;
    std::mutex m_;
    std::condition_variable cv_, done_;
    const std::function<void(size_t)>* f_ = nullptr;
    size_t jobs_ = 0;
    std::atomic<size_t> next_{0};
    int active_ = 0;
    uint64_t gen_ = 0;
    bool stop_ = false;
};

Pool& pool(int threads) {
    static std::mutex m;
    static std::vector<Pool*> pools;
    std::lock_guard<std::mutex> g(m);
    if (threads < 1) threads = 1;
    for (auto* p : pools)
        if (p->threads() == threads) return *p;
    pools.push_back(new Pool(threads));
    return *pools.back();
}

// Row blocks of matmul_quant_multi_at (src/kernels.rs:1753-1771): about total/(8*threads) bytes,
// at least 128 KiB, in multiples of 16 rows.
size_t rows_per_block(size_t total_bytes, size_t n_out, int threads) {
    size_t bytes_per_row = std::max<size_t>(total_bytes / n_out, 1);
    size_t target = std::max<size_t>(total_bytes / ((size_t)threads * 8), 128 * 1024);
    return std::max<size_t>(target / bytes_per_row, 16) / 16 * 16;
}

// Rust's `iter().sum::<f32>()`: a sequential sum from -0.0 (the neutral element since Rust 1.83).
inline float seq_sum(const float* v, size_t n) {
    float s = -0.0f;
    for (size_t i = 0; i < n; i++) s += v[i];
    return s;
}

struct QActBuf {
    std::vector<int8_t> q;
    std::vector<float> scales, fsums, hsums;
    std::vector<int32_t> sums;
    size_t t, n_in;
    QActBuf(const float* x, size_t t_, size_t n) : t(t_), n_in(n) {
        q.resize(t * n);
        scales.resize(t * n / 32);
        sums.resize(t * n / 32);
        fsums.resize(t * n / 32);
        hsums.resize(t * n / 16);
        oxref_quantize_act(x, t, n, q.data(), scales.data(), sums.data(), fsums.data(), hsums.data());
    }
};

// src/ggml.rs:503-509
inline void scale_min_k4(size_t j, const uint8_t* q, uint8_t* sc, uint8_t* mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

}  // namespace

// The public functions take C linkage from their declarations in oxref.h.

int oxref_hw_threads(void) {
    unsigned n = std::thread::hardware_concurrency();
    return n ? (int)n : 1;
}

// ---------------------------------------------------------------------------------------------
// half 2.7.1 conversions (call sites src/quant.rs:449-455, :580-583, src/ggml.rs:1442-1444).
// ---------------------------------------------------------------------------------------------
float oxref_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FF;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        // subnormal: m * 2^-24, exact in f32
        float v = (float)m * bits_f32(0x33800000u);  // 2^-24
        return bits_f32(f32_bits(v) | sign);
    }
    if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13) | (m ? 0x00400000u : 0));
    return bits_f32(sign | ((e + 112) << 23) | (m << 13));
}

uint16_t oxref_f32_to_f16(float x) {
    uint32_t b = f32_bits(x);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    uint32_t e = (b >> 23) & 0xFF, m = b & 0x7FFFFF;
    if (e == 255) return (uint16_t)(sign | 0x7C00 | (m ? (0x0200 | (m >> 13)) : 0));
    int32_t ue = (int32_t)e - 127;
    if (ue > 15) return (uint16_t)(sign | 0x7C00);
    if (ue >= -14) {
        uint32_t he = (uint32_t)(ue + 15), hm = m >> 13, rest = m & 0x1FFF;
        uint32_t v = (he << 10) | hm;
        if (rest > 0x1000 || (rest == 0x1000 && (hm & 1))) v++;  // carries into the exponent correctly
        return (uint16_t)(sign | v);
    }
    if (ue < -25) return sign;  // below half the smallest subnormal
    // subnormal result: value = (1.m) * 2^ue, units of 2^-24
    uint32_t full = m | 0x800000;       // 24 bits, value = full * 2^(ue-23)
    int shift = -ue - 1;                // full * 2^(ue-23) / 2^-24 = full >> (-(ue+1)) ; shift in 14..24
    uint32_t hm = full >> shift;
    uint32_t rest = full & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rest > halfway || (rest == halfway && (hm & 1))) hm++;
    return (uint16_t)(sign | hm);
}

uint16_t oxref_f32_to_bf16(float x) {
    uint32_t b = f32_bits(x);
    if ((b & 0x7FFFFFFF) > 0x7F800000) return (uint16_t)((b >> 16) | 0x0040);  // quiet NaN
    uint32_t round = 0x7FFF + ((b >> 16) & 1);
    return (uint16_t)((b + round) >> 16);
}

float oxref_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }  // src/kernels.rs:16-18

// ---------------------------------------------------------------------------------------------
// Type geometry (src/ggml.rs:173-229)
// ---------------------------------------------------------------------------------------------
size_t oxref_block_size(uint32_t kind) {
    switch (kind) {
        case OXREF_F32: case OXREF_F16: case OXREF_BF16: case OXREF_F8E4M3: return 1;
        case OXREF_Q4_0: case OXREF_Q4_1: case OXREF_Q5_0: case OXREF_Q5_1: case OXREF_Q8_0: case OXREF_MXFP4: return 32;
        case OXREF_Q2_K: case OXREF_Q4_K: case OXREF_Q5_K: case OXREF_Q6_K: return QK_K;
        case OXREF_NVFP4: return 64;
        default: return 0;
    }
}
size_t oxref_type_size(uint32_t kind) {
    switch (kind) {
        case OXREF_F32: return 4;
        case OXREF_F16: case OXREF_BF16: return 2;
        case OXREF_F8E4M3: return 1;
        case OXREF_Q4_0: return 18;
        case OXREF_Q4_1: return 20;
        case OXREF_Q5_0: return 22;
        case OXREF_Q5_1: return 24;
        case OXREF_Q8_0: return 34;
        case OXREF_Q2_K: return 84;
        case OXREF_Q4_K: return 144;
        case OXREF_Q5_K: return 176;
        case OXREF_Q6_K: return 210;
        case OXREF_MXFP4: return 17;
        case OXREF_NVFP4: return 36;
        default: return 0;
    }
}
size_t oxref_row_bytes(uint32_t kind, size_t n) {
    size_t bs = oxref_block_size(kind);
    return bs ? n / bs * oxref_type_size(kind) : 0;
}

// ---------------------------------------------------------------------------------------------
// Fixtures (src/ggml.rs:1437-1496) and the hash of REF_HASHES (src/ggml.rs:1525-1533)
// ---------------------------------------------------------------------------------------------
uint64_t oxref_lcg(uint64_t* seed) {
    *seed = *seed * 6364136223846793005ULL + 1442695040888963407ULL;
    return *seed >> 33;
}

static float rnd_scale(uint64_t* seed, bool is_signed) {
    uint64_t e = 117 + oxref_lcg(seed) % 6;
    uint32_t mant = (uint32_t)oxref_lcg(seed) & 0x7FFFFF;
    float mag = bits_f32((uint32_t)(e << 23) | mant);
    if (is_signed && (oxref_lcg(seed) & 1) == 1) return -mag;
    return mag;
}
static void put_f16(uint8_t* b, size_t i, float v) {
    uint16_t h = oxref_f32_to_f16(v);
    b[i] = (uint8_t)h;
    b[i + 1] = (uint8_t)(h >> 8);
}

void oxref_random_blocks(uint32_t kind, size_t nb, uint64_t* seed, uint8_t* out) {
    size_t ts = oxref_type_size(kind);
    for (size_t i = 0; i < nb * ts; i++) out[i] = (uint8_t)oxref_lcg(seed);
    for (size_t k = 0; k < nb; k++) {
        uint8_t* b = out + k * ts;
        switch (kind) {
            case OXREF_F32: {
                float x = rnd_scale(seed, true) * 64.0f;
                std::memcpy(b, &x, 4);
                break;
            }
            case OXREF_F16: put_f16(b, 0, rnd_scale(seed, true) * 64.0f); break;
            case OXREF_BF16: {
                uint16_t h = oxref_f32_to_bf16(rnd_scale(seed, true) * 64.0f);
                b[0] = (uint8_t)h;
                b[1] = (uint8_t)(h >> 8);
                break;
            }
            case OXREF_Q4_1: case OXREF_Q5_1:
                put_f16(b, 0, rnd_scale(seed, false));
                put_f16(b, 2, rnd_scale(seed, true) * 8.0f);
                break;
            case OXREF_Q2_K:
                put_f16(b, 80, rnd_scale(seed, false));
                put_f16(b, 82, rnd_scale(seed, false));
                break;
            case OXREF_Q4_K: case OXREF_Q5_K:
                put_f16(b, 0, rnd_scale(seed, false));
                put_f16(b, 2, rnd_scale(seed, false));
                break;
            case OXREF_Q6_K: put_f16(b, 208, rnd_scale(seed, true)); break;
            case OXREF_MXFP4: b[0] = (uint8_t)(118 + oxref_lcg(seed) % 7); break;  // src/ggml.rs:1491
            default: put_f16(b, 0, rnd_scale(seed, true)); break;
        }
    }
}

uint64_t oxref_fnv1a_f32(const float* v, size_t n) {
    uint64_t h = 0xcbf29ce484222325ULL;
    for (size_t i = 0; i < n; i++) {
        uint32_t b = f32_bits(v[i]);
        for (int k = 0; k < 4; k++) h = (h ^ ((b >> (8 * k)) & 0xFF)) * 0x100000001b3ULL;
    }
    return h;
}

// MXFP4: E2M1 values stored doubled (src/ggml_tables.rs:1896) and half the value of the block's E8M0 scale byte,
// 2^(e - 128) (src/ggml.rs:466-475: the two smallest codes are subnormal f32 values).
static const int8_t KVALUES_MXFP4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
static float e8m0_half(uint8_t e) { return e < 2 ? bits_f32(0x00200000u << e) : bits_f32(((uint32_t)e - 1) << 23); }
// NVFP4: half the value of an unsigned E4M3 scale byte (src/ggml.rs:477-490): bits 3..6 the exponent (bias 7), bits 0..2
// the mantissa, subnormals m 2^-9; 0 and 0x7f decode to 0; bit 7 is not looked at.
float oxref_ue4m3_half(uint8_t x) {
    if (x == 0 || x == 0x7F) return 0.0f;
    int e = (x >> 3) & 0xF;
    float m = (float)(x & 7);
    float raw = e == 0 ? m * std::ldexp(1.0f, -9) : (1.0f + m / 8.0f) * std::ldexp(1.0f, e - 7);
    return raw * 0.5f;
}

// ---------------------------------------------------------------------------------------------
// dequantize_row (src/ggml.rs:630-793; MXFP4 :922-928)
// ---------------------------------------------------------------------------------------------
void oxref_dequantize_row(uint32_t kind, const uint8_t* src, size_t n, float* out) {
    switch (kind) {
        case OXREF_F32:
            for (size_t i = 0; i < n; i++) out[i] = bits_f32(u32at(src, 4 * i));
            return;
        case OXREF_F16:
            for (size_t i = 0; i < n; i++) out[i] = f16at(src, 2 * i);
            return;
        case OXREF_BF16:
            for (size_t i = 0; i < n; i++) out[i] = oxref_bf16_to_f32(u16at(src, 2 * i));
            return;
        case OXREF_F8E4M3:  // unscaled: the block scales belong to the matrix (src/ggml.rs:661-667)
            for (size_t i = 0; i < n; i++) out[i] = oxref_e4m3_to_f32(src[i]);
            return;
        default: break;
    }
    size_t bs = oxref_block_size(kind), ts = oxref_type_size(kind);
    for (size_t bi = 0; bi < n / bs; bi++) {
        const uint8_t* b = src + bi * ts;
        float* y = out + bi * bs;
        switch (kind) {
            case OXREF_Q4_0: {
                float d = f16at(b, 0);
                for (int j = 0; j < 16; j++) {
                    y[j] = (float)((int)(b[2 + j] & 0xF) - 8) * d;
                    y[j + 16] = (float)((int)(b[2 + j] >> 4) - 8) * d;
                }
                break;
            }
            case OXREF_MXFP4: {
                float d = e8m0_half(b[0]);
                for (int j = 0; j < 16; j++) {
                    y[j] = d * (float)KVALUES_MXFP4[b[1 + j] & 0xF];
                    y[j + 16] = d * (float)KVALUES_MXFP4[b[1 + j] >> 4];
                }
                break;
            }
            case OXREF_NVFP4: {  // src/ggml.rs:936-947: four sub-blocks of 16, scale byte s, then 8 bytes: elements j (low) and j + 8 (high)
                for (int sb = 0; sb < 4; sb++) {
                    float d = oxref_ue4m3_half(b[sb]);
                    const uint8_t* q = b + 4 + 8 * sb;
                    for (int j = 0; j < 8; j++) {
                        y[16 * sb + j] = d * (float)KVALUES_MXFP4[q[j] & 0xF];
                        y[16 * sb + j + 8] = d * (float)KVALUES_MXFP4[q[j] >> 4];
                    }
                }
                break;
            }
            case OXREF_Q4_1: {
                float d = f16at(b, 0), m = f16at(b, 2);
                for (int j = 0; j < 16; j++) {
                    y[j] = (float)(b[4 + j] & 0xF) * d + m;
                    y[j + 16] = (float)(b[4 + j] >> 4) * d + m;
                }
                break;
            }
            case OXREF_Q5_0: {
                float d = f16at(b, 0);
                uint32_t qh = u32at(b, 2);
                for (int j = 0; j < 16; j++) {
                    uint8_t h0 = (uint8_t)(((qh >> j) << 4) & 0x10);
                    uint8_t h1 = (uint8_t)((qh >> (j + 12)) & 0x10);
                    y[j] = (float)((int)((b[6 + j] & 0xF) | h0) - 16) * d;
                    y[j + 16] = (float)((int)((b[6 + j] >> 4) | h1) - 16) * d;
                }
                break;
            }
            case OXREF_Q5_1: {
                float d = f16at(b, 0), m = f16at(b, 2);
                uint32_t qh = u32at(b, 4);
                for (int j = 0; j < 16; j++) {
                    uint8_t h0 = (uint8_t)(((qh >> j) << 4) & 0x10);
                    uint8_t h1 = (uint8_t)((qh >> (j + 12)) & 0x10);
                    y[j] = (float)((b[8 + j] & 0xF) | h0) * d + m;
                    y[j + 16] = (float)((b[8 + j] >> 4) | h1) * d + m;
                }
                break;
            }
            case OXREF_Q8_0: {
                float d = f16at(b, 0);
                for (int j = 0; j < 32; j++) y[j] = (float)(int8_t)b[2 + j] * d;
                break;
            }
            case OXREF_Q2_K: {
                float d = f16at(b, 80), mn = f16at(b, 82);
                const uint8_t *sc = b, *qs = b + 16;
                for (int n2 = 0; n2 < 2; n2++) {
                    const uint8_t* q = qs + 32 * n2;
                    for (int j = 0; j < 4; j++)
                        for (int h = 0; h < 2; h++) {
                            uint8_t s = sc[8 * n2 + 2 * j + h];
                            float dl = d * (float)(s & 0xF), ml = mn * (float)(s >> 4);
                            float* o = y + 128 * n2 + 32 * j + 16 * h;
                            for (int l = 0; l < 16; l++) o[l] = dl * (float)((q[16 * h + l] >> (2 * j)) & 3) - ml;
                        }
                }
                break;
            }
            case OXREF_Q4_K: case OXREF_Q5_K: {
                float d = f16at(b, 0), mn = f16at(b, 2);
                const uint8_t* sc = b + 4;
                bool five = kind == OXREF_Q5_K;
                const uint8_t* qh = b + 16;
                const uint8_t* qs = five ? b + 48 : b + 16;
                for (int j = 0; j < 4; j++) {
                    const uint8_t* q = qs + 32 * j;
                    for (int h = 0; h < 2; h++) {
                        uint8_t s, m;
                        scale_min_k4(2 * j + h, sc, &s, &m);
                        float d1 = d * (float)s, m1 = mn * (float)m;
                        float* o = y + 64 * j + 32 * h;
                        for (int l = 0; l < 32; l++) {
                            uint8_t v = (q[l] >> (4 * h)) & 0xF;
                            if (five && (qh[l] & (1 << (2 * j + h)))) v += 16;
                            o[l] = d1 * (float)v - m1;
                        }
                    }
                }
                break;
            }
            case OXREF_Q6_K: {
                float d = f16at(b, 208);
                for (int n2 = 0; n2 < 2; n2++) {
                    const uint8_t* ql = b + 64 * n2;
                    const uint8_t* qh = b + 128 + 32 * n2;
                    const uint8_t* sc = b + 192 + 8 * n2;
                    float* o = y + 128 * n2;
                    for (int l = 0; l < 32; l++) {
                        int is = l / 16;
                        int q1 = (int)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32;
                        int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                        int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                        int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                        o[l] = d * (float)(int8_t)sc[is] * (float)q1;
                        o[l + 32] = d * (float)(int8_t)sc[is + 2] * (float)q2;
                        o[l + 64] = d * (float)(int8_t)sc[is + 4] * (float)q3;
                        o[l + 96] = d * (float)(int8_t)sc[is + 6] * (float)q4;
                    }
                }
                break;
            }
            default: break;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// decode_i8 (src/ggml.rs:967-1091): block -> int8 q, per-16 scale s and offset m.
// ---------------------------------------------------------------------------------------------
int oxref_decode_i8(uint32_t kind, const uint8_t* b, int8_t* q, float* s, float* m) {
    switch (kind) {
        case OXREF_Q4_0: case OXREF_Q4_1: case OXREF_Q5_0: case OXREF_Q5_1: {
            float d = f16at(b, 0);
            const uint8_t* qs;
            uint32_t qh = 0;
            int off;
            if (kind == OXREF_Q4_0) { qs = b + 2; off = 8; }
            else if (kind == OXREF_Q4_1) { qs = b + 4; off = 0; }
            else if (kind == OXREF_Q5_0) { qs = b + 6; qh = u32at(b, 2); off = 16; }
            else { qs = b + 8; qh = u32at(b, 4); off = 0; }
            for (int j = 0; j < 16; j++) {
                uint8_t h0 = (uint8_t)(((qh >> j) << 4) & 0x10);
                uint8_t h1 = (uint8_t)((qh >> (j + 12)) & 0x10);
                uint8_t lo = (qs[j] & 0xF) | h0, hi = (qs[j] >> 4) | h1;
                q[j] = (int8_t)((int)lo - off);
                q[j + 16] = (int8_t)((int)hi - off);
            }
            s[0] = s[1] = d;
            if (kind == OXREF_Q4_1 || kind == OXREF_Q5_1) {
                int c = kind == OXREF_Q4_1 ? 8 : 16;
                for (int i = 0; i < 32; i++) q[i] = (int8_t)(q[i] - c);
                m[0] = m[1] = f16at(b, 2) + d * (float)c;
                return 1;
            }
            return 0;
        }
        case OXREF_Q8_0:
            for (int j = 0; j < 32; j++) q[j] = (int8_t)b[2 + j];
            s[0] = s[1] = f16at(b, 0);
            return 0;
        case OXREF_MXFP4:  // src/ggml.rs:1209-1216
            s[0] = s[1] = e8m0_half(b[0]);
            for (int j = 0; j < 16; j++) {
                q[j] = KVALUES_MXFP4[b[1 + j] & 0xF];
                q[j + 16] = KVALUES_MXFP4[b[1 + j] >> 4];
            }
            return 0;
        case OXREF_Q2_K: {
            float d = f16at(b, 80), mn = f16at(b, 82);
            for (int n = 0; n < 2; n++)
                for (int j = 0; j < 4; j++)
                    for (int h = 0; h < 2; h++) {
                        int g = 8 * n + 2 * j + h;
                        s[g] = d * (float)(b[g] & 0xF);
                        m[g] = 2.0f * s[g] - mn * (float)(b[g] >> 4);
                        for (int l = 0; l < 16; l++)
                            q[16 * g + l] = (int8_t)(((b[16 + 32 * n + 16 * h + l] >> (2 * j)) & 3) - 2);
                    }
            return 1;
        }
        case OXREF_Q4_K: case OXREF_Q5_K: {
            float d = f16at(b, 0), mn = f16at(b, 2);
            bool five = kind == OXREF_Q5_K;
            const uint8_t* qh = b + 16;
            const uint8_t* qs = five ? b + 48 : b + 16;
            int off = five ? 16 : 8;
            for (int j = 0; j < 4; j++)
                for (int h = 0; h < 2; h++) {
                    uint8_t sc, mv;
                    scale_min_k4(2 * j + h, b + 4, &sc, &mv);
                    int g = 2 * (2 * j + h);
                    s[g] = d * (float)sc;
                    s[g + 1] = s[g];
                    m[g] = (float)off * s[g] - mn * (float)mv;
                    m[g + 1] = m[g];
                    for (int l = 0; l < 32; l++) {
                        uint8_t v = (qs[32 * j + l] >> (4 * h)) & 0xF;
                        if (five && (qh[l] & (1 << (2 * j + h)))) v += 16;
                        q[64 * j + 32 * h + l] = (int8_t)((int)v - off);
                    }
                }
            return 1;
        }
        case OXREF_Q6_K: {
            float d = f16at(b, 208);
            for (int g = 0; g < 16; g++) s[g] = d * (float)(int8_t)b[192 + g];
            for (int n = 0; n < 2; n++) {
                const uint8_t* ql = b + 64 * n;
                const uint8_t* qh = b + 128 + 32 * n;
                int8_t* o = q + 128 * n;
                for (int l = 0; l < 32; l++) {
                    o[l] = (int8_t)((int)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
                    o[l + 32] = (int8_t)((int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
                    o[l + 64] = (int8_t)((int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
                    o[l + 96] = (int8_t)((int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
                }
            }
            return 0;
        }
        default: return -1;
    }
}

// ---------------------------------------------------------------------------------------------
// FP8 E4M3 (src/ggml.rs:259-293, :433-444)
// ---------------------------------------------------------------------------------------------
float oxref_e4m3_to_f32(uint8_t b) {
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int e = (b >> 3) & 0xF, m = b & 7;
    if (e == 0xF && m == 7) return std::nanf("");
    float v = e == 0 ? (float)m / 8.0f * std::ldexp(1.0f, -6) : (1.0f + (float)m / 8.0f) * std::ldexp(1.0f, e - 7);
    return sign * v;
}

void oxref_e4m3_scaled(const uint8_t* src, size_t n, float s, float* out) {
    for (size_t i = 0; i < n; i++) {
        uint32_t b = src[i];
        uint32_t e = (b >> 3) & 0xF, m = b & 7;
        uint32_t normal = ((e + 120) << 23) | (m << 20);
        uint32_t subnormal = f32_bits((float)(int32_t)m * (1.0f / 512.0f));
        uint32_t mag = e == 0 ? subnormal : normal;
        if ((b & 0x7F) == 0x7F) mag = 0x7FC00000u;
        out[i] = bits_f32(mag | ((b & 0x80) << 24)) * s;
    }
}

void oxref_fp8_dequant_rows(const uint8_t* data, const float* scales, size_t n_out, size_t n_in,
                            size_t brows, size_t bcols, size_t r0, size_t r1, float* out) {
    (void)n_out;
    size_t ncb = (n_in + bcols - 1) / bcols;
    for (size_t r = r0; r < r1; r++) {
        const float* srow = scales + (r / brows) * ncb;
        for (size_t cb = 0; cb < ncb; cb++) {
            size_t c0 = cb * bcols, len = std::min(bcols, n_in - c0);
            oxref_e4m3_scaled(data + r * n_in + c0, len, srow[cb], out + (r - r0) * n_in + c0);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Activation quantization (src/quant.rs:243-343, the non-aarch64 arm)
// ---------------------------------------------------------------------------------------------
void oxref_quantize_act(const float* x, size_t t, size_t n_in, int8_t* q, float* scales,
                        int32_t* sums, float* fsums, float* hsums) {
    size_t bpr = n_in / QBLOCK;
    for (size_t r = 0; r < t; r++)
        for (size_t b = 0; b < bpr; b++) {
            const float* blk = x + r * n_in + b * QBLOCK;
            int8_t* qo = q + r * n_in + b * QBLOCK;
            float amax = 0.0f;
            for (size_t i = 0; i < QBLOCK; i++) amax = std::fmax(amax, std::fabs(blk[i]));
            float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
            int32_t s = 0;
            for (size_t i = 0; i < QBLOCK; i++) {
                float v = std::round(blk[i] * inv);  // half away from zero
                int32_t iv = std::isnan(v) ? 0 : (v >= 127.0f ? 127 : (v <= -128.0f ? -128 : (int32_t)v));
                qo[i] = (int8_t)iv;
                s += iv;
            }
            size_t bi = r * bpr + b;
            scales[bi] = amax / 127.0f;
            sums[bi] = s;
            hsums[2 * bi] = seq_sum(blk, 16);
            hsums[2 * bi + 1] = seq_sum(blk + 16, 16);
            fsums[bi] = seq_sum(blk, 32);
        }
}

// ---------------------------------------------------------------------------------------------
// MLX affine 4-bit -> Q4 layout with offsets (src/quant.rs:518-606)
// ---------------------------------------------------------------------------------------------
void oxref_from_mlx_q4(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       size_t n_out, size_t n_in, size_t group, uint8_t* q, uint16_t* sc, uint16_t* off) {
    size_t gpr = n_in / group, bpr = n_in / QBLOCK;
    for (size_t r = 0; r < n_out; r++) {
        const uint32_t* wrow = w + r * n_in / 8;
        for (size_t g = 0; g < gpr; g++) {
            float s = oxref_bf16_to_f32(scales[r * gpr + g]);
            float b = oxref_bf16_to_f32(biases[r * gpr + g]);
            off[r * gpr + g] = oxref_f32_to_bf16(b + 8.0f * s);
            uint16_t d = oxref_f32_to_f16(s);
            for (size_t blk = g * group / QBLOCK; blk < (g + 1) * group / QBLOCK; blk++) sc[r * bpr + blk] = d;
        }
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint32_t* words = wrow + blk * 4;
            auto nib = [&](size_t e) { return (uint8_t)((words[e / 8] >> (4 * (e % 8))) & 15); };
            for (size_t j = 0; j < 16; j++) q[r * n_in / 2 + blk * 16 + j] = (uint8_t)(nib(j) | (nib(j + 16) << 4));
        }
    }
}

void oxref_mlx_dequant_row(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           size_t bits, size_t group, size_t n, float* out) {
    size_t per = 32 / bits;
    uint32_t mask = (1u << bits) - 1;
    for (size_t e = 0; e < n; e++) {
        size_t g = e / group;
        float s = oxref_bf16_to_f32(scales[g]), b = oxref_bf16_to_f32(biases[g]);
        uint32_t qv = (w[e / per] >> (bits * (e % per))) & mask;
        out[e] = s * (float)qv + b;
    }
}

void oxref_dequant_rows_q4(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                           size_t n_in, size_t r0, size_t r1, float* out) {
    size_t bpr = n_in / QBLOCK;
    for (size_t r = r0; r < r1; r++) {
        const uint8_t* qrow = q + r * n_in / 2;
        float* orow = out + (r - r0) * n_in;
        for (size_t b = 0; b < bpr; b++) {
            float d = oxref_f16_to_f32(sc[r * bpr + b]);
            float m = off ? oxref_bf16_to_f32(off[r * (n_in / group) + b * QBLOCK / group]) : 0.0f;
            for (size_t j = 0; j < 16; j++) {
                uint8_t byte = qrow[b * 16 + j];
                orow[b * QBLOCK + j] = (float)((int)(byte & 0x0F) - 8) * d + m;
                orow[b * QBLOCK + j + 16] = (float)((int)(byte >> 4) - 8) * d + m;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Q4 decode, scalar definition (src/kernels_x86.rs:447-474) + add_offsets (src/kernels.rs:1287-1297)
// with dot_bf16's 8-lane form (src/kernels.rs:2060-2073).
// ---------------------------------------------------------------------------------------------
static float dot_bf16_lanes(const uint16_t* w, const float* x, size_t n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t chunks = n / 8;
    for (size_t c = 0; c < chunks; c++)
        for (int i = 0; i < 8; i++) acc[i] += oxref_bf16_to_f32(w[8 * c + i]) * x[8 * c + i];
    float s = seq_sum(acc, 8);
    for (size_t i = chunks * 8; i < n; i++) s += oxref_bf16_to_f32(w[i]) * x[i];
    return s;
}

static void q4_group_sums(const QActBuf& xa, size_t c, size_t group, std::vector<float>& gs) {
    size_t bpr = xa.n_in / QBLOCK, k = group / QBLOCK, gpr = xa.n_in / group;
    gs.resize(gpr);
    for (size_t g = 0; g < gpr; g++) gs[g] = seq_sum(&xa.fsums[c * bpr + g * k], k);
}

void oxref_q4_decode(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                     size_t n_out, size_t n_in, const float* x, size_t t, float* y, int32_t* isums) {
    QActBuf xa(x, t, n_in);
    size_t bpr = n_in / QBLOCK, half_row = n_in / 2;
    std::vector<float> gs;
    for (size_t c = 0; c < t; c++) {
        if (off) q4_group_sums(xa, c, group, gs);
        for (size_t r = 0; r < n_out; r++) {
            float acc = 0.0f;
            for (size_t b = 0; b < bpr; b++) {
                const uint8_t* blk = q + r * half_row + b * 16;
                const int8_t* xq = &xa.q[c * n_in + b * 32];
                int32_t sum = 0;
                for (int j = 0; j < 16; j++) {
                    uint8_t v = blk[j];
                    sum += ((int)(v & 15) - 8) * (int)xq[j];
                    sum += ((int)(v >> 4) - 8) * (int)xq[j + 16];
                }
                if (isums) isums[(c * n_out + r) * bpr + b] = sum;
                acc += (float)sum * oxref_f16_to_f32(sc[r * bpr + b]) * xa.scales[c * bpr + b];
            }
            if (off) acc += dot_bf16_lanes(off + r * (n_in / group), gs.data(), n_in / group);
            y[c * n_out + r] = acc;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Q8 (QMatrix: int8 codes, one f32 scale per block of 32)
// ---------------------------------------------------------------------------------------------
// dequantize_rows (src/quant.rs:405-419): q as f32 * scale.
void oxref_q8_dequant_rows(const int8_t* q, const float* scales, size_t n_in, size_t r0, size_t r1, float* out) {
    size_t bpr = n_in / QBLOCK;
    for (size_t r = r0; r < r1; r++)
        for (size_t b = 0; b < bpr; b++)
            for (size_t j = 0; j < QBLOCK; j++) out[(r - r0) * n_in + b * QBLOCK + j] = (float)q[r * n_in + b * QBLOCK + j] * scales[r * bpr + b];
}

// QMat::rows_t1 for QMatrix, portable branch (src/kernels.rs:1156-1167): per block the exact int32 dot, then
// acc += s as f32 * scale_b * xs_b, blocks in order; every token on its own (rows_tc's portable branch, :1207-1212).
void oxref_q8_decode(const int8_t* q, const float* scales, size_t n_out, size_t n_in, const float* x, size_t t, float* y, int32_t* isums) {
    QActBuf xa(x, t, n_in);
    size_t bpr = n_in / QBLOCK;
    for (size_t c = 0; c < t; c++)
        for (size_t r = 0; r < n_out; r++) {
            float acc = 0.0f;
            for (size_t b = 0; b < bpr; b++) {
                int32_t sum = 0;
                for (size_t j = 0; j < QBLOCK; j++) sum += (int32_t)q[r * n_in + b * QBLOCK + j] * (int32_t)xa.q[c * n_in + b * QBLOCK + j];
                if (isums) isums[(c * n_out + r) * bpr + b] = sum;
                acc += (float)sum * scales[r * bpr + b] * xa.scales[c * bpr + b];
            }
            y[c * n_out + r] = acc;
        }
}

// ---------------------------------------------------------------------------------------------
// GGUF decode, portable definition (src/ggml.rs:1288-1315)
// ---------------------------------------------------------------------------------------------
static void gguf_dot_row(uint32_t kind, const uint8_t* row, size_t n_in, const QActBuf& xa, size_t c0,
                         size_t tc, float* acc, int32_t* isums, size_t isum_stride) {
    size_t bs = oxref_block_size(kind), ts = oxref_type_size(kind);
    int8_t q[QK_K];
    float s[16], m[16];
    for (size_t c = 0; c < tc; c++) acc[c] = 0.0f;
    for (size_t bi = 0; bi < n_in / bs; bi++) {
        int has_min = oxref_decode_i8(kind, row + bi * ts, q, s, m);
        size_t e0 = bi * bs;
        for (size_t c = 0; c < tc; c++) {
            const int8_t* xq = &xa.q[(c0 + c) * n_in + e0];
            const float* xs = &xa.scales[(c0 + c) * n_in / QBLOCK + e0 / QBLOCK];
            float sum = 0.0f;
            for (size_t g = 0; g < bs / 16; g++) {
                int32_t isum = 0;
                for (int i = 0; i < 16; i++) isum += (int32_t)q[16 * g + i] * (int32_t)xq[16 * g + i];
                if (isums) isums[c * isum_stride + e0 / 16 + g] = isum;
                sum += s[g] * xs[g / 2] * (float)isum;
            }
            if (has_min) {
                const float* xh = &xa.hsums[(c0 + c) * n_in / 16 + e0 / 16];
                for (size_t g = 0; g < bs / 16; g++) sum += m[g] * xh[g];
            }
            acc[c] += sum;
        }
    }
}

void oxref_gguf_decode(uint32_t kind, const uint8_t* data, size_t n_out, size_t n_in,
                       const float* x, size_t t, float* y, int32_t* isums) {
    QActBuf xa(x, t, n_in);
    size_t rb = oxref_row_bytes(kind, n_in);
    std::vector<float> acc(t);
    for (size_t r = 0; r < n_out; r++) {
        gguf_dot_row(kind, data + r * rb, n_in, xa, 0, t, acc.data(), isums ? isums + r * (n_in / 16) : nullptr,
                     n_out * (n_in / 16));
        for (size_t c = 0; c < t; c++) y[c * n_out + r] = acc[c];
    }
}

// ---------------------------------------------------------------------------------------------
// AVX2 forms that the CPU baseline times (src/kernels_x86.rs:476-536, src/kernels_ggml_x86.rs:120-431)
// ---------------------------------------------------------------------------------------------
#if defined(__AVX2__)
static inline float hsum256(__m256 v) {  // src/kernels_x86.rs:96-103
    __m128 lo = _mm256_castps256_ps128(v), hi = _mm256_extractf128_ps(v, 1);
    __m128 s = _mm_add_ps(lo, hi);
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ss(s, _mm_shuffle_ps(s, s, 1));
    return _mm_cvtss_f32(s);
}
static inline float f16c(uint16_t h) { return _mm_cvtss_f32(_mm_cvtph_ps(_mm_cvtsi32_si128(h))); }

// R rows x TC tokens, unsigned nibbles with the -8 folded through the activation block sums.
template <int R, int TC>
static void q4_dot_rows_avx2(const uint8_t* q, const uint16_t* s, size_t n_in, const int8_t* xq,
                             const float* xs, const int32_t* xsums, float out[R][TC]) {
    size_t bpr = n_in / 32, half_row = n_in / 2;
    const __m256i ones = _mm256_set1_epi16(1);
    const __m128i m0f = _mm_set1_epi8(0x0F);
    __m256 accf[R][TC];
    float corr[R][TC];
    for (int r = 0; r < R; r++)
        for (int c = 0; c < TC; c++) {
            accf[r][c] = _mm256_setzero_ps();
            corr[r][c] = 0.0f;
        }
    for (size_t b = 0; b < bpr; b++) {
        __m256i xv[TC];
        for (int c = 0; c < TC; c++) xv[c] = _mm256_loadu_si256((const __m256i*)(xq + c * n_in + b * 32));
        for (int r = 0; r < R; r++) {
            __m128i bytes = _mm_loadu_si128((const __m128i*)(q + r * half_row + b * 16));
            __m128i lo = _mm_and_si128(bytes, m0f);
            __m128i hi = _mm_and_si128(_mm_srli_epi16(bytes, 4), m0f);
            __m256i wv = _mm256_set_m128i(hi, lo);
            float d = f16c(s[r * bpr + b]);
            for (int c = 0; c < TC; c++) {
                __m256i p16 = _mm256_maddubs_epi16(wv, xv[c]);
                __m256i p32 = _mm256_madd_epi16(p16, ones);
                float scv = d * xs[c * bpr + b];
                accf[r][c] = _mm256_fmadd_ps(_mm256_cvtepi32_ps(p32), _mm256_set1_ps(scv), accf[r][c]);
                corr[r][c] += scv * (float)xsums[c * bpr + b];
            }
        }
    }
    for (int r = 0; r < R; r++)
        for (int c = 0; c < TC; c++) out[r][c] = hsum256(accf[r][c]) - 8.0f * corr[r][c];
}

template <int TC>
static void q4_rows_avx2(const uint8_t* q, const uint16_t* sc, size_t n_out, size_t n_in, const QActBuf& xa,
                         size_t c0, float* y, size_t r0, size_t r1) {
    size_t bpr = n_in / 32;
    const int8_t* xq = &xa.q[c0 * n_in];
    const float* xs = &xa.scales[c0 * bpr];
    const int32_t* xsums = &xa.sums[c0 * bpr];
    size_t r = r0;
    for (; r + 2 <= r1; r += 2) {
        float o[2][TC];
        q4_dot_rows_avx2<2, TC>(q + r * n_in / 2, sc + r * bpr, n_in, xq, xs, xsums, o);
        for (int rr = 0; rr < 2; rr++)
            for (int c = 0; c < TC; c++) y[(c0 + c) * n_out + r + rr] = o[rr][c];
    }
    if (r < r1) {
        float o[1][TC];
        q4_dot_rows_avx2<1, TC>(q + r * n_in / 2, sc + r * bpr, n_in, xq, xs, xsums, o);
        for (int c = 0; c < TC; c++) y[(c0 + c) * n_out + r] = o[0][c];
    }
}

// unpack (src/kernels_ggml_x86.rs:120-261): decode_i8 with the int8 values formed in registers.
static inline __m256i nibbles256(const uint8_t* p) {
    __m128i bytes = _mm_loadu_si128((const __m128i*)p);
    __m128i m = _mm_set1_epi8(0x0F);
    return _mm256_set_m128i(_mm_and_si128(_mm_srli_epi16(bytes, 4), m), _mm_and_si128(bytes, m));
}
static inline __m256i shr_and(__m256i v, int n, int8_t mask) {
    return _mm256_and_si256(_mm256_srl_epi16(v, _mm_cvtsi32_si128(n)), _mm256_set1_epi8(mask));
}
static inline void st256(int8_t* q, size_t at, __m256i v) { _mm256_storeu_si256((__m256i*)(q + at), v); }

static int unpack_avx2(uint32_t kind, const uint8_t* b, int8_t* q, float* s, float* m) {
    switch (kind) {
        case OXREF_Q8_0:
            st256(q, 0, _mm256_loadu_si256((const __m256i*)(b + 2)));
            s[0] = s[1] = f16c(u16at(b, 0));
            return 0;
        case OXREF_Q4_0:
            st256(q, 0, _mm256_sub_epi8(nibbles256(b + 2), _mm256_set1_epi8(8)));
            s[0] = s[1] = f16c(u16at(b, 0));
            return 0;
        case OXREF_Q4_K: {
            float d = f16c(u16at(b, 0)), mn = f16c(u16at(b, 2));
            const uint8_t* qs = b + 16;
            for (int j = 0; j < 4; j++) {
                __m256i v = _mm256_loadu_si256((const __m256i*)(qs + 32 * j));
                for (int h = 0; h < 2; h++) {
                    uint8_t sc, mv;
                    scale_min_k4(2 * j + h, b + 4, &sc, &mv);
                    int g = 2 * (2 * j + h);
                    s[g] = d * (float)sc;
                    s[g + 1] = s[g];
                    m[g] = 8.0f * s[g] - mn * (float)mv;
                    m[g + 1] = m[g];
                    st256(q, 64 * j + 32 * h, _mm256_sub_epi8(shr_and(v, 4 * h, 0x0F), _mm256_set1_epi8(8)));
                }
            }
            return 1;
        }
        case OXREF_Q6_K: {
            float d = f16c(u16at(b, 208));
            for (int g = 0; g < 16; g++) s[g] = d * (float)(int8_t)b[192 + g];
            const __m256i c32 = _mm256_set1_epi8(32);
            for (int n = 0; n < 2; n++) {
                __m256i ql[2] = {_mm256_loadu_si256((const __m256i*)(b + 64 * n)),
                                 _mm256_loadu_si256((const __m256i*)(b + 64 * n + 32))};
                __m256i qh = _mm256_loadu_si256((const __m256i*)(b + 128 + 32 * n));
                for (int k = 0; k < 4; k++) {
                    __m256i lo = shr_and(ql[k % 2], 4 * (k / 2), 0x0F);
                    __m256i hi = _mm256_slli_epi16(shr_and(qh, 2 * k, 3), 4);
                    st256(q, 128 * n + 32 * k, _mm256_sub_epi8(_mm256_or_si256(lo, hi), c32));
                }
            }
            return 0;
        }
        default: return oxref_decode_i8(kind, b, q, s, m);
    }
}

static inline __m256i dot32(const int8_t* w, const int8_t* x) {  // src/kernels_ggml_x86.rs:335-340
    __m256i wv = _mm256_loadu_si256((const __m256i*)w), xv = _mm256_loadu_si256((const __m256i*)x);
    __m256i p16 = _mm256_maddubs_epi16(_mm256_sign_epi8(wv, wv), _mm256_sign_epi8(xv, wv));
    return _mm256_madd_epi16(p16, _mm256_set1_epi16(1));
}

static void products_avx2(const int8_t* q, const float* s, const int8_t* xq, const float* xs, size_t bs, float* p) {
    if (bs == QBLOCK) {
        __m256i v = dot32(q, xq);
        __m128i lo = _mm256_castsi256_si128(v), hi = _mm256_extracti128_si256(v, 1);
        __m128i t = _mm_hadd_epi32(lo, hi);
        t = _mm_hadd_epi32(t, t);
        p[0] = s[0] * xs[0] * (float)_mm_cvtsi128_si32(t);
        p[1] = s[1] * xs[0] * (float)_mm_extract_epi32(t, 1);
        return;
    }
    const __m256i order = _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7);
    const __m256i twice = _mm256_setr_epi32(0, 0, 1, 1, 2, 2, 3, 3);
    for (size_t h = 0; h < bs / 128; h++) {
        const int8_t *qh = q + 128 * h, *xh = xq + 128 * h;
        __m256i t0 = _mm256_hadd_epi32(dot32(qh, xh), dot32(qh + 32, xh + 32));
        __m256i t1 = _mm256_hadd_epi32(dot32(qh + 64, xh + 64), dot32(qh + 96, xh + 96));
        __m256i isum = _mm256_permutevar8x32_epi32(_mm256_hadd_epi32(t0, t1), order);
        __m256 sv = _mm256_loadu_ps(s + 8 * h);
        __m256 xsv = _mm256_permutevar8x32_ps(_mm256_castps128_ps256(_mm_loadu_ps(xs + 4 * h)), twice);
        __m256 pv = _mm256_mul_ps(_mm256_mul_ps(sv, xsv), _mm256_cvtepi32_ps(isum));
        _mm256_storeu_ps(p + 8 * h, pv);
    }
}

template <int TC>
static void gguf_rows_avx2(uint32_t kind, const uint8_t* data, size_t n_out, size_t n_in, const QActBuf& xa,
                           size_t c0, float* y, size_t r0, size_t r1) {
    size_t bs = oxref_block_size(kind), ts = oxref_type_size(kind), rb = oxref_row_bytes(kind, n_in);
    alignas(32) int8_t q[QK_K];
    float s[16], m[16], p[16];
    for (size_t r = r0; r < r1; r++) {
        const uint8_t* row = data + r * rb;
        float acc[TC];
        for (int c = 0; c < TC; c++) acc[c] = 0.0f;
        for (size_t bi = 0; bi < n_in / bs; bi++) {
            int has_min = unpack_avx2(kind, row + bi * ts, q, s, m);
            size_t e0 = bi * bs;
            for (int c = 0; c < TC; c++) {
                const int8_t* xq = &xa.q[(c0 + c) * n_in + e0];
                const float* xs = &xa.scales[(c0 + c) * n_in / QBLOCK + e0 / QBLOCK];
                products_avx2(q, s, xq, xs, bs, p);
                float sum = 0.0f;
                for (size_t g = 0; g < bs / 16; g++) sum += p[g];
                if (has_min) {
                    const float* xh = &xa.hsums[(c0 + c) * n_in / 16 + e0 / 16];
                    for (size_t g = 0; g < bs / 16; g++) sum += m[g] * xh[g];
                }
                acc[c] += sum;
            }
        }
        for (int c = 0; c < TC; c++) y[(c0 + c) * n_out + r] = acc[c];
    }
}
#endif  // __AVX2__

// Column groups of the x86 multi-token decode path (src/kernels.rs:1693-1705): at most 8 tokens and
// 64 KiB of int8 activations per group (2 at least), as even as possible.
static void col_groups(size_t t, size_t n_in, std::vector<std::pair<size_t, size_t>>& out) {
    size_t wmax = std::min<size_t>(std::max<size_t>(64 * 1024 / std::max<size_t>(n_in, 1), 2), 8);
    size_t n = (t + wmax - 1) / wmax;
    for (size_t g = 0; g < n; g++) out.emplace_back(g * t / n, (g + 1) * t / n);
}

void oxref_q4_decode_avx2(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                          size_t n_out, size_t n_in, const float* x, size_t t, float* y, int threads) {
#if defined(__AVX2__)
    QActBuf xa(x, t, n_in);
    size_t total = n_out * (n_in / 2 + n_in / 32 * 2 + (off ? n_in / group * 2 : 0));
    size_t rpb = rows_per_block(total, n_out, threads);
    size_t nblocks = (n_out + rpb - 1) / rpb;
    std::vector<std::vector<float>> gs(t);
    if (off)
        for (size_t c = 0; c < t; c++) q4_group_sums(xa, c, group, gs[c]);
    pool(threads).run(nblocks, [&](size_t b) {
        size_t r0 = b * rpb, r1 = std::min(n_out, r0 + rpb);
        // token pairs, as decode_rows does (src/kernels.rs:1913-1927)
        for (size_t c = 0; c < t;) {
            size_t tc = std::min<size_t>(t - c, 2);
            if (tc == 1) q4_rows_avx2<1>(q, sc, n_out, n_in, xa, c, y, r0, r1);
            else q4_rows_avx2<2>(q, sc, n_out, n_in, xa, c, y, r0, r1);
            c += tc;
        }
        if (off)
            for (size_t c = 0; c < t; c++)
                for (size_t r = r0; r < r1; r++)
                    y[c * n_out + r] += dot_bf16_lanes(off + r * (n_in / group), gs[c].data(), n_in / group);
    });
#else
    (void)threads;
    oxref_q4_decode(q, sc, off, group, n_out, n_in, x, t, y, nullptr);
#endif
}

void oxref_gguf_decode_avx2(uint32_t kind, const uint8_t* data, size_t n_out, size_t n_in,
                            const float* x, size_t t, float* y, int threads) {
#if defined(__AVX2__)
    QActBuf xa(x, t, n_in);
    size_t rb = oxref_row_bytes(kind, n_in);
    size_t rpb = rows_per_block(n_out * rb, n_out, threads);
    size_t nblocks = (n_out + rpb - 1) / rpb;
    std::vector<std::pair<size_t, size_t>> groups;
    if (t <= 2) groups.emplace_back(0, t);
    else col_groups(t, n_in, groups);
    pool(threads).run(nblocks, [&](size_t b) {
        size_t r0 = b * rpb, r1 = std::min(n_out, r0 + rpb);
        // row tiles of 64 KiB inside the block, each swept by every column group
        size_t tile = std::max<size_t>(64 * 1024 / std::max<size_t>(rb, 1), 4);
        for (size_t ta = r0; ta < r1; ta += tile) {
            size_t tb = std::min(r1, ta + tile);
            for (auto& g : groups) {
                size_t c0 = g.first;
                switch (g.second - g.first) {
                    case 1: gguf_rows_avx2<1>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 2: gguf_rows_avx2<2>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 3: gguf_rows_avx2<3>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 4: gguf_rows_avx2<4>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 5: gguf_rows_avx2<5>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 6: gguf_rows_avx2<6>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 7: gguf_rows_avx2<7>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    case 8: gguf_rows_avx2<8>(kind, data, n_out, n_in, xa, c0, y, ta, tb); break;
                    default: break;
                }
            }
        }
    });
#else
    (void)threads;
    oxref_gguf_decode(kind, data, n_out, n_in, x, t, y, nullptr);
#endif
}

// ---------------------------------------------------------------------------------------------
// Prefill on x86 (src/kernels.rs:1998-2038, :297-316; src/kernels_x86.rs:296-324): tokens packed
// in panels of 8, one fused multiply-add per k per output, k ascending.
// ---------------------------------------------------------------------------------------------
static void pack_xt(const float* x, size_t t, size_t n_in, std::vector<float>& xt) {
    size_t tiles = (t + 7) / 8;
    xt.assign(tiles * n_in * 8, 0.0f);
    for (size_t tile = 0; tile < tiles; tile++)
        for (size_t c = 0; c < 8; c++) {
            size_t tok = tile * 8 + c;
            if (tok >= t) break;
            for (size_t k = 0; k < n_in; k++) xt[tile * n_in * 8 + k * 8 + c] = x[tok * n_in + k];
        }
}

// 8 (or fewer) rows of f32 weights against one packed panel.
static void gemm_rows_panel(const float* w, size_t rows, size_t n_in, const float* xt, float* y, size_t n_out,
                            size_t rb, size_t c0, size_t c_valid) {
#if defined(__AVX2__) && defined(__FMA__)
    __m256 acc[8];
    for (size_t r = 0; r < rows; r++) acc[r] = _mm256_setzero_ps();
    for (size_t k = 0; k < n_in; k++) {
        __m256 xv = _mm256_loadu_ps(xt + k * 8);
        for (size_t r = 0; r < rows; r++) acc[r] = _mm256_fmadd_ps(_mm256_broadcast_ss(w + r * n_in + k), xv, acc[r]);
    }
    float tmp[8];
    for (size_t r = 0; r < rows; r++) {
        _mm256_storeu_ps(tmp, acc[r]);
        for (size_t c = 0; c < c_valid; c++) y[(c0 + c) * n_out + rb + r] = tmp[c];
    }
#else
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < c_valid; c++) {
            float acc = 0.0f;
            for (size_t k = 0; k < n_in; k++) acc = std::fmaf(w[r * n_in + k], xt[k * 8 + c], acc);
            y[(c0 + c) * n_out + rb + r] = acc;
        }
#endif
}

void oxref_gemm_f32(const float* w, size_t n_out, size_t n_in, const float* x, size_t t, float* y, int threads) {
    std::vector<float> xt;
    pack_xt(x, t, n_in, xt);
    size_t tiles = (t + 7) / 8, rblocks = (n_out + 7) / 8;
    pool(threads).run(rblocks, [&](size_t rbk) {
        size_t r = rbk * 8, rows = std::min<size_t>(8, n_out - r);
        for (size_t tile = 0; tile < tiles; tile++)
            gemm_rows_panel(w + r * n_in, rows, n_in, xt.data() + tile * n_in * 8, y, n_out, r, tile * 8,
                            std::min<size_t>(8, t - tile * 8));
    });
}

// GgufMatrix::dequantize_rows for a block format that carries scales on top of what its kind decodes (NVFP4's global
// scale; src/ggml.rs:420-432): dequantize_row, then every run of `bcols` columns times s[(r / brows) * ncb + c / bcols].
void oxref_gguf_dequant_rows_scaled(uint32_t kind, const uint8_t* data, const float* scales, size_t n_in, size_t brows, size_t bcols,
                                    size_t r0, size_t r1, float* out) {
    size_t rb = oxref_row_bytes(kind, n_in), ncb = scales ? (n_in + bcols - 1) / bcols : 0;
    for (size_t r = r0; r < r1; r++) {
        float* o = out + (r - r0) * n_in;
        oxref_dequantize_row(kind, data + r * rb, n_in, o);
        if (!scales) continue;
        for (size_t c = 0; c < n_in; c++) o[c] *= scales[(r / brows) * ncb + c / bcols];
    }
}

void oxref_gemm_quant(int64_t kind, const void* data, const void* aux0, const void* aux1, size_t group,
                      size_t brows, size_t bcols, size_t n_out, size_t n_in, const float* x, size_t t,
                      float* y, int threads) {
    std::vector<float> xt;
    pack_xt(x, t, n_in, xt);
    size_t tiles = (t + 7) / 8;
    size_t row_bytes = kind == -1 ? n_in / 2 + n_in / 32 * 2 + (aux1 ? n_in / group * 2 : 0)
                                  : (kind == OXREF_F8E4M3 ? n_in : oxref_row_bytes((uint32_t)kind, n_in));
    size_t rpb = rows_per_block(n_out * row_bytes, n_out, threads);
    size_t nblocks = (n_out + rpb - 1) / rpb;
    pool(threads).run(nblocks, [&](size_t b) {
        std::vector<float> scratch(8 * n_in);
        size_t r0 = b * rpb, r1 = std::min(n_out, r0 + rpb);
        for (size_t r = r0; r < r1; r += 8) {
            size_t rows = std::min<size_t>(8, r1 - r);
            if (kind == -1)
                oxref_dequant_rows_q4((const uint8_t*)data, (const uint16_t*)aux0, (const uint16_t*)aux1, group, n_in,
                                      r, r + rows, scratch.data());
            else if (kind == OXREF_F8E4M3)
                oxref_fp8_dequant_rows((const uint8_t*)data, (const float*)aux0, n_out, n_in, brows, bcols, r, r + rows,
                                       scratch.data());
            else if (kind == OXREF_NVFP4)  // float-stored (is_float, src/ggml.rs:219-224), its global scale in aux0 (may be null)
                oxref_gguf_dequant_rows_scaled((uint32_t)kind, (const uint8_t*)data, (const float*)aux0, n_in, brows, bcols, r, r + rows,
                                               scratch.data());
            else
                for (size_t i = 0; i < rows; i++)
                    oxref_dequantize_row((uint32_t)kind, (const uint8_t*)data + (r + i) * row_bytes, n_in,
                                         scratch.data() + i * n_in);
            for (size_t tile = 0; tile < tiles; tile++)
                gemm_rows_panel(scratch.data(), rows, n_in, xt.data() + tile * n_in * 8, y, n_out, r, tile * 8,
                                std::min<size_t>(8, t - tile * 8));
        }
    });
}

// ---------------------------------------------------------------------------------------------
// int8 prefill GEMM semantics, one activation plane (src/kernels_i8gemm.rs:160-315, with the Q4 row
// unpacking of src/kernels.rs:1304-1329): per block of 32, acc = fma(f32(I), ds*xs, acc), then
// acc -= mn*f with mn = -offset.  The block sum f is only fixed to ~1 ulp by the reference (NEON
// pairwise adds); this restatement adds four interleaved lanes then reduces them pairwise.
// ---------------------------------------------------------------------------------------------
void oxref_i8gemm_q4(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                     size_t n_out, size_t n_in, const float* x, size_t t, float* y, int32_t* isums) {
    size_t nb = n_in / QBLOCK;
    std::vector<int8_t> xq(t * n_in);
    std::vector<float> xs(t * nb), xf(t * nb);
    for (size_t c = 0; c < t; c++)
        for (size_t b = 0; b < nb; b++) {
            const float* src = x + c * n_in + 32 * b;
            float lanes[4] = {0, 0, 0, 0}, amax = 0.0f;
            for (int i = 0; i < 8; i++)
                for (int l = 0; l < 4; l++) {
                    amax = std::fmax(amax, std::fabs(src[4 * i + l]));
                    lanes[l] = lanes[l] + src[4 * i + l];
                }
            float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
            for (int i = 0; i < 32; i++) {
                float v = std::round(src[i] * inv);
                xq[c * n_in + 32 * b + i] = (int8_t)(v >= 127.0f ? 127 : (v <= -128.0f ? -128 : (int)v));
            }
            xs[c * nb + b] = amax / 127.0f;
            xf[c * nb + b] = (lanes[0] + lanes[1]) + (lanes[2] + lanes[3]);
        }
    for (size_t c = 0; c < t; c++)
        for (size_t r = 0; r < n_out; r++) {
            float acc = 0.0f;
            for (size_t b = 0; b < nb; b++) {
                const uint8_t* blk = q + r * n_in / 2 + b * 16;
                const int8_t* xb = &xq[c * n_in + 32 * b];
                int32_t I = 0;
                for (int j = 0; j < 16; j++) {
                    I += ((int)(blk[j] & 15) - 8) * (int)xb[j];
                    I += ((int)(blk[j] >> 4) - 8) * (int)xb[j + 16];
                }
                if (isums) isums[(c * n_out + r) * nb + b] = I;
                float ds = oxref_f16_to_f32(sc[r * nb + b]);
                acc = std::fmaf((float)I, ds * xs[c * nb + b], acc);
                if (off) {
                    float mn = -oxref_bf16_to_f32(off[r * (n_in / group) + b * QBLOCK / group]);
                    acc = std::fmaf(-mn, xf[c * nb + b], acc);
                }
            }
            y[c * n_out + r] = acc;
        }
}

// ---------------------------------------------------------------------------------------------
// Elementwise + routing (src/kernels.rs:2188-2231, src/moe.rs:39-42, :180-193)
// ---------------------------------------------------------------------------------------------
float oxref_fast_exp(float x) {
    x = std::fmin(std::fmax(x, -87.0f), 88.0f);
    float fx = std::round(x * 1.44269504088896340736f);
    float r = (x - fx * 0.693359375f) - fx * -2.12194440e-4f;
    float p = 1.0f + r * (1.0f + r * (0.5f + r * (0.16666667f + r * (0.041666668f + r * (0.008333334f + r * 0.0013888889f)))));
    return bits_f32((uint32_t)(((int32_t)fx + 127) << 23)) * p;
}

void oxref_silu_mul(float* a, const float* b, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float x = a[i];
        a[i] = x / (1.0f + oxref_fast_exp(-x)) * b[i];
    }
}

void oxref_route_top_k(const float* logits, size_t n, size_t k, uint32_t* idx, float* w) {
    std::vector<uint32_t> order(n);
    for (size_t i = 0; i < n; i++) order[i] = (uint32_t)i;
    // total_cmp order on the logits, descending, ties to the lower index
    auto key = [&](uint32_t i) {
        int32_t b = (int32_t)f32_bits(logits[i]);
        return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
    };
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
        int32_t ka = key(a), kb = key(b);
        return ka != kb ? ka > kb : a < b;
    });
    k = std::min(k, n);
    float m = logits[order[0]];
    std::vector<float> e(k);
    for (size_t i = 0; i < k; i++) e[i] = std::exp(logits[order[i]] - m);
    float s = seq_sum(e.data(), k);
    for (size_t i = 0; i < k; i++) {
        idx[i] = order[i];
        w[i] = e[i] / s;
    }
}

// ---------------------------------------------------------------------------------------------
// MoE over repacked MLX-4bit experts (src/moe.rs:438-617 decode path; :735-827 grouped path).
// Every row is independent in both paths (activations are quantized per row, padding rows are
// zero), so the result of the batched / grouped schedules equals running each (token, route) pair
// on its own, which is what this does; the combine is an unfused y += w * o in route order.
// ---------------------------------------------------------------------------------------------
// Act::apply (src/moe.rs:18-37) of n pairs in place: kind 0 SiLU (silu_mul), 1 GELU-tanh (gelu_mul, gelu_tanh
// src/kernels.rs:2233-2239: both through fast_exp), 2 SiLU with DeepSeek V4's clamp `param` (gate min, up clamp, then
// silu_mul).
void oxref_act_apply(uint32_t kind, float param, float* g, const float* u, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float x = g[i], b = u[i];
        if (kind == 1) {
            const float K2 = 2.0f * 0.7978846f;
            float t = K2 * (x + 0.044715f * x * x * x);
            g[i] = x / (1.0f + oxref_fast_exp(-t)) * b;
            continue;
        }
        if (kind == 2) {
            x = std::fmin(x, param);
            b = std::fmin(std::fmax(b, -param), param);
        }
        g[i] = x / (1.0f + oxref_fast_exp(-x)) * b;
    }
}

// Act::scalar (src/moe.rs:39-46), what the grouped prefill path applies: libm's exp for the SiLU kinds, gelu_tanh
// (fast_exp) for GELU.
float oxref_act_scalar(uint32_t kind, float param, float g, float u) {
    if (kind == 1) {
        const float K2 = 2.0f * 0.7978846f;
        float t = K2 * (g + 0.044715f * g * g * g);
        return g / (1.0f + oxref_fast_exp(-t)) * u;
    }
    if (kind == 2) {
        g = std::fmin(g, param);
        u = std::fmin(std::fmax(u, -param), param);
    }
    return g / (1.0f + std::exp(-g)) * u;
}

// `up` == nullptr: gate_up[e] is the fused [2 inter, h] matrix (gate rows, then up rows); else gate_up[e] is the gate
// [inter, h] and up[e] the up projection [inter, h] (src/gpu.rs:206-216).
void oxref_moe_q4_act(const oxref_q4_ref* gate_up, const oxref_q4_ref* up, const oxref_q4_ref* down, size_t ne, size_t group,
                      size_t h, size_t inter, const float* x, size_t t, const uint32_t* route_idx,
                      const float* route_w, size_t k, float* y, int decode_path, uint32_t act_kind, float act_param) {
    int threads = oxref_hw_threads();
    // expert -> (token, slot) pairs
    std::vector<std::vector<std::pair<size_t, size_t>>> by(ne);
    for (size_t ti = 0; ti < t; ti++)
        for (size_t j = 0; j < k; j++) by[route_idx[ti * k + j]].emplace_back(ti, j);
    std::vector<float> outs(t * k * h);
    pool(threads).run(ne, [&](size_t e) {
        size_t n = by[e].size();
        if (!n) return;
        std::vector<float> xs(n * h), g(n * inter), u(n * inter), a(n * inter), o(n * h);
        for (size_t i = 0; i < n; i++) std::memcpy(&xs[i * h], x + by[e][i].first * h, h * 4);
        // the gate and up products as [n][inter] each
        auto split = [&](const std::vector<float>& gu) {
            for (size_t i = 0; i < n; i++) {
                std::memcpy(&g[i * inter], &gu[i * 2 * inter], inter * 4);
                std::memcpy(&u[i * inter], &gu[i * 2 * inter + inter], inter * 4);
            }
        };
        if (decode_path) {
            if (!up) {
                std::vector<float> gu(n * 2 * inter);
                oxref_q4_decode(gate_up[e].q, gate_up[e].sc, gate_up[e].off, group, 2 * inter, h, xs.data(), n, gu.data(), nullptr);
                split(gu);
            } else {
                oxref_q4_decode(gate_up[e].q, gate_up[e].sc, gate_up[e].off, group, inter, h, xs.data(), n, g.data(), nullptr);
                oxref_q4_decode(up[e].q, up[e].sc, up[e].off, group, inter, h, xs.data(), n, u.data(), nullptr);
            }
            oxref_act_apply(act_kind, act_param, g.data(), u.data(), n * inter);
            a = g;
            oxref_q4_decode(down[e].q, down[e].sc, down[e].off, group, h, inter, a.data(), n, o.data(), nullptr);
        } else {
            const size_t gr = up ? inter : 2 * inter;
            std::vector<float> wf(gr * h);
            oxref_dequant_rows_q4(gate_up[e].q, gate_up[e].sc, gate_up[e].off, group, h, 0, gr, wf.data());
            if (!up) {
                std::vector<float> gu(n * 2 * inter);
                oxref_gemm_f32(wf.data(), 2 * inter, h, xs.data(), n, gu.data(), 1);
                split(gu);
            } else {
                oxref_gemm_f32(wf.data(), inter, h, xs.data(), n, g.data(), 1);
                oxref_dequant_rows_q4(up[e].q, up[e].sc, up[e].off, group, h, 0, inter, wf.data());
                oxref_gemm_f32(wf.data(), inter, h, xs.data(), n, u.data(), 1);
            }
            for (size_t i = 0; i < n * inter; i++) a[i] = oxref_act_scalar(act_kind, act_param, g[i], u[i]);
            wf.resize(h * inter);
            oxref_dequant_rows_q4(down[e].q, down[e].sc, down[e].off, group, inter, 0, h, wf.data());
            oxref_gemm_f32(wf.data(), h, inter, a.data(), n, o.data(), 1);
        }
        for (size_t i = 0; i < n; i++)
            std::memcpy(&outs[(by[e][i].first * k + by[e][i].second) * h], &o[i * h], h * 4);
    });
    for (size_t ti = 0; ti < t; ti++)
        for (size_t j = 0; j < k; j++) {
            float w = route_w[ti * k + j];
            const float* o = &outs[(ti * k + j) * h];
            for (size_t i = 0; i < h; i++) y[ti * h + i] += w * o[i];
        }
}

void oxref_moe_q4(const oxref_q4_ref* gate_up, const oxref_q4_ref* down, size_t ne, size_t group,
                  size_t h, size_t inter, const float* x, size_t t, const uint32_t* route_idx,
                  const float* route_w, size_t k, float* y, int decode_path) {
    oxref_moe_q4_act(gate_up, nullptr, down, ne, group, h, inter, x, t, route_idx, route_w, k, y, decode_path, 0, 0.0f);
}

// The decode-sized MoE pass as the x86 CPU schedules it, for the timed baseline (values as oxref_moe_q4's decode
// path up to the AVX2 kernels' f32 order): activations quantized once per expert's rows, every expert's matmul cut
// into row blocks of one shared parallel region (matmul_quant_batch, src/kernels.rs:1937-1994), the AVX2 decode
// kernels per block (src/kernels_x86.rs:476-519), silu_mul (src/kernels.rs:2188-2198), requantize, down, combine in
// route order (src/moe.rs:608-615).
void oxref_moe_q4_avx2(const oxref_q4_ref* gate_up, const oxref_q4_ref* down, size_t ne, size_t group,
                       size_t h, size_t inter, const float* x, size_t t, const uint32_t* route_idx,
                       const float* route_w, size_t k, float* y, int threads) {
#if defined(__AVX2__)
    std::vector<std::vector<std::pair<size_t, size_t>>> by(ne);
    for (size_t ti = 0; ti < t; ti++)
        for (size_t j = 0; j < k; j++) by[route_idx[ti * k + j]].emplace_back(ti, j);
    std::vector<size_t> used;
    for (size_t e = 0; e < ne; e++)
        if (!by[e].empty()) used.push_back(e);
    struct Job {
        size_t e, n;
        std::vector<float> xs, gu, a, o;
        std::unique_ptr<QActBuf> xa, aq;
        std::vector<std::vector<float>> gs;
    };
    std::vector<Job> jobs(used.size());
    for (size_t u = 0; u < used.size(); u++) {
        Job& jb = jobs[u];
        jb.e = used[u];
        jb.n = by[jb.e].size();
        jb.xs.resize(jb.n * h);
        for (size_t i = 0; i < jb.n; i++) std::memcpy(&jb.xs[i * h], x + by[jb.e][i].first * h, h * 4);
        jb.xa.reset(new QActBuf(jb.xs.data(), jb.n, h));
        jb.gu.resize(jb.n * 2 * inter);
        jb.a.resize(jb.n * inter);
        jb.o.resize(jb.n * h);
    }
    struct Block {
        size_t u, r0, r1;
    };
    auto run_phase = [&](bool second) {
        const size_t n_out = second ? h : 2 * inter, n_in = second ? inter : h;
        const size_t bytes_per_row = n_in / 2 + n_in / 32 * 2 + n_in / group * 2;
        const size_t rpb = rows_per_block(jobs.size() * n_out * bytes_per_row, jobs.size() * n_out, threads);
        std::vector<Block> blocks;
        for (size_t u = 0; u < jobs.size(); u++) {
            Job& jb = jobs[u];
            const QActBuf& xa = second ? *jb.aq : *jb.xa;
            jb.gs.assign(jb.n, std::vector<float>());
            for (size_t c = 0; c < jb.n; c++) q4_group_sums(xa, c, group, jb.gs[c]);
            for (size_t r = 0; r < n_out; r += rpb) blocks.push_back(Block{u, r, std::min(n_out, r + rpb)});
        }
        pool(threads).run(blocks.size(), [&](size_t b) {
            const Block& bl = blocks[b];
            Job& jb = jobs[bl.u];
            const oxref_q4_ref& w = second ? down[jb.e] : gate_up[jb.e];
            const QActBuf& xa = second ? *jb.aq : *jb.xa;
            float* out = second ? jb.o.data() : jb.gu.data();
            for (size_t c = 0; c < jb.n;) {
                size_t tc = std::min<size_t>(jb.n - c, 2);
                if (tc == 1) q4_rows_avx2<1>(w.q, w.sc, n_out, n_in, xa, c, out, bl.r0, bl.r1);
                else q4_rows_avx2<2>(w.q, w.sc, n_out, n_in, xa, c, out, bl.r0, bl.r1);
                c += tc;
            }
            if (w.off)
                for (size_t c = 0; c < jb.n; c++)
                    for (size_t r = bl.r0; r < bl.r1; r++)
                        out[c * n_out + r] += dot_bf16_lanes(w.off + r * (n_in / group), jb.gs[c].data(), n_in / group);
        });
    };
    run_phase(false);
    pool(threads).run(jobs.size(), [&](size_t u) {
        Job& jb = jobs[u];
        for (size_t i = 0; i < jb.n; i++) {
            float* g = &jb.gu[i * 2 * inter];
            oxref_silu_mul(g, g + inter, inter);
            std::memcpy(&jb.a[i * inter], g, inter * 4);
        }
        jb.aq.reset(new QActBuf(jb.a.data(), jb.n, inter));
    });
    run_phase(true);
    for (size_t ti = 0; ti < t; ti++)
        for (size_t j = 0; j < k; j++) {
            const size_t e = route_idx[ti * k + j];
            size_t u = std::lower_bound(used.begin(), used.end(), e) - used.begin();
            size_t i = 0;
            while (by[e][i] != std::make_pair(ti, j)) i++;
            const float w = route_w[ti * k + j];
            const float* o = &jobs[u].o[i * h];
            for (size_t c = 0; c < h; c++) y[ti * h + c] += w * o[c];
        }
#else
    (void)threads;
    oxref_moe_q4(gate_up, down, ne, group, h, inter, x, t, route_idx, route_w, k, y, 1);
#endif
}

