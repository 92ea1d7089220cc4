// The C ABI: the device context, uploads, and the `Backend` surface (src/gpu.rs:151-294 of the
// reference) over the kernels of this library.
#include "backend.hpp"

#include <vector>

namespace oxhip {

static thread_local std::string g_err;
void set_error(const std::string& m) { g_err = m; }

}  // namespace oxhip

using namespace oxhip;

// Scratch of the allocation-free decode entry point (oxhip_dev_decode_noalloc): partial rows of the K slices, then
// their arrival counters. Every GPU the library runs on holds its own copy of this array until the process ends.
constexpr size_t NOALLOC_PARTIAL_FLOATS = (size_t)1 << 20;       // 4 MiB
constexpr size_t NOALLOC_COUNTERS = (size_t)2048 * CTR_STRIDE;   // 2048 row groups, a 128-byte line each: 256 KiB
static __device__ __align__(256) unsigned char scratch[NOALLOC_PARTIAL_FLOATS * 4 + NOALLOC_COUNTERS * 4];
// The array's address on each device (the name above is only a host-side stand-in for it), looked up by oxhip_open.
constexpr int NOALLOC_MAX_DEVICES = 64;
static void* g_scratch_ptr[NOALLOC_MAX_DEVICES];
static std::mutex g_scratch_mu;

__global__ void fill_zero_kernel(uint32_t* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

namespace oxhip {
// Clears n dwords with a kernel on `s` (not a memset: memset nodes captured into a graph have replayed wrongly, and a
// memset on the null stream waits for the whole device).
hipError_t launch_fill_zero(uint32_t* p, size_t n, hipStream_t s) {
    if (!n) return hipSuccess;
    fill_zero_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p, n);
    return hipGetLastError();
}
}  // namespace oxhip

namespace {

struct Planes {
    size_t off[4] = {0, 0, 0, 0};
    size_t total = 0;
    void add(int i, size_t bytes) {
        off[i] = total;
        total = align_up(total + bytes, 256);
    }
};

bool have_memory(size_t bytes) {
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return false;
    return free_b >= bytes + VRAM_RESERVE;
}

void bind(oxhip_weight* w, const Planes& pl, int nplanes) {
    const uint8_t* b = static_cast<const uint8_t*>(w->base);
    const uint8_t** dst[4] = {&w->v.p0, &w->v.p1, &w->v.p2, &w->v.p3};
    for (int i = 0; i < nplanes; i++) *dst[i] = b + pl.off[i];
}

// Uploads host bytes into a temporary device buffer.
struct Temp {
    void* p = nullptr;
    ~Temp() {
        if (p) (void)hipFree(p);
    }
    bool put(const void* src, size_t bytes, hipStream_t s) {
        if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) return false;
        return hipMemcpyAsync(p, src, bytes, hipMemcpyHostToDevice, s) == hipSuccess;
    }
};

}  // namespace

extern "C" {

const char* oxhip_last_error(void) { return g_err.c_str(); }

int oxhip_probe(oxhip_gpu_info* out, int cap) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();  // no driver or no device: not an error of the caller's
        return 0;
    }
    int rt = 0;
    (void)hipRuntimeGetVersion(&rt);
    for (int d = 0; d < n && out && d < cap; d++) {
        oxhip_gpu_info& g = out[d];
        std::memset(&g, 0, sizeof g);
        g.index = d;
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, d) != hipSuccess) continue;
        std::snprintf(g.name, sizeof g.name, "%s", prop.name);
        std::string arch = prop.gcnArchName;
        arch = arch.substr(0, arch.find(':'));
        std::snprintf(g.arch, sizeof g.arch, "%s", arch.c_str());
        g.memory_bytes = prop.totalGlobalMem;
        std::snprintf(g.driver, sizeof g.driver, "HIP runtime %d.%d, %s, %d CUs", rt / 10000000, (rt / 100000) % 100, arch.c_str(),
                      prop.multiProcessorCount);
        g.usable = arch == "gfx950";
    }
    return n;
}

int oxhip_open(int device, oxhip_ctx** out) {
    if (!out) return 0;
    *out = nullptr;
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n), "hipGetDeviceCount");
    if (device < 0 || device >= n) {
        set_error("device " + std::to_string(device) + ": not available (" + std::to_string(n) + " HIP devices)");
        return 0;
    }
    HIP_TRY(hipSetDevice(device), "hipSetDevice");
    if (device < NOALLOC_MAX_DEVICES) {  // once per device, with that device current
        std::lock_guard<std::mutex> g(g_scratch_mu);
        if (!g_scratch_ptr[device]) {
            void* ptr = nullptr;
            HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
            g_scratch_ptr[device] = ptr;
        }
    }
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    std::string arch = prop.gcnArchName;
    arch = arch.substr(0, arch.find(':'));
    if (arch != "gfx950") {
        set_error("device " + std::to_string(device) + " is " + arch + ": this library holds gfx950 code only");
        return 0;
    }
    auto* c = new oxhip_ctx();
    c->device = device;
    c->name = "hip (" + arch + ")";
    // 16 MiB of partial rows (32 slices x 8 tokens x 16384 outputs) and 16384 counters (a line each), zero between launches
    c->dec.partial_floats = (size_t)4 << 20;
    c->dec.ncounters = (size_t)16384 * CTR_STRIDE;
    if (hipMalloc(reinterpret_cast<void**>(&c->dec.partial), c->dec.partial_floats * 4) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&c->dec.counters), c->dec.ncounters * 4) != hipSuccess ||
        hipMemset(c->dec.counters, 0, c->dec.ncounters * 4) != hipSuccess) {
        set_error("decode scratch allocation failed");
        if (c->dec.partial) (void)hipFree(c->dec.partial);
        if (c->dec.counters) (void)hipFree(c->dec.counters);
        delete c;
        return 0;
    }
    if (hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) != hipSuccess) {
        set_error("hipStreamCreate failed");
        (void)hipFree(c->dec.partial);
        (void)hipFree(c->dec.counters);
        delete c;
        return 0;
    }
    *out = c;
    return 1;
}

void oxhip_close(oxhip_ctx* c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    (void)hipStreamSynchronize(c->stream);
    c->x.release();
    c->xq.release();
    c->y.release();
    c->gemm_ws.release();
    free_stream_scratch(c);
    (void)hipFree(c->dec.partial);
    (void)hipFree(c->dec.counters);
    (void)hipStreamDestroy(c->stream);
    delete c;
}

const char* oxhip_name(const oxhip_ctx* c) { return c ? c->name.c_str() : ""; }

size_t oxhip_stats(oxhip_ctx* c, char* buf, size_t len) {
    if (!c || !buf || !len) return 0;
    std::lock_guard<std::mutex> g(c->mu);
    int n = snprintf(buf, len, "hip: %zu calls, copy-in %.2f ms, gpu %.2f ms, copy-out %.2f ms", c->calls, c->ms_in, c->ms_gpu,
                     c->ms_out);
    return n < 0 ? 0 : ((size_t)n < len ? (size_t)n : len - 1);
}

// The device reads weights at several TB/s and a launch costs a few microseconds, so unlike the
// reference's PCIe-attached policy (t >= 32, 1 GFLOP) any whole-block shape is worth taking; the
// activations still cross the host link on this surface, which is what bounds small calls.
int oxhip_wants(const oxhip_ctx* c, size_t n_out, size_t n_in, size_t t) {
    if (!c || !t || !n_out) return 0;
    return n_in % 32 == 0 && n_in >= 32;
}

size_t oxhip_weight_bytes(const oxhip_weight* w) { return w ? w->bytes : 0; }

void oxhip_free_weight(oxhip_ctx* c, oxhip_weight* w) {
    if (!w) return;
    if (c) (void)hipSetDevice(c->device);
    if (w->base) (void)hipFree(w->base);
    delete w;
}

// `q4_0_blocks`: the planar Q4 data of this call are GGUF Q4_0 blocks split by the caller below (no offset term at all)
static oxhip_weight* upload_weight(oxhip_ctx* c, const oxhip_weight_desc* d, bool q4_0_blocks) {
    if (!c || !d || !d->data) {
        set_error("upload: null argument");
        return nullptr;
    }
    const size_t n_out = d->n_out, n_in = d->n_in;
    if (!n_out || !n_in || n_out > 0x7FFFFFFFu || n_in > 0x7FFFFFFFu) {
        set_error("upload: bad shape");
        return nullptr;
    }
    if (hipSetDevice(c->device) != hipSuccess) {
        set_error("hipSetDevice failed");
        return nullptr;
    }
    auto w = new oxhip_weight();
    w->v.n_out = (uint32_t)n_out;
    w->v.n_in = (uint32_t)n_in;
    auto fail = [&](const std::string& why) -> oxhip_weight* {
        set_error("upload: " + why);
        if (w->base) (void)hipFree(w->base);
        delete w;
        return nullptr;
    };
    auto alloc = [&](const Planes& pl, int nplanes) -> bool {
        if (!have_memory(pl.total)) return false;
        if (hipMalloc(&w->base, pl.total) != hipSuccess) {
            w->base = nullptr;
            return false;
        }
        w->bytes = pl.total;
        bind(w, pl, nplanes);
        return true;
    };
    hipStream_t s = c->stream;
    Planes pl;
    switch (d->kind) {
        case OXHIP_W_Q8: {  // QMatrix (src/quant.rs:128-133)
            if (n_in % 32 || !d->scales) return fail("Q8 needs n_in % 32 == 0 and its f32 scales");
            w->v.fmt = FMT_Q8F;
            pl.add(0, t8f_bytes((uint32_t)n_out, (uint32_t)n_in));
            if (!alloc(pl, 1)) return fail("device memory short");
            Temp q, sc;
            if (!have_memory(n_out * n_in + n_out * (n_in / 32) * 4) || !q.put(d->data, n_out * n_in, s) || !sc.put(d->scales, n_out * (n_in / 32) * 4, s))
                return fail("device memory short");
            if (launch_pack_q8f(static_cast<const int8_t*>(q.p), static_cast<const float*>(sc.p), n_out, n_in, static_cast<uint8_t*>(w->base), s) != hipSuccess)
                return fail("pack launch failed");
            if (hipStreamSynchronize(s) != hipSuccess) return fail("pack failed");
            break;
        }
        case OXHIP_W_BF16: {
            if (n_in % 8) return fail("bf16 rows must be a multiple of 8");
            w->v.fmt = FMT_BF16;
            pl.add(0, n_out * n_in * 2);
            if (!alloc(pl, 1)) return fail("device memory short");
            if (hipMemcpyAsync(w->base, d->data, n_out * n_in * 2, hipMemcpyHostToDevice, s) != hipSuccess) return fail("copy failed");
            break;
        }
        case OXHIP_W_Q4: {
            if (n_in % 32 || !d->scales) return fail("Q4 needs n_in % 32 == 0 and scales");
            size_t group = d->offsets ? d->group : 0;
            if (d->offsets && (group == 0 || group % 32 || n_in % group)) return fail("Q4 offset group must be a multiple of 32 dividing n_in");
            w->v.fmt = FMT_Q4;
            w->v.group = (uint32_t)group;
            // one scale per offset group when the blocks of a group agree (MLX), else per 32
            size_t sgroup = group ? group : 32;
            for (int attempt = 0; attempt < 2; attempt++) {
                pl = Planes();
                pl.add(0, n_out * n_in / 2);
                pl.add(1, n_out * (n_in / sgroup) * 2);
                if (group) pl.add(2, n_out * (n_in / group) * 2);
                if (!alloc(pl, group ? 3 : 2)) return fail("device memory short");
                w->v.sgroup = (uint32_t)sgroup;
                uint8_t* b = static_cast<uint8_t*>(w->base);
                if (hipMemcpyAsync(b + pl.off[0], d->data, n_out * n_in / 2, hipMemcpyHostToDevice, s) != hipSuccess) return fail("copy failed");
                if (group && hipMemcpyAsync(b + pl.off[2], d->offsets, n_out * (n_in / group) * 2, hipMemcpyHostToDevice, s) != hipSuccess)
                    return fail("copy failed");
                if (sgroup == 32) {
                    if (hipMemcpyAsync(b + pl.off[1], d->scales, n_out * (n_in / 32) * 2, hipMemcpyHostToDevice, s) != hipSuccess)
                        return fail("copy failed");
                    break;
                }
                Temp t32, flag;
                int zero = 0, mismatch = 0;
                if (!t32.put(d->scales, n_out * (n_in / 32) * 2, s) || !flag.put(&zero, sizeof zero, s)) return fail("device memory short");
                if (launch_q4_scale_groups(static_cast<const uint16_t*>(t32.p), n_out, n_in, sgroup, reinterpret_cast<uint16_t*>(b + pl.off[1]),
                                           static_cast<int*>(flag.p), s) != hipSuccess)
                    return fail("scale repack launch failed");
                if (hipMemcpyAsync(&mismatch, flag.p, sizeof mismatch, hipMemcpyDeviceToHost, s) != hipSuccess ||
                    hipStreamSynchronize(s) != hipSuccess)
                    return fail("scale repack failed");
                if (!mismatch) break;
                (void)hipFree(w->base);  // scales differ inside a group: keep one per block
                w->base = nullptr;
                sgroup = 32;
            }
            break;
        }
        case OXHIP_W_MLX_Q4: {
            size_t group = d->group;
            if (!d->scales || !d->offsets || group == 0 || group % 32 || n_in % group) return fail("MLX 4-bit needs scales, biases and a group that is a multiple of 32 dividing n_in");
            w->v.fmt = FMT_Q4;
            w->v.group = w->v.sgroup = (uint32_t)group;
            pl.add(0, n_out * n_in / 2);
            pl.add(1, n_out * (n_in / group) * 2);
            pl.add(2, n_out * (n_in / group) * 2);
            if (!alloc(pl, 3)) return fail("device memory short");
            Temp tw, ts, tb;
            if (!tw.put(d->data, n_out * n_in / 2, s) || !ts.put(d->scales, n_out * (n_in / group) * 2, s) ||
                !tb.put(d->offsets, n_out * (n_in / group) * 2, s))
                return fail("device memory short");
            if (launch_repack_mlx_q4(static_cast<const uint32_t*>(tw.p), static_cast<const uint16_t*>(ts.p), static_cast<const uint16_t*>(tb.p),
                                     n_out, n_in, group, w->v, s) != hipSuccess)
                return fail("repack launch failed");
            if (hipStreamSynchronize(s) != hipSuccess) return fail("repack failed");
            break;
        }
        case OXHIP_W_GGUF: {
            if (d->ggml_type == OXHIP_GGML_F8E4M3) {
                if (!d->block_scales || !d->bs_rows || !d->bs_cols) return fail("FP8 needs block scales");
                if (n_in % 16 || d->bs_cols % 16) return fail("FP8 rows and scale blocks must be multiples of 16 columns");
                w->v.fmt = FMT_FP8;
                w->v.br = d->bs_rows;
                w->v.bc = d->bs_cols;
                size_t ns = ((n_out + d->bs_rows - 1) / d->bs_rows) * ((n_in + d->bs_cols - 1) / d->bs_cols);
                const bool tiled = fp8_tileable(n_in, d->bs_rows, d->bs_cols);
                w->v.group = tiled ? 1 : 0;
                pl.add(0, tiled ? (size_t)row_tiles((uint32_t)n_out) * (n_in / 128) * 2048 : n_out * n_in);
                pl.add(1, ns * 4);
                if (!alloc(pl, 2)) return fail("device memory short");
                uint8_t* b = static_cast<uint8_t*>(w->base);
                if (hipMemcpyAsync(b + pl.off[1], d->block_scales, ns * 4, hipMemcpyHostToDevice, s) != hipSuccess) return fail("copy failed");
                if (tiled) {
                    Temp raw;
                    if (!raw.put(d->data, n_out * n_in, s)) return fail("device memory short");
                    if (launch_pack_fp8(static_cast<const uint8_t*>(raw.p), n_out, n_in, b + pl.off[0], s) != hipSuccess)
                        return fail("pack launch failed");
                    if (hipStreamSynchronize(s) != hipSuccess) return fail("pack failed");
                } else if (hipMemcpyAsync(b + pl.off[0], d->data, n_out * n_in, hipMemcpyHostToDevice, s) != hipSuccess) {
                    return fail("copy failed");
                }
                break;
            }
            if (d->ggml_type == OXHIP_GGML_Q4_0) {
                // Q4_0 (18 B per 32: f16 d, then 16 bytes whose byte j holds elements j and j + 16; src/ggml.rs:675-683) is
                // the Q4Matrix layout with the scale inside the block: split it into codes and scales and take that path
                if (n_in % 32) return fail("Q4_0 rows must be whole blocks of 32");
                const size_t nb = n_out * (n_in / 32);
                std::vector<uint8_t> q(nb * 16);
                std::vector<uint16_t> sc(nb);
                const uint8_t* src = static_cast<const uint8_t*>(d->data);
                for (size_t b = 0; b < nb; b++) {
                    std::memcpy(&sc[b], src + 18 * b, 2);
                    std::memcpy(&q[16 * b], src + 18 * b + 2, 16);
                }
                oxhip_weight_desc d2{};
                d2.kind = OXHIP_W_Q4;
                d2.n_out = n_out;
                d2.n_in = n_in;
                d2.data = q.data();
                d2.scales = sc.data();
                delete w;
                return upload_weight(c, &d2, true);
            }
            size_t raw_bytes;
            int np;
            if (d->ggml_type == OXHIP_GGML_NVFP4) {
                // ggml's blocks of 64 (36 B) with, optionally, the matrix's scales on top (compressed-tensors' global scale
                // as a whole-matrix block, src/model.rs:550-557; any block geometry whose blocks are whole tiles)
                if (n_in % 64) return fail("NVFP4 rows must be whole blocks of 64");
                const bool scaled = d->block_scales != nullptr;
                if (scaled && (!d->bs_rows || !d->bs_cols)) return fail("NVFP4 scales need their block geometry");
                if (scaled && !((d->bs_rows % 16 == 0 || d->bs_rows >= n_out) && (d->bs_cols % 128 == 0 || d->bs_cols >= n_in)))
                    return fail("NVFP4 scale blocks must be multiples of 16 rows x 128 columns (or span the matrix)");
                w->v.fmt = FMT_NVFP4;
                w->v.br = scaled ? d->bs_rows : 0;
                w->v.bc = scaled ? d->bs_cols : 0;
                const size_t ns = scaled ? ((n_out + d->bs_rows - 1) / d->bs_rows) * ((n_in + d->bs_cols - 1) / d->bs_cols) : 0;
                pl.add(0, t4n_bytes((uint32_t)n_out, (uint32_t)n_in));
                if (scaled) pl.add(1, ns * 4);
                if (!alloc(pl, scaled ? 2 : 1)) return fail("device memory short");
                if (scaled && hipMemcpyAsync(static_cast<uint8_t*>(w->base) + pl.off[1], d->block_scales, ns * 4, hipMemcpyHostToDevice, s) != hipSuccess)
                    return fail("copy failed");
                raw_bytes = n_out * (n_in / 64) * 36;
                Temp raw;
                if (!have_memory(raw_bytes) || !raw.put(d->data, raw_bytes, s)) return fail("device memory short");
                if (launch_repack_gguf(w->v.fmt, static_cast<const uint8_t*>(raw.p), n_out, n_in, w->v, s) != hipSuccess)
                    return fail("repack launch failed");
                if (hipStreamSynchronize(s) != hipSuccess) return fail("repack failed");
                break;
            }
            if (d->ggml_type == OXHIP_GGML_Q8_0) {
                if (n_in % 32) return fail("Q8_0 rows must be whole blocks of 32");
                w->v.fmt = FMT_Q8_0;
                pl.add(0, t8_bytes((uint32_t)n_out, (uint32_t)n_in));
                raw_bytes = n_out * (n_in / 32) * 34;
                np = 1;
            } else if (d->ggml_type == OXHIP_GGML_Q4_K) {
                if (n_in % 256) return fail("Q4_K rows must be whole blocks of 256");
                w->v.fmt = FMT_Q4_K;
                pl.add(0, tk4_bytes((uint32_t)n_out, (uint32_t)n_in));
                raw_bytes = n_out * (n_in / 256) * 144;
                np = 1;
            } else if (d->ggml_type == OXHIP_GGML_Q5_K) {
                if (n_in % 256) return fail("Q5_K rows must be whole blocks of 256");
                w->v.fmt = FMT_Q5_K;
                pl.add(0, tk5_bytes((uint32_t)n_out, (uint32_t)n_in));
                raw_bytes = n_out * (n_in / 256) * 176;
                np = 1;
            } else if (d->ggml_type == OXHIP_GGML_MXFP4) {
                if (n_in % 32) return fail("MXFP4 rows must be whole blocks of 32");
                w->v.fmt = FMT_MXFP4;
                pl.add(0, t4x_bytes((uint32_t)n_out, (uint32_t)n_in));
                raw_bytes = n_out * (n_in / 32) * 17;
                np = 1;
            } else if (d->ggml_type == OXHIP_GGML_Q6_K) {
                if (n_in % 256) return fail("Q6_K rows must be whole blocks of 256");
                w->v.fmt = FMT_Q6_K;
                pl.add(0, t6k_bytes((uint32_t)n_out, (uint32_t)n_in));
                raw_bytes = n_out * (n_in / 256) * 210;
                np = 1;
            } else {
                return fail("GGUF type " + std::to_string(d->ggml_type) + " has no device kernels");
            }
            if (!alloc(pl, np)) return fail("device memory short");
            Temp raw;
            if (!have_memory(raw_bytes) || !raw.put(d->data, raw_bytes, s)) return fail("device memory short");
            if (launch_repack_gguf(w->v.fmt, static_cast<const uint8_t*>(raw.p), n_out, n_in, w->v, s) != hipSuccess)
                return fail("repack launch failed");
            if (hipStreamSynchronize(s) != hipSuccess) return fail("repack failed");
            break;
        }
        default: return fail("weight kind " + std::to_string(d->kind) + " has no device kernels");
    }
    if (hipStreamSynchronize(s) != hipSuccess) return fail("upload failed");
    const bool q40 = q4_0_blocks && w->v.fmt == FMT_Q4;
    if (q40) w->v.br = 1;  // (kept should the tile packing below be skipped for lack of memory)
    if ((w->v.fmt == FMT_Q4 && w->v.group == 64 && w->v.sgroup == 64) || q40) {
        // one scale and one offset per 64 (MLX checkpoints), or GGUF Q4_0's scale per 32: tile-packed for the matrix cores
        const size_t bytes = t4m_bytes((uint32_t)n_out, (uint32_t)n_in);
        void* packed = nullptr;
        if (have_memory(bytes) && hipMalloc(&packed, bytes) == hipSuccess) {
            if (launch_pack_q4m(w->v.p0, reinterpret_cast<const uint16_t*>(w->v.p1), q40 ? nullptr : reinterpret_cast<const uint16_t*>(w->v.p2), n_out,
                                n_in, static_cast<uint8_t*>(packed), s) != hipSuccess ||
                hipStreamSynchronize(s) != hipSuccess) {
                (void)hipFree(packed);
                return fail("tile packing failed");
            }
            (void)hipFree(w->base);
            w->base = packed;
            w->bytes = bytes;
            w->v.fmt = q40 ? FMT_Q40 : FMT_Q4M;
            w->v.p0 = static_cast<const uint8_t*>(packed);
            w->v.p1 = w->v.p2 = nullptr;
        }
    }
    return w;
}

oxhip_weight* oxhip_upload(oxhip_ctx* c, const oxhip_weight_desc* d) { return upload_weight(c, d, false); }

// ---- device-pointer entry points ---------------------------------------------------------------
int oxhip_dev_quantize_act(oxhip_ctx* c, const float* x, size_t t, size_t n_in, const oxhip_qact* out, void* stream) {
    if (!c || !x || !out || n_in % 32) {
        set_error("quantize_act: bad arguments (n_in must be a multiple of 32)");
        return 0;
    }
    HIP_TRY(launch_quantize_act(x, t, n_in, *out, static_cast<hipStream_t>(stream)), "quantize_act launch");
    return 1;
}

int oxhip_dev_quantize_act_batch(oxhip_ctx* c, const oxhip_quant_job* jobs, size_t n_jobs, void* stream) {
    if (!c || (!jobs && n_jobs)) {
        set_error("quantize_act_batch: bad arguments");
        return 0;
    }
    std::vector<const float*> xs(n_jobs);
    std::vector<size_t> ts(n_jobs), ns(n_jobs);
    std::vector<oxhip_qact> outs(n_jobs);
    for (size_t j = 0; j < n_jobs; j++) {
        if (!jobs[j].x || !jobs[j].out || jobs[j].n_in % 32) {
            set_error("quantize_act_batch: job " + std::to_string(j) + ": bad arguments (n_in must be a multiple of 32)");
            return 0;
        }
        xs[j] = jobs[j].x;
        ts[j] = jobs[j].t;
        ns[j] = jobs[j].n_in;
        outs[j] = *jobs[j].out;
    }
    HIP_TRY(launch_quantize_act_batch(xs.data(), ts.data(), ns.data(), outs.data(), n_jobs, static_cast<hipStream_t>(stream)), "quantize_act_batch launch");
    return 1;
}

int oxhip_dev_dequantize(oxhip_ctx* c, const oxhip_weight* w, size_t r0, size_t r1, float* out, void* stream) {
    if (!c || !w || !out || r0 > r1 || r1 > w->v.n_out) {
        set_error("dequantize: bad arguments");
        return 0;
    }
    HIP_TRY(launch_dequantize(w->v, r0, r1, out, static_cast<hipStream_t>(stream)), "dequantize launch");
    return 1;
}

static int decode_one(oxhip_ctx* c, const oxhip_weight* w, const oxhip_qact* xa, const float* x, size_t t, float* y, void* stream,
                      hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (!c || !w || !y || t == 0 || t > 16) {
        set_error("decode: bad arguments (1 <= t <= 16)");
        return 0;
    }
    QActView v{};
    if (is_dense(w)) {
        if (!x) {
            set_error("decode: float-stored weights take f32 rows");
            return 0;
        }
    } else {
        if (!xa || xa->n_in != w->v.n_in || xa->t < t) {
            set_error("decode: quantized activations missing or of another shape");
            return 0;
        }
        v = view_of(*xa);
    }
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    StreamScratch* sc = scratch_for(c, static_cast<hipStream_t>(stream), needs_slices(w));
    if (!sc) {
        set_error(stream_recording(static_cast<hipStream_t>(stream)) ? "decode: the stream's K-slice scratch does not exist yet and a plan records on it (run the chain once before recording)"
                                                                     : "decode: device memory short");
        return 0;
    }
    HIP_TRY(launch_decode(w->v, v, x, t, y, static_cast<hipStream_t>(stream), sc->dec, ev_start, ev_stop), "decode launch");
    return 1;
}

int oxhip_dev_decode(oxhip_ctx* c, const oxhip_weight* w, const oxhip_qact* xa, const float* x, size_t t, float* y, void* stream) {
    return decode_one(c, w, xa, x, t, y, stream, nullptr, nullptr);
}

int oxhip_dev_decode_noalloc(oxhip_ctx* c, const oxhip_weight* w, const oxhip_qact* xa, size_t t, float* y, void* stream) {
    if (!c || !w || !xa || !y || t == 0 || t > 16) {
        set_error("decode_noalloc: bad arguments (1 <= t <= 16)");
        return 0;
    }
    if (!mfma_decode_format(w->v.fmt)) {
        set_error("decode_noalloc: only the quantized formats of the matrix-core decode kernel (Q8, Q8_0, Q4_0, Q4_K, Q5_K, Q6_K, MXFP4, MLX 4-bit)");
        return 0;
    }
    if (xa->n_in != w->v.n_in || xa->t < t) {
        set_error("decode_noalloc: quantized activations of another shape");
        return 0;
    }
    void* ptr = c->device < NOALLOC_MAX_DEVICES ? g_scratch_ptr[c->device] : nullptr;
    if (!ptr) {
        set_error("decode_noalloc: no static scratch on device " + std::to_string(c->device));
        return 0;
    }
    size_t need_p = 0, need_c = 0;
    decode_scratch_need(w->v, &need_p, &need_c);
    if (need_p > NOALLOC_PARTIAL_FLOATS || need_c > NOALLOC_COUNTERS) {
        set_error("decode_noalloc: [" + std::to_string(w->v.n_out) + ", " + std::to_string(w->v.n_in) + "] needs " + std::to_string(need_p * 4) +
                  " bytes of partial rows and " + std::to_string(need_c / CTR_STRIDE) + " row-group counters; the static scratch holds " +
                  std::to_string(NOALLOC_PARTIAL_FLOATS * 4) + " bytes and " + std::to_string(NOALLOC_COUNTERS / CTR_STRIDE) + " counters");
        return 0;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");  // `ptr` is this device's copy of the array
    DecodeScratch sc;
    sc.partial = static_cast<float*>(ptr);
    sc.counters = reinterpret_cast<uint32_t*>(static_cast<unsigned char*>(ptr) + NOALLOC_PARTIAL_FLOATS * 4);
    sc.partial_floats = NOALLOC_PARTIAL_FLOATS;
    sc.ncounters = NOALLOC_COUNTERS;
    if (need_c) {
        // the array keeps what the last call (of any caller on this GPU) left: the counters must start at zero. A small
        // kernel, not a memset: memset nodes captured into a graph have replayed wrongly.
        HIP_TRY(launch_fill_zero(sc.counters, need_c, s), "decode_noalloc: counter clear launch");
    }
    HIP_TRY(launch_decode_mfma(w->v, view_of(*xa), t, y, sc, s), "decode_noalloc launch");
    return 1;
}

int oxhip_dev_decode_batch(oxhip_ctx* c, const oxhip_decode_job* jobs, size_t n_jobs, void* stream) {
    if (!c || (!jobs && n_jobs)) {
        set_error("decode_batch: bad arguments");
        return 0;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    bool any_slices = false;
    for (size_t k = 0; k < n_jobs; k++) any_slices |= jobs[k].w && needs_slices(jobs[k].w);
    StreamScratch* ssc = scratch_for(c, s, any_slices);
    if (!ssc) {
        set_error(stream_recording(s) ? "decode_batch: the stream's K-slice scratch does not exist yet and a plan records on it (run the chain once before recording)"
                                      : "decode_batch: device memory short");
        return 0;
    }
    // Runs of jobs that the matrix-core decode kernel takes share one launch; the others go out one by one.
    auto fusable = [&](const oxhip_decode_job& jb) {
        return jb.w && jb.xa && jb.y && !is_dense(jb.w) && jb.xa->n_in == jb.w->v.n_in && jb.xa->t >= jb.t && decode_batchable(jb.w->v, jb.t);
    };
    size_t j = 0;
    std::vector<DecodeBatchItem> items;
    while (j < n_jobs) {
        size_t e = j;
        while (e < n_jobs && fusable(jobs[e])) e++;
        if (e - j >= 2) {
            // the first start event and the last stop event of the run bracket the shared launch; any others are
            // recorded on the stream around it
            items.clear();
            hipEvent_t e0 = nullptr, e1 = nullptr;
            for (size_t k = j; k < e; k++) {
                if (jobs[k].ev_start) {
                    if (!e0) e0 = static_cast<hipEvent_t>(jobs[k].ev_start);
                    else HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(jobs[k].ev_start), s), "event record");
                }
                items.push_back(DecodeBatchItem{jobs[k].w->v, view_of(*jobs[k].xa), jobs[k].y, (uint32_t)jobs[k].t, Epi{}});
            }
            for (size_t k = e; k-- > j;)
                if (jobs[k].ev_stop) {
                    e1 = static_cast<hipEvent_t>(jobs[k].ev_stop);
                    break;
                }
            const hipError_t err = launch_decode_mfma_batch(items.data(), items.size(), ssc->dec, s, e0, e1);
            if (err == hipErrorOutOfMemory) {  // the scratch does not hold these jobs together: one launch each
                if (e0) HIP_TRY(hipEventRecord(e0, s), "event record");
                for (size_t k = j; k < e; k++)
                    if (!oxhip_dev_decode(c, jobs[k].w, jobs[k].xa, jobs[k].x, jobs[k].t, jobs[k].y, stream)) return 0;
                if (e1) HIP_TRY(hipEventRecord(e1, s), "event record");
            } else {
                HIP_TRY(err, "decode batch launch");
            }
            for (size_t k = j; k < e; k++)
                if (jobs[k].ev_stop && static_cast<hipEvent_t>(jobs[k].ev_stop) != e1) HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(jobs[k].ev_stop), s), "event record");
            j = e;
            continue;
        }
        const oxhip_decode_job& jb = jobs[j];
        if (!decode_one(c, jb.w, jb.xa, jb.x, jb.t, jb.y, stream, static_cast<hipEvent_t>(jb.ev_start), static_cast<hipEvent_t>(jb.ev_stop))) return 0;
        j++;
    }
    return 1;
}

void* oxhip_event_create(void) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
        set_error("hipEventCreate failed");
        return nullptr;
    }
    return e;
}

void oxhip_event_destroy(void* ev) {
    if (ev) (void)hipEventDestroy(static_cast<hipEvent_t>(ev));
}

float oxhip_event_elapsed_ms(void* a, void* b) {
    float ms = -1.0f;
    if (!a || !b) return ms;
    if (hipEventSynchronize(static_cast<hipEvent_t>(b)) != hipSuccess) return -1.0f;
    if (hipEventElapsedTime(&ms, static_cast<hipEvent_t>(a), static_cast<hipEvent_t>(b)) != hipSuccess) return -1.0f;
    return ms;
}

int oxhip_dev_isums(oxhip_ctx* c, const oxhip_weight* w, const oxhip_qact* xa, int32_t* out, void* stream) {
    if (!c || !w || !xa || !out || is_dense(w) || xa->n_in != w->v.n_in) {
        set_error("isums: bad arguments");
        return 0;
    }
    HIP_TRY(launch_isums(w->v, view_of(*xa), xa->t, out, static_cast<hipStream_t>(stream)), "isums launch");
    return 1;
}

// ---- Backend surface ---------------------------------------------------------------------------
int oxhip_matmul(oxhip_ctx* c, const float* x, size_t t, size_t n_in, oxhip_job* jobs, size_t n_jobs) {
    if (!c || !x || !jobs || !t || !n_jobs || n_in % 32) {
        set_error("matmul: bad arguments");
        return 0;
    }
    size_t y_total = 0;
    bool any_q = false;
    for (size_t j = 0; j < n_jobs; j++) {
        const oxhip_weight* w = jobs[j].w;
        if (!w || !jobs[j].y || w->v.n_in != n_in || w->v.n_out != jobs[j].n_out) {
            set_error("matmul: job " + std::to_string(j) + " does not match its weight");
            return 0;
        }
        y_total += t * w->v.n_out;
        any_q |= !is_dense(w);
    }
    std::lock_guard<std::mutex> g(c->mu);
    HIP_TRY(hipSetDevice(c->device), "hipSetDevice");
    hipStream_t s = c->stream;
    if (!c->x.grow(t * n_in * 4) || !c->y.grow(y_total * 4) || (any_q && !c->xq.grow(qact_bytes(t, n_in)))) {
        set_error("matmul: device memory short");
        return 0;
    }
    hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr, e3 = nullptr;
    auto done = [&](int rc) {
        for (hipEvent_t e : {e0, e1, e2, e3})
            if (e) (void)hipEventDestroy(e);
        return rc;
    };
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess || hipEventCreate(&e2) != hipSuccess ||
        hipEventCreate(&e3) != hipSuccess) {
        set_error("matmul: hipEventCreate failed");
        return done(0);
    }
    // Everything is computed into device staging first; y is written only once all jobs ran.
    (void)hipEventRecord(e0, s);
    if (hipMemcpyAsync(c->x.p, x, t * n_in * 4, hipMemcpyHostToDevice, s) != hipSuccess) {
        set_error("matmul: copy-in failed");
        return done(0);
    }
    (void)hipEventRecord(e1, s);
    oxhip_qact xa{};
    if (any_q) {
        xa = carve_qact(c->xq.p, t, n_in);
        if (launch_quantize_act(static_cast<const float*>(c->x.p), t, n_in, xa, s) != hipSuccess) {
            set_error("matmul: quantize_act launch failed");
            return done(0);
        }
    }
    float* yd = static_cast<float*>(c->y.p);
    // Routing, as matmul_quant_multi_at does (src/kernels.rs:1731-1879): up to 8 tokens the jobs that the matrix-core
    // decode kernel takes share one launch; more than 16 tokens go to the prefill GEMM where the format has one (MLX
    // 4-bit, FP8 with 128-column blocks: bf16 matrix cores, f32 accumulation); everything else runs the decode
    // kernels over 16 tokens at a time.
    std::vector<DecodeBatchItem> fused;
    std::vector<size_t> offs(n_jobs);
    size_t off = 0;
    for (size_t j = 0; j < n_jobs; j++) {
        offs[j] = off;
        off += t * jobs[j].w->v.n_out;
    }
    auto fail = [&](const char* what) {
        set_error(std::string("matmul: ") + what);
        (void)hipStreamSynchronize(s);
        return done(0);
    };
    for (size_t j = 0; j < n_jobs; j++) {
        const oxhip_weight* w = jobs[j].w;
        if (t <= 8 && !is_dense(w) && decode_batchable(w->v, t)) {
            fused.push_back(DecodeBatchItem{w->v, view_of(xa), yd + offs[j], (uint32_t)t, Epi{}});
            continue;
        }
        const bool gemm = t > 16 && gemm_bf16_ok(w->v);
        if (gemm) {
            if (!gemm_bf16_run(c->gemm_ws, w, c->x.p, false, t, yd + offs[j], false, s)) {
                (void)hipStreamSynchronize(s);
                return done(0);
            }
            continue;
        }
        for (size_t c0 = 0; c0 < t; c0 += 16) {
            const size_t tc = t - c0 < 16 ? t - c0 : 16;
            QActView v = view_of(xa);
            if (!is_dense(w)) {
                v.q += c0 * n_in;
                v.scales += c0 * (n_in / 32);
                v.sums += c0 * (n_in / 32);
                v.fsums += c0 * (n_in / 32);
                v.hsums += c0 * (n_in / 16);
                v.sums16 += c0 * (n_in / 16);
            }
            if (launch_decode(w->v, v, static_cast<const float*>(c->x.p) + c0 * n_in, tc, yd + offs[j] + c0 * w->v.n_out, s, c->dec) != hipSuccess)
                return fail("decode launch failed");
        }
    }
    if (fused.size() == 1) {
        if (launch_decode(fused[0].w, fused[0].xa, nullptr, t, fused[0].y, s, c->dec) != hipSuccess) return fail("decode launch failed");
    } else if (!fused.empty()) {
        hipError_t e = launch_decode_mfma_batch(fused.data(), fused.size(), c->dec, s);
        if (e == hipErrorOutOfMemory) {
            for (auto& it : fused)
                if (launch_decode(it.w, it.xa, nullptr, t, it.y, s, c->dec) != hipSuccess) return fail("decode launch failed");
        } else if (e != hipSuccess) {
            return fail("decode batch launch failed");
        }
    }
    (void)hipEventRecord(e2, s);
    if (hipStreamSynchronize(s) != hipSuccess) {
        set_error("matmul: kernels failed");
        return done(0);
    }
    off = 0;
    std::vector<float> host(y_total);
    if (hipMemcpyAsync(host.data(), yd, y_total * 4, hipMemcpyDeviceToHost, s) != hipSuccess) {
        set_error("matmul: copy-out failed");
        return done(0);
    }
    (void)hipEventRecord(e3, s);
    if (hipStreamSynchronize(s) != hipSuccess) {
        set_error("matmul: copy-out failed");
        return done(0);
    }
    for (size_t j = 0; j < n_jobs; j++) {
        size_t n = t * jobs[j].w->v.n_out;
        std::memcpy(jobs[j].y, host.data() + off, n * 4);
        off += n;
    }
    float a = 0, b = 0, d = 0;
    (void)hipEventElapsedTime(&a, e0, e1);
    (void)hipEventElapsedTime(&b, e1, e2);
    (void)hipEventElapsedTime(&d, e2, e3);
    c->ms_in += a;
    c->ms_gpu += b;
    c->ms_out += d;
    c->calls++;
    return done(1);
}

}  // extern "C"
