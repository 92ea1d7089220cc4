// A recorded run of device-pointer ops that replays as one submission: the matmul side of the reference's DecodePlan
// (src/gpu_decode.rs:572-587; the CUDA backend builds a fixed launch list per graph once and re-issues it every token,
// src/cuda_decode.rs:1044-1049). Here the list is a HIP graph captured from the library's own launches: between
// oxhip_plan_begin and oxhip_plan_end every oxhip_dev_* call on the plan's stream is recorded instead of run, and
// oxhip_plan_replay submits all of them at once, so a token pays one host call for its whole chain of launches.
//
// What makes the library's launches recordable: nothing in a warmed call allocates, frees, synchronizes or clears memory
// with a memset (arrival counters return to zero inside the kernels that use them; the few clears there are go through a
// fill kernel). Scratch that grows on first use (a stream's K-slice rows, an MoE layer's pass buffers, packed GEMM
// activations) must exist before recording starts: run the chain once on the same stream first. A call that would have to
// allocate while recording fails the recording (oxhip_plan_end reports it), and nothing is replayable then.
#include "backend.hpp"

using namespace oxhip;

struct oxhip_plan {
    oxhip_ctx* ctx = nullptr;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    bool recording = false;
    size_t nodes = 0;
};

extern "C" {

oxhip_plan* oxhip_plan_begin(oxhip_ctx* c, void* stream) {
    if (!c || !stream) {
        set_error("plan_begin: needs a context and a stream of its own (not the null stream)");
        return nullptr;
    }
    if (hipSetDevice(c->device) != hipSuccess) {
        set_error("plan_begin: hipSetDevice failed");
        return nullptr;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    // thread-local mode: other threads of the process may go on allocating while this one records
    hipError_t e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) {
        set_error(std::string("plan_begin: hipStreamBeginCapture: ") + hipGetErrorString(e));
        return nullptr;
    }
    {
        std::lock_guard<std::mutex> lk(c->smu);
        c->record_failed.erase(s);
    }
    auto* p = new oxhip_plan();
    p->ctx = c;
    p->stream = s;
    p->recording = true;
    return p;
}

int oxhip_plan_end(oxhip_plan* p) {
    if (!p || !p->recording) {
        set_error("plan_end: no recording in progress");
        return 0;
    }
    p->recording = false;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(p->stream, &g);
    bool refused;
    {
        std::lock_guard<std::mutex> lk(p->ctx->smu);
        refused = p->ctx->record_failed.erase(p->stream) != 0;
    }
    if (refused) {  // a recorded call declined because it would have had to allocate: its launches are missing from the graph
        if (g) (void)hipGraphDestroy(g);
        (void)hipGetLastError();
        set_error("plan_end: a recorded call needed scratch that did not exist yet (run the chain once on this stream before recording)");
        return 0;
    }
    if (e != hipSuccess || !g) {
        (void)hipGetLastError();
        set_error(std::string("plan_end: the recording was invalidated (a recorded call allocated, synchronized or failed): ") + hipGetErrorString(e));
        return 0;
    }
    size_t n = 0;
    (void)hipGraphGetNodes(g, nullptr, &n);
    if (!n) {
        (void)hipGraphDestroy(g);
        set_error("plan_end: nothing was recorded on the plan's stream");
        return 0;
    }
    hipGraphExec_t x = nullptr;
    e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        set_error(std::string("plan_end: hipGraphInstantiate: ") + hipGetErrorString(e));
        return 0;
    }
    p->graph = g;
    p->exec = x;
    p->nodes = n;
    return 1;
}

size_t oxhip_plan_launches(const oxhip_plan* p) { return p ? p->nodes : 0; }

int oxhip_plan_replay(oxhip_plan* p, void* stream) {
    if (!p || !p->exec) {
        set_error("plan_replay: the plan holds no finished recording");
        return 0;
    }
    HIP_TRY(hipSetDevice(p->ctx->device), "hipSetDevice");
    HIP_TRY(hipGraphLaunch(p->exec, stream ? static_cast<hipStream_t>(stream) : p->stream), "plan_replay: hipGraphLaunch");
    return 1;
}

void oxhip_plan_free(oxhip_plan* p) {
    if (!p) return;
    if (p->ctx) (void)hipSetDevice(p->ctx->device);
    if (p->recording) {  // abandon the recording
        hipGraph_t g = nullptr;
        (void)hipStreamEndCapture(p->stream, &g);
        if (g) (void)hipGraphDestroy(g);
        (void)hipGetLastError();
    }
    if (p->exec) (void)hipGraphExecDestroy(p->exec);
    if (p->graph) (void)hipGraphDestroy(p->graph);
    delete p;
}

}  // extern "C"
