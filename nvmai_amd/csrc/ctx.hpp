// Host-side context shared by every entry-point file.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

#include "../../include/nvmai_hip.h"

struct nvmai_hip_ctx {
    int device;
    int compute_units;       // of the device (persistent grids are sized from it)
    int act;                 // NVMAI_ACT_BF16 / NVMAI_ACT_FP16
    // Workspace: one device buffer carved by a bump pointer inside each entry
    // point.  Work on one stream is ordered, so consecutive calls may reuse it.
    uint8_t* ws;
    size_t ws_cap;
    size_t ws_used;
    // Blocks the workspace has outgrown.  They stay allocated until the context is destroyed: a
    // captured graph keeps the addresses it was recorded with, and replaying it must stay valid
    // after a later, larger call has moved the workspace.
    std::vector<void*> ws_retired;
    uint8_t* static_scratch; // device address of the library's static scratch array on this device (moe_api.hip)
    uint32_t* tickets;       // zero-initialised device words for last-block-done kernels (TICKET_WORDS)
    // Optional per-kernel timing: event pairs recorded around tagged launches.
    bool prof_on;
    struct ProfSpan { int tag; hipEvent_t start, stop; };
    std::vector<ProfSpan> prof_spans;
    std::vector<hipEvent_t> prof_free;
};

namespace nvmai {

// The context's persistent zeroed words: [0] work-list ticket, [8] prefill grouping error word,
// [16, 48) sampler block counters, [TICKET_GROUPS, TICKET_WORDS) router token-group tickets.
constexpr uint32_t TICKET_WORDS = 2048;
constexpr uint32_t TICKET_GROUPS = 64;

#define NVMAI_HIP_TRY(expr)                         \
    do {                                            \
        hipError_t e_ = (expr);                     \
        if (e_ != hipSuccess) return NVMAI_ERR_HIP; \
    } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Make the workspace at least `bytes` large and reset the bump pointer.  Growing allocates a new
// block (sizes double, so the retired blocks together are smaller than the live one) and never
// frees the old one: launches already recorded into a graph keep pointing at it.  A call that
// would have to grow while `stream` is being captured returns NVMAI_ERR_SCRATCH instead of
// allocating inside the capture: size the workspace first, with an eager call of the same shape
// or with nvmai_hip_ctx_reserve.
inline int ws_begin(nvmai_hip_ctx* ctx, nvmai_stream stream, size_t bytes) {
    ctx->ws_used = 0;
    if (bytes <= ctx->ws_cap) return NVMAI_OK;
    hipStreamCaptureStatus cap_status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cap_status) != hipSuccess) {
        (void)hipGetLastError();
        cap_status = hipStreamCaptureStatusNone;
    }
    if (cap_status != hipStreamCaptureStatusNone) return NVMAI_ERR_SCRATCH;
    size_t cap = ctx->ws_cap ? ctx->ws_cap : (size_t)1 << 20;
    while (cap < bytes) cap *= 2;
    uint8_t* block = nullptr;
    NVMAI_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&block), cap));
    if (ctx->ws) ctx->ws_retired.push_back(ctx->ws);
    ctx->ws = block;
    ctx->ws_cap = cap;
    return NVMAI_OK;
}

inline size_t ws_round(size_t bytes) { return (bytes + 255) & ~(size_t)255; }

template <typename T>
inline T* ws_take(nvmai_hip_ctx* ctx, size_t count) {
    T* p = reinterpret_cast<T*>(ctx->ws + ctx->ws_used);
    ctx->ws_used += ws_round(count * sizeof(T));
    return p;
}

// Brackets the launches of one kernel with events while profiling is switched on.
struct ProfScope {
    nvmai_hip_ctx* ctx;
    hipStream_t stream;
    hipEvent_t stop;
    ProfScope(nvmai_hip_ctx* c, int tag, hipStream_t s) : ctx(c), stream(s), stop(nullptr) {
        if (!c->prof_on) return;
        hipEvent_t ev[2] = {nullptr, nullptr};
        for (auto& e : ev) {
            if (!c->prof_free.empty()) { e = c->prof_free.back(); c->prof_free.pop_back(); }
            else if (hipEventCreate(&e) != hipSuccess) return;
        }
        (void)hipEventRecord(ev[0], s);
        stop = ev[1];
        c->prof_spans.push_back({tag, ev[0], ev[1]});
    }
    ~ProfScope() { if (stop) (void)hipEventRecord(stop, stream); }
};

// One expert over all rows through the grouped-GEMM kernels (prefill_api.hip).
int expert_ffn_dense(nvmai_hip_ctx* ctx, hipStream_t s, const uint8_t* blob, const nvmai_expert_offsets* off,
                     uint32_t bits, const void* x, uint32_t x_stride, uint32_t tokens, uint32_t d, uint32_t f,
                     void* act, void* tmp, const float* gate_logit, void* y, uint32_t y_stride);

// Dense BF16 rows against BF16 inputs on the matrix cores (step_api.hip).
int dense_bf16_gemv(nvmai_hip_ctx* ctx, hipStream_t s, const uint16_t* w, const void* x, uint32_t x_stride,
                    uint32_t n_tokens, uint32_t m, uint32_t n, void* y, float* y_f32, uint32_t y_stride);

// Affine 4 / 8-bit rows against 1 .. 32 input rows on the matrix cores, the matrix read once
// (gemv_mfma_api.hip).  gemv_mfma_ok: the shapes and alignments it takes.
bool gemv_mfma_ok(const uint8_t* w, const uint16_t* s, const uint16_t* b, uint32_t bits, const void* x,
                  uint32_t x_stride, uint32_t n_tokens, uint32_t m, uint32_t n, const void* y, const float* y_f32,
                  uint32_t y_stride);
int gemv_mfma(nvmai_hip_ctx* ctx, hipStream_t s, const uint8_t* w, const uint16_t* scales, const uint16_t* biases,
              uint32_t bits, const void* x, uint32_t x_stride, uint32_t n_tokens, uint32_t m, uint32_t n, void* y,
              float* y_f32, uint32_t y_stride);

inline int launch_status() { return hipGetLastError() == hipSuccess ? NVMAI_OK : NVMAI_ERR_HIP; }

}  // namespace nvmai
