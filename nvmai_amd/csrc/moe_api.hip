// Entry points of the decode-side MoE path: context, quantizer, affine GEMV,
// router top-k, routed phase 1 / phase 2, shared expert, fused decode layer.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <new>

#include "ctx.hpp"
#include "moe_kernels.hpp"

using namespace nvmai;

namespace {

// Scratch of the allocation-free decode entry point: one array per device, in the library's image,
// so that a caller which may not allocate (HIP graph capture, a serving loop, a harness that
// forbids hipMalloc) still has the step's intermediate buffers.  Host code never uses the
// array's name as an address: the device address comes from hipGetSymbolAddress, once per device.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)4 << 20;
static __device__ __align__(256) __attribute__((used)) uint8_t scratch[STATIC_SCRATCH_BYTES];
constexpr int STATIC_SCRATCH_MAX_DEVICES = 64;
// Device address of `scratch` on each device, nullptr = not asked yet.  Contexts may be created from several
// threads: the slots are atomics (every thread that fills one stores the same address, so no lock is needed).
std::atomic<uint8_t*> g_static_scratch[STATIC_SCRATCH_MAX_DEVICES];

// The device address of this device's copy of the array (the device must be current).
int static_scratch_ptr(int device, uint8_t** out) {
    if (device < 0 || device >= STATIC_SCRATCH_MAX_DEVICES) return NVMAI_ERR_INVALID_ARG;
    uint8_t* known = g_static_scratch[device].load(std::memory_order_acquire);
    if (!known) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
            (void)hipGetLastError();
            return NVMAI_ERR_HIP;
        }
        known = static_cast<uint8_t*>(ptr);
        g_static_scratch[device].store(known, std::memory_order_release);
    }
    *out = known;
    return NVMAI_OK;
}

}  // namespace

// ---------------------------------------------------------------------------
// context
// ---------------------------------------------------------------------------
extern "C" int nvmai_hip_ctx_create(int device, int act_dtype, nvmai_hip_ctx** out) {
    if (!out || (act_dtype != NVMAI_ACT_BF16 && act_dtype != NVMAI_ACT_FP16)) return NVMAI_ERR_INVALID_ARG;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return NVMAI_ERR_NO_DEVICE;
    if (device < 0 || device >= count) return NVMAI_ERR_INVALID_ARG;
    NVMAI_HIP_TRY(hipSetDevice(device));
    nvmai_hip_ctx* ctx = new (std::nothrow) nvmai_hip_ctx();
    if (!ctx) return NVMAI_ERR_HIP;
    ctx->device = device;
    ctx->compute_units = 256;
    {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && cus > 0)
            ctx->compute_units = cus;
    }
    ctx->act = act_dtype;
    ctx->ws = nullptr;
    ctx->ws_cap = 0;
    ctx->ws_used = 0;
    ctx->prof_on = false;
    ctx->tickets = nullptr;
    if (hipMalloc(reinterpret_cast<void**>(&ctx->tickets), TICKET_WORDS * 4) != hipSuccess ||
        hipMemset(ctx->tickets, 0, TICKET_WORDS * 4) != hipSuccess) {
        delete ctx;
        return NVMAI_ERR_HIP;
    }
    // device address of this device's static scratch array (nullptr if the lookup fails: only the
    // allocation-free entry point needs it, and it then reports the failure)
    ctx->static_scratch = nullptr;
    (void)static_scratch_ptr(device, &ctx->static_scratch);
    *out = ctx;
    return NVMAI_OK;
}

extern "C" void nvmai_hip_ctx_destroy(nvmai_hip_ctx* ctx) {
    if (!ctx) return;
    if (ctx->ws) (void)hipFree(ctx->ws);
    for (void* block : ctx->ws_retired) (void)hipFree(block);
    if (ctx->tickets) (void)hipFree(ctx->tickets);
    for (auto& sp : ctx->prof_spans) { (void)hipEventDestroy(sp.start); (void)hipEventDestroy(sp.stop); }
    for (auto& e : ctx->prof_free) (void)hipEventDestroy(e);
    delete ctx;
}

extern "C" int nvmai_hip_ctx_reserve(nvmai_hip_ctx* ctx, size_t bytes) {
    if (!ctx) return NVMAI_ERR_INVALID_ARG;
    NVMAI_HIP_TRY(hipSetDevice(ctx->device));
    return ws_begin(ctx, nullptr, bytes);
}

extern "C" size_t nvmai_hip_ctx_workspace_bytes(const nvmai_hip_ctx* ctx) { return ctx ? ctx->ws_cap : 0; }

extern "C" int nvmai_hip_profile_enable(nvmai_hip_ctx* ctx, int on) {
    if (!ctx) return NVMAI_ERR_INVALID_ARG;
    if (on) {
        for (auto& sp : ctx->prof_spans) {
            NVMAI_HIP_TRY(hipEventSynchronize(sp.stop));
            ctx->prof_free.push_back(sp.start);
            ctx->prof_free.push_back(sp.stop);
        }
        ctx->prof_spans.clear();
    }
    ctx->prof_on = on != 0;
    return NVMAI_OK;
}

extern "C" int nvmai_hip_profile_read(nvmai_hip_ctx* ctx, int tag, double* total_ms, uint32_t* launches) {
    if (!ctx || !total_ms || !launches) return NVMAI_ERR_INVALID_ARG;
    double total = 0.0;
    uint32_t n = 0;
    for (auto& sp : ctx->prof_spans) {
        if (sp.tag != tag) continue;
        NVMAI_HIP_TRY(hipEventSynchronize(sp.stop));
        float ms = 0.0f;
        NVMAI_HIP_TRY(hipEventElapsedTime(&ms, sp.start, sp.stop));
        total += ms;
        ++n;
    }
    *total_ms = total;
    *launches = n;
    return NVMAI_OK;
}

extern "C" const char* nvmai_hip_status_string(int status) {
    switch (status) {
        case NVMAI_OK: return "ok";
        case NVMAI_ERR_INVALID_ARG: return "invalid argument";
        case NVMAI_ERR_UNSUPPORTED: return "unsupported configuration";
        case NVMAI_ERR_ALIGNMENT: return "pointer or stride not 16-byte aligned";
        case NVMAI_ERR_SCRATCH: return "scratch too small";
        case NVMAI_ERR_HIP: return "HIP runtime error";
        case NVMAI_ERR_NO_DEVICE: return "no HIP device";
        default: return "unknown status";
    }
}

extern "C" int nvmai_expert_offsets_for(uint32_t d, uint32_t f, uint32_t bits,
                                        nvmai_expert_offsets* out, uint64_t* stride_bytes) {
    if (!out || d == 0 || f == 0 || d % NVMAI_GROUP || f % NVMAI_GROUP) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    const uint64_t gate_w = (uint64_t)f * d * bits / 8, gate_meta = (uint64_t)f * (d / NVMAI_GROUP) * 2;
    const uint64_t down_w = (uint64_t)d * f * bits / 8, down_meta = (uint64_t)d * (f / NVMAI_GROUP) * 2;
    uint64_t o = 0;
    if (gate_w * 2 + down_w + 4 * gate_meta + 2 * down_meta > 0xFFFFFFFFull) return NVMAI_ERR_INVALID_ARG;
    out->gate_w = (uint32_t)o; o += gate_w;
    out->gate_s = (uint32_t)o; o += gate_meta;
    out->gate_b = (uint32_t)o; o += gate_meta;
    out->up_w = (uint32_t)o; o += gate_w;
    out->up_s = (uint32_t)o; o += gate_meta;
    out->up_b = (uint32_t)o; o += gate_meta;
    out->down_w = (uint32_t)o; o += down_w;
    out->down_s = (uint32_t)o; o += down_meta;
    out->down_b = (uint32_t)o; o += down_meta;
    if (stride_bytes) *stride_bytes = o;
    return NVMAI_OK;
}

// ---------------------------------------------------------------------------
// rows-engine dispatch
// ---------------------------------------------------------------------------
namespace {

template <int ACT, int BITS, int SEG, int NCH, int MAXTOK, bool DUAL, bool XF32, int RPI, int ITERS>
void launch_fast(RowsParams& p, uint32_t max_entries, hipStream_t s) {
    constexpr uint32_t rows_per_block = 4 * (64 / SEG) * RPI * ITERS;
    p.blocks_per_entry = (p.rows + rows_per_block - 1) / rows_per_block;
    const size_t lds = rows_fast_lds_bytes(p.n, NCH, SEG);
    expert_rows_fast<ACT, BITS, SEG, NCH, MAXTOK, DUAL, XF32, RPI, ITERS>
        <<<dim3(max_entries * p.blocks_per_entry), dim3(256), lds, s>>>(p);
}

template <int ACT, int BITS, bool DUAL, bool XF32>
void launch_rows_t(RowsParams& p, int maxtok, uint32_t max_entries, hipStream_t s) {
    const uint32_t chunks = p.n * BITS / 128;
#define NVMAI_FAST(SEG, NCH, RPI, ITERS)                                                        \
    do {                                                                                        \
        if (maxtok == 1) launch_fast<ACT, BITS, SEG, NCH, 1, DUAL, XF32, RPI, ITERS>(p, max_entries, s); \
        else launch_fast<ACT, BITS, SEG, NCH, 4, DUAL, XF32, RPI, ITERS>(p, max_entries, s);    \
        return;                                                                                 \
    } while (0)
    // Few entries (a small decode batch): short blocks, so that the launch still covers the device.
    const bool few = max_entries <= 40;
    if constexpr (DUAL) {
        if (few && chunks == 64) NVMAI_FAST(64, 1, 1, 2);
        if (few && chunks == 128) NVMAI_FAST(64, 2, 1, 2);
    } else {
        if (few && chunks == 16) NVMAI_FAST(16, 1, 1, 2);
        if (few && chunks == 32) NVMAI_FAST(32, 1, 2, 2);
    }
    if constexpr (DUAL) {
        if (chunks == 64) {
            // as long a block as still leaves about five blocks per CU (measured at 4 bit, hidden
            // 2048: batch 32 52 -> 47 us with eight steps, batch 8 faster with two)
            const uint64_t units = (uint64_t)max_entries * ((p.rows + 15) / 16);   // blocks at two steps
            if (units >= 4 * 1280) NVMAI_FAST(64, 1, 2, 8);
            if (units >= 2 * 1280) NVMAI_FAST(64, 1, 2, 4);
            NVMAI_FAST(64, 1, 2, 2);
        }
        if (chunks == 128) {
            const uint64_t units = (uint64_t)max_entries * ((p.rows + 7) / 8);     // blocks at two steps
            if (units >= 4 * 1280) NVMAI_FAST(64, 2, 1, 8);
            if (units >= 2 * 1280) NVMAI_FAST(64, 2, 1, 4);
            NVMAI_FAST(64, 2, 1, 2);
        }
    } else {
        // short rows: everything a wave reads is requested up front, more waves are resident
        if (chunks == 16) NVMAI_FAST(16, 1, 2, 2);
        if (chunks == 32) NVMAI_FAST(32, 1, 4, 2);
        if (chunks == 64) NVMAI_FAST(64, 1, 2, 4);
        if (chunks == 128) NVMAI_FAST(64, 2, 1, 8);
    }
#undef NVMAI_FAST
    p.blocks_per_entry = (p.rows + 15) / 16;
    expert_rows_generic<ACT, BITS, DUAL, XF32>
        <<<dim3(max_entries * p.blocks_per_entry), dim3(256), 0, s>>>(p);
}

// maxtok: 1 when every entry holds one pair, else MAX_TOK.
void launch_rows(int act, uint32_t bits, bool dual, bool xf32, RowsParams& p, int maxtok,
                 uint32_t max_entries, hipStream_t s) {
    if (max_entries == 0) return;
    if (xf32 && !dual) {   // inputs are fp32: one instantiation serves both activation types
        if (bits == 8) launch_rows_t<ACT_BF16, 8, false, true>(p, maxtok, max_entries, s);
        else launch_rows_t<ACT_BF16, 4, false, true>(p, maxtok, max_entries, s);
        return;
    }
#define NVMAI_ROWS(ACT, BITS)                                                   \
    do {                                                                        \
        if (dual) launch_rows_t<ACT, BITS, true, false>(p, maxtok, max_entries, s);   \
        else launch_rows_t<ACT, BITS, false, false>(p, maxtok, max_entries, s); \
    } while (0)
    if (act == ACT_BF16) { if (bits == 8) NVMAI_ROWS(ACT_BF16, 8); else NVMAI_ROWS(ACT_BF16, 4); }
    else { if (bits == 8) NVMAI_ROWS(ACT_FP16, 8); else NVMAI_ROWS(ACT_FP16, 4); }
#undef NVMAI_ROWS
}

// One matrix against dense_count 16-bit input rows in ONE launch (no work-list launch before it,
// no copy-out after it): the shapes the fast engine has a single-matrix instantiation for.
// Returns false, having launched nothing, for any other shape.
template <int ACT, int BITS>
bool launch_dense_rows_t(RowsParams& p, int maxtok, uint32_t ents, hipStream_t s) {
    const uint32_t chunks = p.n * BITS / 128;
    if ((p.n * BITS) % 128) return false;
#define NVMAI_DENSE(SEG, NCH, RPI, ITERS)                                                          \
    do {                                                                                           \
        constexpr uint32_t rows_per_block = 4 * (64 / SEG) * RPI * ITERS;                          \
        p.blocks_per_entry = (p.rows + rows_per_block - 1) / rows_per_block;                       \
        const size_t lds = rows_fast_lds_bytes(p.n, NCH, SEG);                                     \
        const dim3 grid(ents * p.blocks_per_entry);                                                \
        if (maxtok == 1) expert_rows_fast<ACT, BITS, SEG, NCH, 1, false, false, RPI, ITERS, true><<<grid, 256, lds, s>>>(p); \
        else expert_rows_fast<ACT, BITS, SEG, NCH, 4, false, false, RPI, ITERS, true><<<grid, 256, lds, s>>>(p);             \
        return true;                                                                               \
    } while (0)
    const bool few = ents <= 40;      // the same block shapes as the work-list launches
    // a projection of a decode step (a few thousand rows): blocks of 8 or 16 rows, so that the
    // launch covers the device; the long blocks below are for matrices like the LM head
    const uint64_t total_rows = (uint64_t)ents * p.rows;
    if (total_rows <= 4096 && chunks == 64) NVMAI_DENSE(64, 1, 1, 2);
    if (total_rows <= 4096 && chunks == 128) NVMAI_DENSE(64, 2, 1, 2);
    if (total_rows <= 16384 && chunks == 64) NVMAI_DENSE(64, 1, 2, 2);
    if (total_rows <= 16384 && chunks == 128) NVMAI_DENSE(64, 2, 1, 4);
    if (few && chunks == 16) NVMAI_DENSE(16, 1, 1, 2);
    if (few && chunks == 32) NVMAI_DENSE(32, 1, 2, 2);
    if (chunks == 16) NVMAI_DENSE(16, 1, 2, 2);
    if (chunks == 32) NVMAI_DENSE(32, 1, 4, 2);
    if (chunks == 64) NVMAI_DENSE(64, 1, 2, 4);
    if (chunks == 128) NVMAI_DENSE(64, 2, 1, 8);
#undef NVMAI_DENSE
    return false;
}

// Gate/up + SwiGLU of ONE expert (blob slot 0) over dense_count input rows in one launch, short blocks.
template <int ACT, int BITS>
bool launch_dense_dual_t(RowsParams& p, int maxtok, uint32_t ents, hipStream_t s) {
    const uint32_t chunks = p.n * BITS / 128;
    if ((p.n * BITS) % 128 || (chunks != 64 && chunks != 128)) return false;
    constexpr uint32_t rows_per_block = 4 * 1 * 1 * 2;
    p.blocks_per_entry = (p.rows + rows_per_block - 1) / rows_per_block;
    const dim3 grid(ents * p.blocks_per_entry);
#define NVMAI_DUAL(NCH)                                                                                          \
    do {                                                                                                         \
        const size_t lds = rows_fast_lds_bytes(p.n, NCH, 64);                                                    \
        if (maxtok == 1) expert_rows_fast<ACT, BITS, 64, NCH, 1, true, false, 1, 2, true><<<grid, 256, lds, s>>>(p); \
        else expert_rows_fast<ACT, BITS, 64, NCH, 4, true, false, 1, 2, true><<<grid, 256, lds, s>>>(p);         \
    } while (0)
    if (chunks == 64) NVMAI_DUAL(1); else NVMAI_DUAL(2);
#undef NVMAI_DUAL
    return true;
}

bool launch_dense_dual(int act, uint32_t bits, RowsParams& p, int maxtok, uint32_t ents, hipStream_t s) {
    if (act == ACT_BF16) return bits == 8 ? launch_dense_dual_t<ACT_BF16, 8>(p, maxtok, ents, s)
                                          : launch_dense_dual_t<ACT_BF16, 4>(p, maxtok, ents, s);
    return bits == 8 ? launch_dense_dual_t<ACT_FP16, 8>(p, maxtok, ents, s)
                     : launch_dense_dual_t<ACT_FP16, 4>(p, maxtok, ents, s);
}

bool launch_dense_rows(int act, uint32_t bits, RowsParams& p, int maxtok, uint32_t ents, hipStream_t s) {
    if (act == ACT_BF16) return bits == 8 ? launch_dense_rows_t<ACT_BF16, 8>(p, maxtok, ents, s)
                                          : launch_dense_rows_t<ACT_BF16, 4>(p, maxtok, ents, s);
    return bits == 8 ? launch_dense_rows_t<ACT_FP16, 8>(p, maxtok, ents, s)
                     : launch_dense_rows_t<ACT_FP16, 4>(p, maxtok, ents, s);
}

int check_shape(uint32_t d, uint32_t f, uint32_t bits) {
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (d == 0 || f == 0 || d % NVMAI_GROUP || f % NVMAI_GROUP) return NVMAI_ERR_INVALID_ARG;
    return NVMAI_OK;
}

int check_offsets(const nvmai_expert_offsets* o) {
    if (!o) return NVMAI_ERR_INVALID_ARG;
    if ((o->gate_w | o->up_w | o->down_w) & 15u) return NVMAI_ERR_ALIGNMENT;
    if ((o->gate_s | o->gate_b | o->up_s | o->up_b | o->down_s | o->down_b) & 1u) return NVMAI_ERR_ALIGNMENT;
    return NVMAI_OK;
}

void set_phase1(RowsParams& p, const nvmai_expert_offsets& o, uint32_t d, uint32_t f) {
    p.wA = o.gate_w; p.sA = o.gate_s; p.bA = o.gate_b;
    p.wB = o.up_w; p.sB = o.up_s; p.bB = o.up_b;
    p.rows = f; p.n = d;
}

void set_phase2(RowsParams& p, const nvmai_expert_offsets& o, uint32_t d, uint32_t f) {
    p.wA = o.down_w; p.sA = o.down_s; p.bA = o.down_b;
    p.wB = p.sB = p.bB = 0;
    p.rows = d; p.n = f;
}

// chunks of 16 bytes per row of d elements in router format `kind`
uint32_t rows_chunks(int kind, uint32_t d) { return kind == 16 ? d / 8 : (kind == 8 ? d / 16 : d / 32); }

template <int ACT>
void run_router_t(const RouterParams& rp, uint32_t cpl, dim3 grid, hipStream_t s) {
    // the block's token rows (+ the raw row and the inverse norm of the prologue)
    const size_t lds = (size_t)ROUTER_TOK * rp.d * 2 + (rp.pre_weight ? (size_t)rp.d * 2 + 16 : 0);
    if (cpl <= 1) router_logits_kernel<ACT, 1><<<grid, 256, lds, s>>>(rp);
    else if (cpl <= 2) router_logits_kernel<ACT, 2><<<grid, 256, lds, s>>>(rp);
    else if (cpl <= 4) router_logits_kernel<ACT, 4><<<grid, 256, lds, s>>>(rp);
    else router_logits_kernel<ACT, 8><<<grid, 256, lds, s>>>(rp);
}

// d <= 2048 dense / 4096 at 8 bit / 8192 at 4 bit (8 chunks per lane).
template <int ACT>
void run_router_tiled(const RouterParams& rp, const RowsDesc& r, uint32_t n_rows, float* out, uint32_t out_ld,
                      hipStream_t s) {
    const uint32_t cpl = (rows_chunks(r.kind, rp.d) + 31) / 32;
    if (n_rows == 1 && rp.x_vec && cpl <= 8) {      // one row (the shared expert's gate): a half-wave per token, no staging
        const dim3 sgrid((rp.tokens + 7) / 8);
#define NVMAI_SINGLE(KIND)                                                                        \
        do {                                                                                      \
            if (cpl <= 4) router_single_row_kernel<ACT, KIND, 4><<<sgrid, 256, 0, s>>>(rp, r, out, out_ld); \
            else router_single_row_kernel<ACT, KIND, 8><<<sgrid, 256, 0, s>>>(rp, r, out, out_ld);         \
        } while (0)
        if (r.kind == 16) NVMAI_SINGLE(16);
        else if (r.kind == 8) NVMAI_SINGLE(8);
        else NVMAI_SINGLE(4);
#undef NVMAI_SINGLE
        return;
    }
    const size_t lds = (size_t)RT_TOK * rp.d * 2;
    const uint32_t per_block = 8 * (r.kind == 4 ? 2 : 4);
    dim3 grid((n_rows + per_block - 1) / per_block, (rp.tokens + RT_TOK - 1) / RT_TOK);
#define NVMAI_TILED(KIND)                                                                                    \
    do {                                                                                                     \
        if (rp.eff_scale) router_logits_tiled_kernel<ACT, KIND, true><<<grid, 256, lds, s>>>(rp, r, n_rows, out, out_ld);  \
        else router_logits_tiled_kernel<ACT, KIND, false><<<grid, 256, lds, s>>>(rp, r, n_rows, out, out_ld);  \
    } while (0)
    if (r.kind == 16) NVMAI_TILED(16);
    else if (r.kind == 8) NVMAI_TILED(8);
    else NVMAI_TILED(4);
#undef NVMAI_TILED
}

int run_router(int act, RouterParams& rp, hipStream_t s) {
    rp.x_vec = aligned16(rp.x) && (rp.x_stride % 8 == 0);
    // Many tokens (a prefill block): the register-tiled kernel, same logits bit for bit
    if (rp.tokens >= 64 && (size_t)RT_TOK * rp.d * 2 <= 65536) {
        if (act == ACT_BF16) {
            if (rp.num_experts) run_router_tiled<ACT_BF16>(rp, rp.router, rp.num_experts, rp.logits, rp.num_experts, s);
            if (rp.gate.kind) run_router_tiled<ACT_BF16>(rp, rp.gate, 1, rp.gate_logit, 1, s);
        } else {
            if (rp.num_experts) run_router_tiled<ACT_FP16>(rp, rp.router, rp.num_experts, rp.logits, rp.num_experts, s);
            if (rp.gate.kind) run_router_tiled<ACT_FP16>(rp, rp.gate, 1, rp.gate_logit, 1, s);
        }
        return NVMAI_OK;
    }
    uint32_t chunks = rp.router.kind ? rows_chunks(rp.router.kind, rp.d) : 0;
    if (rp.gate.kind) chunks = chunks > rows_chunks(rp.gate.kind, rp.d) ? chunks : rows_chunks(rp.gate.kind, rp.d);
    const uint32_t cpl = (chunks + 31) / 32;
    if (cpl > 8) return NVMAI_ERR_UNSUPPORTED;
    const uint32_t rows = rp.num_experts + (rp.gate.kind ? 1u : 0u);
    dim3 grid((rows + 7) / 8, (rp.tokens + ROUTER_TOK - 1) / ROUTER_TOK);
    if (act == ACT_BF16) run_router_t<ACT_BF16>(rp, cpl, grid, s);
    else run_router_t<ACT_FP16>(rp, cpl, grid, s);
    return NVMAI_OK;
}

int check_rows_desc(const nvmai_rows* r, uint32_t d, bool allow_absent) {
    if (!r || r->kind == 0) return allow_absent ? NVMAI_OK : NVMAI_ERR_INVALID_ARG;
    if (r->kind != 4 && r->kind != 8 && r->kind != 16) return NVMAI_ERR_UNSUPPORTED;
    if (!r->weights || (r->kind != 16 && (!r->scales || !r->biases))) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(r->weights)) return NVMAI_ERR_ALIGNMENT;
    if (d % NVMAI_GROUP) return NVMAI_ERR_INVALID_ARG;
    return NVMAI_OK;
}

RowsDesc to_desc(const nvmai_rows* r) {
    RowsDesc d{};
    if (r && r->kind) { d.w = r->weights; d.s = r->scales; d.b = r->biases; d.kind = r->kind; }
    return d;
}

void run_combine(int act, const CombineParams& cp, hipStream_t s) {
    dim3 grid((cp.d + 255) / 256, cp.tokens);
    if (act == ACT_BF16) combine_kernel<ACT_BF16><<<grid, 256, 0, s>>>(cp);
    else combine_kernel<ACT_FP16><<<grid, 256, 0, s>>>(cp);
}

// Small decode batches in three launches (router logits; gate/up that selects for itself; down
// projection + combine) -- for the shapes both kernels are instantiated for.
// one or two tokens; up to four with 8-bit experts (measured: 36.9 us at three, 46.3 against 48.4 us
// at four tokens; with 4-bit experts four tokens are slower this way, 47 against 42.5 us)
constexpr uint32_t FUSED_DECODE_MAX_TOKENS = 2;

bool fused_decode_ok(uint32_t T, uint32_t K, bool has_shared, uint32_t d, uint32_t f, uint32_t bits) {
    const uint32_t c1 = d * bits / 128, c2 = f * bits / 128;
    return T <= (bits == 8 ? 4u : FUSED_DECODE_MAX_TOKENS) && T * K <= 64 && K + (has_shared ? 1u : 0u) <= 4 * DC_SLOTS_PER_WAVE &&
           (d * bits) % 128 == 0 && (c1 == 64 || c1 == 128) &&
           (f * bits) % 128 == 0 && (c2 == 16 || c2 == 32 || c2 == 64);
}

template <int ACT, int BITS>
void launch_routed_t(RowsParams& p, const SelectParams& sel, const RoutedStats& rs, uint32_t slots, hipStream_t s) {
    const uint32_t chunks = p.n * BITS / 128;
    constexpr uint32_t rows_per_block = 4 * 1 * 1 * 2;       // four waves, SEG 64, RPI 1, ITERS 2
    p.blocks_per_entry = (p.rows + rows_per_block - 1) / rows_per_block;
    const dim3 grid(slots * p.blocks_per_entry, sel.tokens);
    if (chunks == 64)
        expert_rows_routed<ACT, BITS, 64, 1, 1, 2><<<grid, 256, rows_fast_lds_bytes(p.n, 1, 64), s>>>(p, sel, rs);
    else
        expert_rows_routed<ACT, BITS, 64, 2, 1, 2><<<grid, 256, rows_fast_lds_bytes(p.n, 2, 64), s>>>(p, sel, rs);
}

void launch_routed(int act, uint32_t bits, RowsParams& p, const SelectParams& sel, const RoutedStats& rs,
                   uint32_t slots, hipStream_t s) {
    if (act == ACT_BF16) {
        if (bits == 8) launch_routed_t<ACT_BF16, 8>(p, sel, rs, slots, s);
        else launch_routed_t<ACT_BF16, 4>(p, sel, rs, slots, s);
    } else {
        if (bits == 8) launch_routed_t<ACT_FP16, 8>(p, sel, rs, slots, s);
        else launch_routed_t<ACT_FP16, 4>(p, sel, rs, slots, s);
    }
}

template <int ACT, int BITS>
void launch_slots_t(RowsParams& p, const uint32_t* active_slots, uint32_t count, uint32_t top_k, hipStream_t s) {
    const uint32_t chunks = p.n * BITS / 128;
    constexpr uint32_t rows_per_block = 4 * 1 * 1 * 2;       // four waves, SEG 64, RPI 1, ITERS 2
    p.blocks_per_entry = (p.rows + rows_per_block - 1) / rows_per_block;
    const dim3 grid(count * p.blocks_per_entry);
    if (chunks == 64)
        expert_rows_slots<ACT, BITS, 64, 1, 1, 2><<<grid, 256, rows_fast_lds_bytes(p.n, 1, 64), s>>>(p, active_slots, top_k);
    else
        expert_rows_slots<ACT, BITS, 64, 2, 1, 2><<<grid, 256, rows_fast_lds_bytes(p.n, 2, 64), s>>>(p, active_slots, top_k);
}

void launch_slots(int act, uint32_t bits, RowsParams& p, const uint32_t* active_slots, uint32_t count, uint32_t top_k,
                  hipStream_t s) {
    if (act == ACT_BF16) {
        if (bits == 8) launch_slots_t<ACT_BF16, 8>(p, active_slots, count, top_k, s);
        else launch_slots_t<ACT_BF16, 4>(p, active_slots, count, top_k, s);
    } else {
        if (bits == 8) launch_slots_t<ACT_FP16, 8>(p, active_slots, count, top_k, s);
        else launch_slots_t<ACT_FP16, 4>(p, active_slots, count, top_k, s);
    }
}

template <int ACT, int BITS>
void launch_down_combine_t(const DownCombineParams& p, hipStream_t s) {
    const uint32_t chunks = p.n * BITS / 128;
    const dim3 grid((p.rows + DC_ROWS - 1) / DC_ROWS, p.tokens);
    if (chunks == 16) down_combine_kernel<ACT, BITS, 16><<<grid, 256, 0, s>>>(p);
    else if (chunks == 32) down_combine_kernel<ACT, BITS, 32><<<grid, 256, 0, s>>>(p);
    else down_combine_kernel<ACT, BITS, 64><<<grid, 256, 0, s>>>(p);
}

void launch_down_combine(int act, uint32_t bits, const DownCombineParams& p, hipStream_t s) {
    if (act == ACT_BF16) {
        if (bits == 8) launch_down_combine_t<ACT_BF16, 8>(p, s);
        else launch_down_combine_t<ACT_BF16, 4>(p, s);
    } else {
        if (bits == 8) launch_down_combine_t<ACT_FP16, 8>(p, s);
        else launch_down_combine_t<ACT_FP16, 4>(p, s);
    }
}

}  // namespace

// ---------------------------------------------------------------------------
// quantizer
// ---------------------------------------------------------------------------
extern "C" int nvmai_hip_quantize_affine(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* w,
                                         int w_is_bf16, uint32_t rows, uint32_t n, uint32_t bits,
                                         uint8_t* packed, uint16_t* scales, uint16_t* biases) {
    if (!ctx || !w || !packed || !scales || !biases) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (n == 0 || n % NVMAI_GROUP) return NVMAI_ERR_INVALID_ARG;
    if (rows == 0) return NVMAI_OK;
    QuantParams q{w, w_is_bf16, rows, n, bits, packed, scales, biases};
    const uint64_t groups = (uint64_t)rows * (n / NVMAI_GROUP);
    quantize_affine_kernel<<<dim3((uint32_t)((groups + 3) / 4)), dim3(256), 0, (hipStream_t)stream>>>(q);
    return launch_status();
}

extern "C" int nvmai_hip_dequantize_affine(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                           const uint8_t* packed, const uint16_t* scales,
                                           const uint16_t* biases, uint64_t count, uint32_t bits,
                                           uint8_t* codes_out, void* values_out) {
    if (!ctx || !packed) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (values_out && (!scales || !biases)) return NVMAI_ERR_INVALID_ARG;
    if (count % NVMAI_GROUP) return NVMAI_ERR_INVALID_ARG;
    if (count == 0) return NVMAI_OK;
    dim3 grid((uint32_t)((count + 255) / 256));
    if (ctx->act == ACT_BF16)
        dequantize_affine_kernel<ACT_BF16><<<grid, 256, 0, (hipStream_t)stream>>>(packed, scales, biases, count, bits, codes_out, values_out);
    else
        dequantize_affine_kernel<ACT_FP16><<<grid, 256, 0, (hipStream_t)stream>>>(packed, scales, biases, count, bits, codes_out, values_out);
    return launch_status();
}

// ---------------------------------------------------------------------------
// affine GEMV
// ---------------------------------------------------------------------------
namespace {
// x holds activations of the context's type, or fp32 when x_is_f32 (the reference's CPU kernel
// takes fp32 inputs, nvmai_kernels.h:22-28).
int affine_gemv_any(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                    const uint16_t* scales, const uint16_t* biases, uint32_t bits, const void* x,
                    bool x_is_f32, uint32_t x_stride, uint32_t n_tokens, uint32_t m, uint32_t n, void* y,
                    float* y_f32, uint32_t y_stride) {
    if (!ctx || !weights || !scales || !biases || !x || (!y && !y_f32)) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (n == 0 || n % NVMAI_GROUP || x_stride < n || y_stride < m) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(weights) || !aligned16(x) || (x_stride % 8)) return NVMAI_ERR_ALIGNMENT;
    if (m == 0 || n_tokens == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const int maxtok = n_tokens == 1 ? 1 : MAX_TOK;
    const uint32_t ents = (n_tokens + maxtok - 1) / maxtok;
    if (!x_is_f32) {
        RowsParams p{};
        p.src.slot[0] = weights;
        p.sA = reinterpret_cast<const uint8_t*>(scales) - weights;
        p.bA = reinterpret_cast<const uint8_t*>(biases) - weights;
        p.x = x; p.x_stride = x_stride; p.rows = m; p.n = n;
        p.out = y_f32; p.out_stride = y_stride; p.out_act = y; p.out_act_stride = y_stride;
        p.dense_count = n_tokens;
        if (launch_dense_rows(ctx->act, bits, p, maxtok, ents, s)) return launch_status();
    }
    const bool need_tmp = (y != nullptr) || y_stride != m;
    size_t need = ws_round(ents * sizeof(WorkEntry)) + ws_round(16) + 2 * ws_round(n_tokens * 4u) +
                  (need_tmp ? ws_round((size_t)n_tokens * m * 4u) : 0);
    int rc = ws_begin(ctx, stream, need);
    if (rc) return rc;
    WorkEntry* entries = ws_take<WorkEntry>(ctx, ents);
    uint32_t* n_entries = ws_take<uint32_t>(ctx, 4);
    uint32_t* pair_token = ws_take<uint32_t>(ctx, n_tokens);
    uint32_t* pair_id = ws_take<uint32_t>(ctx, n_tokens);
    float* tmp = need_tmp ? ws_take<float>(ctx, (size_t)n_tokens * m) : y_f32;
    dense_entries_kernel<<<(n_tokens + 255) / 256, 256, 0, s>>>(entries, n_entries, pair_token, pair_id,
                                                              n_tokens, (uint32_t)maxtok, 0u);
    RowsParams p{};
    p.src.slot[0] = weights;
    p.entries = entries; p.n_entries = n_entries; p.pair_in = pair_token; p.pair_out = pair_id;
    p.wA = 0;
    p.sA = reinterpret_cast<const uint8_t*>(scales) - weights;
    p.bA = reinterpret_cast<const uint8_t*>(biases) - weights;
    p.x = x; p.x_stride = x_stride; p.out = tmp; p.out_stride = m; p.rows = m; p.n = n;
    launch_rows(ctx->act, bits, false, x_is_f32, p, maxtok, ents, s);
    if (need_tmp) {
        // copy out with the caller's stride (and convert when asked)
        const dim3 grid((m + 255) / 256, n_tokens);
        if (ctx->act == ACT_BF16) store_rows_kernel<ACT_BF16><<<grid, 256, 0, s>>>(tmp, y, y_f32, m, y_stride);
        else store_rows_kernel<ACT_FP16><<<grid, 256, 0, s>>>(tmp, y, y_f32, m, y_stride);
    }
    return launch_status();
}
}  // namespace

extern "C" int nvmai_hip_affine_gemv(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                                     const uint16_t* scales, const uint16_t* biases, uint32_t bits,
                                     const void* x, uint32_t x_stride, uint32_t n_tokens,
                                     uint32_t m, uint32_t n, void* y, float* y_f32,
                                     uint32_t y_stride) {
    if (bits == 16) {                     // dense BF16 rows: the BF16 LM head
        if (!ctx || !weights || !x || (!y && !y_f32)) return NVMAI_ERR_INVALID_ARG;
        return nvmai::dense_bf16_gemv(ctx, (hipStream_t)stream, reinterpret_cast<const uint16_t*>(weights), x, x_stride,
                                      n_tokens, m, n, y, y_f32, y_stride);
    }
    // Five to 32 input rows against a projection-sized matrix: the matrix-core GEMV reads the matrix
    // once for all of them.  (Every block of it stages the inputs for itself, which a matrix of
    // LM-head size pays thousands of times: 165 / 280 us at 16 / 32 rows against 116 us through the
    // dense product below -- so that one keeps the large matrices unless fp32 results are asked for.)
    if (ctx && n_tokens > 4 && n_tokens <= 32 && (m < 32768 || y_f32 || !y) &&
        nvmai::gemv_mfma_ok(weights, scales, biases, bits, x, x_stride, n_tokens, m, n, y, y_f32, y_stride))
        return nvmai::gemv_mfma(ctx, (hipStream_t)stream, weights, scales, biases, bits, x, x_stride, n_tokens, m, n, y,
                                y_f32, y_stride);
    // More than four input rows of a large matrix: the row engine would stream the matrix once per
    // four rows; the matrix-core product reads and dequantizes it once (from five rows on it is
    // the faster of the two at LM-head sizes).  Only where its preconditions hold and 16-bit
    // outputs are all that is asked for.
    // ... and for a matrix with enough column tiles to cover the device: a projection of a few thousand
    // rows gives the product a few dozen blocks, and four passes of the row engine are faster
    // (12,352 x 2048 at 16 rows: 37 us against 13).
    if (ctx && n_tokens > 4 && (m >= 32768 || (n_tokens > 32 && m >= 1024)) && y && !y_f32 && weights && scales && biases && x &&
        (bits == 4 || bits == 8) && n && n % NVMAI_GROUP == 0 && x_stride >= n && y_stride >= m &&
        aligned16(weights) && aligned16(x) && x_stride % 8 == 0 && aligned16(y) &&
        (uint64_t)n_tokens * x_stride * 2 <= 0xFFFFFFFFull && (uint64_t)m * n * bits / 8 <= 0xFFFFFFFFull)
        return nvmai_hip_affine_qmm(ctx, stream, weights, scales, biases, bits, x, x_stride, y, y_stride, n_tokens, m, n);
    return affine_gemv_any(ctx, stream, weights, scales, biases, bits, x, false, x_stride, n_tokens, m, n, y,
                           y_f32, y_stride);
}

namespace {
// The dense rows engine with the residual add + RMSNorm prologue, for the block shapes a projection of
// a decode step takes (up to 16,384 rows of 2048 codes).  False, having launched nothing, otherwise.
template <int ACT, int BITS>
bool launch_dense_prenorm_t(RowsParams& p, int maxtok, hipStream_t s) {
    if ((p.n * BITS) % 128) return false;
    const uint32_t chunks = p.n * BITS / 128;
#define NVMAI_PRE(SEG, NCH, RPI, ITERS)                                                            \
    do {                                                                                           \
        constexpr uint32_t rows_per_block = 4 * (64 / SEG) * RPI * ITERS;                          \
        p.blocks_per_entry = (p.rows + rows_per_block - 1) / rows_per_block;                       \
        const size_t lds = rows_fast_lds_bytes_prenorm(p.n, NCH, SEG);                             \
        const dim3 grid(p.blocks_per_entry);                                                       \
        if (maxtok == 1) expert_rows_fast<ACT, BITS, SEG, NCH, 1, false, false, RPI, ITERS, true, true><<<grid, 256, lds, s>>>(p); \
        else expert_rows_fast<ACT, BITS, SEG, NCH, 4, false, false, RPI, ITERS, true, true><<<grid, 256, lds, s>>>(p);             \
        return true;                                                                               \
    } while (0)
    if (p.rows <= 4096 && chunks == 64) NVMAI_PRE(64, 1, 1, 2);
    if (p.rows <= 4096 && chunks == 128) NVMAI_PRE(64, 2, 1, 2);
    if (p.rows <= 16384 && chunks == 64) NVMAI_PRE(64, 1, 2, 2);
    if (p.rows <= 16384 && chunks == 128) NVMAI_PRE(64, 2, 1, 4);
#undef NVMAI_PRE
    return false;
}
}  // namespace

extern "C" int nvmai_hip_affine_gemv_prenorm(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                                             const uint16_t* scales, const uint16_t* biases, uint32_t bits,
                                             const void* hidden, uint32_t hidden_stride, const void* delta,
                                             uint32_t delta_stride, const uint16_t* norm_weight, float eps,
                                             void* hidden_out, uint32_t hidden_out_stride, void* normed_scratch,
                                             uint32_t normed_stride, uint32_t n_tokens, uint32_t m, uint32_t n, void* y,
                                             uint32_t y_stride) {
    if (!ctx || !weights || !scales || !biases || !hidden || !norm_weight || !hidden_out || !y) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (n == 0 || n % NVMAI_GROUP || hidden_stride < n || hidden_out_stride < n || (delta && delta_stride < n) || y_stride < m)
        return NVMAI_ERR_INVALID_ARG;
    if (m == 0 || n_tokens == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const bool rows16 = aligned16(hidden) && hidden_stride % 8 == 0 && aligned16(hidden_out) && hidden_out_stride % 8 == 0 &&
                        aligned16(norm_weight) && (!delta || (aligned16(delta) && delta_stride % 8 == 0));
    // every block norms the rows for itself when they are few, short and may be moved 16 bytes at a time,
    // and the updated residual rows do not overwrite the ones other blocks still read
    if (n_tokens <= (uint32_t)MAX_TOK && n <= 2048 && rows16 && aligned16(weights) && hidden_out != hidden) {
        RowsParams p{};
        p.src.slot[0] = weights;
        p.sA = reinterpret_cast<const uint8_t*>(scales) - weights;
        p.bA = reinterpret_cast<const uint8_t*>(biases) - weights;
        p.x = hidden; p.x_stride = hidden_stride; p.rows = m; p.n = n;
        p.out = nullptr; p.out_stride = y_stride; p.out_act = y; p.out_act_stride = y_stride;
        p.dense_count = n_tokens;
        p.pre_delta = (const uint16_t*)delta; p.pre_delta_stride = delta_stride; p.pre_weight = norm_weight;
        p.pre_hidden_out = (uint16_t*)hidden_out; p.pre_hidden_stride = hidden_out_stride; p.pre_eps = eps;
        const int maxtok = n_tokens == 1 ? 1 : MAX_TOK;
        const bool done = ctx->act == ACT_BF16
                              ? (bits == 8 ? launch_dense_prenorm_t<ACT_BF16, 8>(p, maxtok, s) : launch_dense_prenorm_t<ACT_BF16, 4>(p, maxtok, s))
                              : (bits == 8 ? launch_dense_prenorm_t<ACT_FP16, 8>(p, maxtok, s) : launch_dense_prenorm_t<ACT_FP16, 4>(p, maxtok, s));
        if (done) return launch_status();
    }
    // otherwise the steps one after the other, through the caller's scratch rows
    if (!normed_scratch || normed_stride < n) return NVMAI_ERR_UNSUPPORTED;
    if (hidden_out != hidden) {
        const hipError_t e = hipMemcpy2DAsync(hidden_out, (size_t)hidden_out_stride * 2, hidden, (size_t)hidden_stride * 2,
                                              (size_t)n * 2, n_tokens, hipMemcpyDeviceToDevice, s);
        if (e != hipSuccess) return NVMAI_ERR_HIP;
    }
    int rc = delta ? nvmai_hip_residual_add_rmsnorm(ctx, stream, hidden_out, hidden_out_stride, delta, delta_stride,
                                                    norm_weight, normed_scratch, normed_stride, n_tokens, n, eps)
                   : nvmai_hip_rmsnorm(ctx, stream, hidden_out, hidden_out_stride, norm_weight, normed_scratch, normed_stride,
                                       n_tokens, n, eps);
    if (rc) return rc;
    return nvmai_hip_affine_gemv(ctx, stream, weights, scales, biases, bits, normed_scratch, normed_stride, n_tokens, m, n, y,
                                 nullptr, y_stride);
}

// The reference's CPU entry point with its own signature (host pointers, fp32 x, out written,
// nothing returned): the operands travel to the device, the GEMV runs there, the result
// travels back, and the call returns when `out` is complete.  A failure cannot be returned,
// so it is reported on stderr and `out` is filled with NaN: never a silently wrong result.
extern "C" void nvmai_int4_affine_gemv(const uint8_t* weights, const uint16_t* scales,
                                       const uint16_t* biases, const float* x, size_t rows, size_t n,
                                       float* out) {
    if (rows == 0) return;
    static nvmai_hip_ctx* host_ctx = nullptr;
    int rc = NVMAI_OK;
    if (!host_ctx) rc = nvmai_hip_ctx_create(0, NVMAI_ACT_BF16, &host_ctx);
    const size_t wb = rows * n / 2, mb = rows * (n / NVMAI_GROUP) * 2;
    uint8_t* dev = nullptr;
    // one allocation: weights | scales | biases | x | out, each 256-byte aligned
    const size_t o_s = ws_round(wb), o_b = o_s + ws_round(mb), o_x = o_b + ws_round(mb), o_y = o_x + ws_round(n * 4);
    if (rc == NVMAI_OK && (!weights || !scales || !biases || !x || !out || n == 0 || n % NVMAI_GROUP ||
                           rows > 0xFFFFFFFFull || n > 0xFFFFFFFFull))
        rc = NVMAI_ERR_INVALID_ARG;
    if (rc == NVMAI_OK && hipMalloc(reinterpret_cast<void**>(&dev), o_y + rows * 4) != hipSuccess) rc = NVMAI_ERR_HIP;
    if (rc == NVMAI_OK &&
        (hipMemcpy(dev, weights, wb, hipMemcpyHostToDevice) != hipSuccess ||
         hipMemcpy(dev + o_s, scales, mb, hipMemcpyHostToDevice) != hipSuccess ||
         hipMemcpy(dev + o_b, biases, mb, hipMemcpyHostToDevice) != hipSuccess ||
         hipMemcpy(dev + o_x, x, n * 4, hipMemcpyHostToDevice) != hipSuccess))
        rc = NVMAI_ERR_HIP;
    if (rc == NVMAI_OK)
        rc = affine_gemv_any(host_ctx, nullptr, dev, reinterpret_cast<const uint16_t*>(dev + o_s),
                             reinterpret_cast<const uint16_t*>(dev + o_b), 4, dev + o_x, true, (uint32_t)n, 1,
                             (uint32_t)rows, (uint32_t)n, nullptr, reinterpret_cast<float*>(dev + o_y),
                             (uint32_t)rows);
    if (rc == NVMAI_OK && hipMemcpy(out, dev + o_y, rows * 4, hipMemcpyDeviceToHost) != hipSuccess) rc = NVMAI_ERR_HIP;
    if (dev) (void)hipFree(dev);
    if (rc != NVMAI_OK) {
        fprintf(stderr, "nvmai_int4_affine_gemv: %s\n", nvmai_hip_status_string(rc));
        if (out) for (size_t r = 0; r < rows; ++r) out[r] = __builtin_nanf("");
    }
}

// ---------------------------------------------------------------------------
// router
// ---------------------------------------------------------------------------
extern "C" int nvmai_hip_moe_router_topk(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                         const nvmai_rows* router, const void* hidden,
                                         uint32_t hidden_stride, uint32_t n_tokens,
                                         const uint16_t* eff_scale, const uint16_t* per_expert_scale,
                                         uint32_t num_experts, uint32_t d, uint32_t top_k,
                                         uint32_t* out_idx, uint16_t* out_w, float* logits_out) {
    if (!ctx || !hidden || !out_idx || !out_w) return NVMAI_ERR_INVALID_ARG;
    int rc = check_rows_desc(router, d, false);
    if (rc) return rc;
    if (num_experts == 0 || num_experts > 64 * TOPK_MAX_PER_LANE) return NVMAI_ERR_INVALID_ARG;
    if (top_k == 0 || top_k > 64 || top_k > num_experts || hidden_stride < d) return NVMAI_ERR_INVALID_ARG;
    if (n_tokens == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    float* logits = logits_out;
    if (!logits) {
        rc = ws_begin(ctx, stream, ws_round((size_t)n_tokens * num_experts * 4));
        if (rc) return rc;
        logits = ws_take<float>(ctx, (size_t)n_tokens * num_experts);
    }
    RouterParams rp{};
    rp.router = to_desc(router);
    rp.x = hidden; rp.eff_scale = eff_scale; rp.x_stride = hidden_stride; rp.tokens = n_tokens;
    rp.num_experts = num_experts; rp.d = d; rp.logits = logits; rp.gate_logit = nullptr;
    rc = run_router(ctx->act, rp, s);
    if (rc) return rc;
    SelectParams sp{logits, per_expert_scale, n_tokens, num_experts, top_k, out_idx, out_w};
    select_topk_kernel<<<(n_tokens + 3) / 4, 256, 0, s>>>(sp);
    return launch_status();
}

// ---------------------------------------------------------------------------
// routed phase 1 / phase 2 over the top-k slot blobs of one token
// ---------------------------------------------------------------------------
namespace {

int slots_prologue(nvmai_hip_ctx* ctx, const void* const* blobs, const nvmai_expert_offsets* off,
                   uint32_t bits, uint32_t d, uint32_t f, uint32_t top_k, RowsParams& p) {
    if (!ctx || !blobs) return NVMAI_ERR_INVALID_ARG;
    int rc = check_shape(d, f, bits);
    if (rc) return rc;
    rc = check_offsets(off);
    if (rc) return rc;
    if (top_k == 0 || top_k > 8) return NVMAI_ERR_INVALID_ARG;   // MoE.swift:455-458 requires 8
    for (uint32_t i = 0; i < top_k; ++i) {
        if (!blobs[i]) return NVMAI_ERR_INVALID_ARG;
        if (!aligned16(blobs[i])) return NVMAI_ERR_ALIGNMENT;
        p.src.slot[i] = (const uint8_t*)blobs[i];
    }
    return NVMAI_OK;
}

}  // namespace

extern "C" int nvmai_hip_moe_phase1_gate_up_act_subset(
    nvmai_hip_ctx* ctx, nvmai_stream stream, const void* const* blobs,
    const nvmai_expert_offsets* off, uint32_t bits, const void* x, float* acts, uint32_t d,
    uint32_t f, uint32_t top_k, const uint32_t* active_slots, uint32_t active_count) {
    RowsParams p{};
    int rc = slots_prologue(ctx, blobs, off, bits, d, f, top_k, p);
    if (rc) return rc;
    if (!x || !acts || (active_count && !active_slots) || active_count > top_k) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(x) || !aligned16(acts)) return NVMAI_ERR_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    {   // one launch where the row engine has a short-block instantiation: the entries are made in the kernel
        const uint32_t c1 = d * bits / 128;
        if ((d * bits) % 128 == 0 && (c1 == 64 || c1 == 128)) {
            const uint32_t n = active_slots ? active_count : top_k;
            if (n == 0) return NVMAI_OK;
            set_phase1(p, *off, d, f);
            p.x = x; p.x_stride = d; p.out = acts; p.out_stride = f;
            launch_slots(ctx->act, bits, p, active_slots, n, top_k, s);
            return launch_status();
        }
    }
    rc = ws_begin(ctx, stream, ws_round(8 * sizeof(WorkEntry)) + 3 * ws_round(64));
    if (rc) return rc;
    WorkEntry* entries = ws_take<WorkEntry>(ctx, 8);
    uint32_t* n_entries = ws_take<uint32_t>(ctx, 4);
    uint32_t* pair_token = ws_take<uint32_t>(ctx, 8);
    uint32_t* pair_id = ws_take<uint32_t>(ctx, 8);
    uint32_t count = active_slots ? active_count : top_k;
    if (active_slots) {
        subset_entries_kernel<<<1, 64, 0, s>>>(entries, n_entries, pair_token, pair_id, active_slots,
                                              active_count, top_k);
    } else {
        // dense over the slots: entry i -> slot i, input row 0, output row i
        slot_entries_kernel<<<1, 64, 0, s>>>(entries, n_entries, pair_token, pair_id, top_k, 0);
    }
    p.entries = entries; p.n_entries = n_entries; p.pair_in = pair_token; p.pair_out = pair_id;
    set_phase1(p, *off, d, f);
    p.x = x; p.x_stride = d; p.out = acts; p.out_stride = f;
    launch_rows(ctx->act, bits, true, false, p, 1, count, s);
    return launch_status();
}

extern "C" int nvmai_hip_moe_phase1_gate_up_act(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                                const void* const* blobs,
                                                const nvmai_expert_offsets* off, uint32_t bits,
                                                const void* x, float* acts, uint32_t d, uint32_t f,
                                                uint32_t top_k) {
    return nvmai_hip_moe_phase1_gate_up_act_subset(ctx, stream, blobs, off, bits, x, acts, d, f, top_k,
                                                   nullptr, 0);
}

extern "C" int nvmai_hip_moe_phase2_down_reduce(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                                const void* const* blobs,
                                                const nvmai_expert_offsets* off, uint32_t bits,
                                                const float* acts, const uint16_t* routing_w,
                                                const void* residual, void* y, uint32_t d, uint32_t f,
                                                uint32_t top_k) {
    RowsParams p{};
    int rc = slots_prologue(ctx, blobs, off, bits, d, f, top_k, p);
    if (rc) return rc;
    if (!acts || !routing_w || !y) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(acts)) return NVMAI_ERR_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    {   // one launch (down projection of every slot + weighted sum) where that kernel is instantiated
        const uint32_t c2 = f * bits / 128;
        if ((f * bits) % 128 == 0 && (c2 == 16 || c2 == 32 || c2 == 64)) {
            DownCombineParams dc{};
            dc.src = p.src;
            dc.wA = off->down_w; dc.sA = off->down_s; dc.bA = off->down_b;
            dc.acts = acts; dc.idx = nullptr; dc.w = routing_w; dc.residual = residual; dc.res_stride = d;
            dc.gate_logit = nullptr; dc.has_shared = 0; dc.tokens = 1; dc.top_k = top_k; dc.rows = d; dc.n = f;
            dc.y_stride = d; dc.y = y;
            launch_down_combine(ctx->act, bits, dc, s);
            return launch_status();
        }
    }
    rc = ws_begin(ctx, stream, ws_round(8 * sizeof(WorkEntry)) + 3 * ws_round(64) + ws_round((size_t)top_k * d * 4));
    if (rc) return rc;
    WorkEntry* entries = ws_take<WorkEntry>(ctx, 8);
    uint32_t* n_entries = ws_take<uint32_t>(ctx, 4);
    uint32_t* pair_in = ws_take<uint32_t>(ctx, 8);
    uint32_t* pair_id = ws_take<uint32_t>(ctx, 8);
    float* partials = ws_take<float>(ctx, (size_t)top_k * d);
    slot_entries_kernel<<<1, 64, 0, s>>>(entries, n_entries, pair_in, pair_id, top_k, 1);
    p.entries = entries; p.n_entries = n_entries; p.pair_in = pair_in; p.pair_out = pair_id;
    set_phase2(p, *off, d, f);
    p.x = acts; p.x_stride = f; p.out = partials; p.out_stride = d;
    launch_rows(ctx->act, bits, false, true, p, 1, top_k, s);
    CombineParams cp{};
    cp.partials = partials; cp.w = routing_w; cp.residual = residual; cp.gate_logit = nullptr;
    cp.has_shared = 0; cp.tokens = 1; cp.top_k = top_k; cp.d = d; cp.res_stride = d; cp.y_stride = d;
    cp.y = y;
    run_combine(ctx->act, cp, s);
    return launch_status();
}

// ---------------------------------------------------------------------------
// shared expert
// ---------------------------------------------------------------------------
extern "C" int nvmai_hip_shared_expert(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* blob,
                                       const nvmai_expert_offsets* off, uint32_t bits,
                                       const nvmai_rows* shared_gate, const void* x,
                                       uint32_t x_stride, uint32_t n_tokens, void* y,
                                       uint32_t y_stride, uint32_t d, uint32_t f) {
    if (!ctx || !blob || !x || !y) return NVMAI_ERR_INVALID_ARG;
    int rc = check_shape(d, f, bits);
    if (rc) return rc;
    rc = check_offsets(off);
    if (rc) return rc;
    rc = check_rows_desc(shared_gate, d, true);
    if (rc) return rc;
    if (x_stride < d || y_stride < d) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(blob) || !aligned16(x) || (x_stride % 8)) return NVMAI_ERR_ALIGNMENT;
    if (n_tokens == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    // A block of tokens (prefill): the expert's matrices are read once for all of them by the
    // grouped-GEMM kernels instead of once per four tokens (the reference runs its dense QMM
    // there, MPPPrefillInt4QMM.swift:18-128).  Operands past the kernels' 32-bit offsets, and
    // small batches (the two ways cost the same at about 200 tokens), take the row engine below.
    if (n_tokens >= 192 && (uint64_t)n_tokens * x_stride * 2 <= 0xFFFFFFFFull &&
        (uint64_t)n_tokens * d * 2 <= 0xFFFFFFFFull && (uint64_t)d * f * bits / 8 <= 0xFFFFFFFFull) {
        const bool gated_d = shared_gate && shared_gate->kind;
        rc = ws_begin(ctx, stream, ws_round((size_t)n_tokens * f * 2) + ws_round((size_t)n_tokens * d * 2) +
                               ws_round(n_tokens * 4u) + ws_round(16));
        if (rc) return rc;
        uint16_t* act = ws_take<uint16_t>(ctx, (size_t)n_tokens * f);
        uint16_t* tmp = ws_take<uint16_t>(ctx, (size_t)n_tokens * d);
        float* gate_logit = ws_take<float>(ctx, n_tokens);
        float* dummy_logits = ws_take<float>(ctx, 4);
        if (gated_d) {
            RouterParams rp{};
            rp.gate = to_desc(shared_gate);
            rp.x = x; rp.x_stride = x_stride; rp.tokens = n_tokens; rp.num_experts = 0; rp.d = d;
            rp.logits = dummy_logits; rp.gate_logit = gate_logit;
            rc = run_router(ctx->act, rp, s);
            if (rc) return rc;
        }
        return nvmai::expert_ffn_dense(ctx, s, (const uint8_t*)blob, off, bits, x, x_stride, n_tokens, d, f, act, tmp,
                                       gated_d ? gate_logit : nullptr, y, y_stride);
    }
    const int maxtok = n_tokens == 1 ? 1 : MAX_TOK;
    const uint32_t ents = (n_tokens + maxtok - 1) / maxtok;
    // A handful of tokens: gate logit, gate/up with its entries made in the kernel, and the down
    // projection with the gate applied in its epilogue -- three launches (two without a gate)
    // instead of five.  The down kernel reads the matrix once per token, hence the limit.
    {
        const uint32_t c1 = d * bits / 128, c2 = f * bits / 128;
        if (n_tokens <= 4 && (d * bits) % 128 == 0 && (c1 == 64 || c1 == 128) && (f * bits) % 128 == 0 &&
            (c2 == 16 || c2 == 32 || c2 == 64)) {
            const bool gated_s = shared_gate && shared_gate->kind;
            rc = ws_begin(ctx, stream, ws_round((size_t)n_tokens * f * 4) + ws_round(n_tokens * 4u) + ws_round(16));
            if (rc) return rc;
            float* acts = ws_take<float>(ctx, (size_t)n_tokens * f);
            float* gate_logit = ws_take<float>(ctx, n_tokens);
            float* dummy_logits = ws_take<float>(ctx, 4);
            if (gated_s) {
                RouterParams rp{};
                rp.gate = to_desc(shared_gate);
                rp.x = x; rp.x_stride = x_stride; rp.tokens = n_tokens; rp.num_experts = 0; rp.d = d;
                rp.logits = dummy_logits; rp.gate_logit = gate_logit;
                rc = run_router(ctx->act, rp, s);
                if (rc) return rc;
            }
            RowsParams p{};
            p.src.slot[0] = (const uint8_t*)blob;
            set_phase1(p, *off, d, f);
            p.x = x; p.x_stride = x_stride; p.out = acts; p.out_stride = f; p.dense_count = n_tokens;
            if (launch_dense_dual(ctx->act, bits, p, maxtok, ents, s)) {
                DownCombineParams dc{};
                dc.src.slot[8] = (const uint8_t*)blob;
                dc.wA = off->down_w; dc.sA = off->down_s; dc.bA = off->down_b;
                dc.acts = acts; dc.gate_logit = gated_s ? gate_logit : nullptr;
                dc.has_shared = 1; dc.tokens = n_tokens; dc.top_k = 0; dc.rows = d; dc.n = f;
                dc.y_stride = y_stride; dc.y = y;
                launch_down_combine(ctx->act, bits, dc, s);
                return launch_status();
            }
        }
    }
    size_t need = ws_round(ents * sizeof(WorkEntry)) + ws_round(16) + 2 * ws_round(n_tokens * 4u) +
                  ws_round((size_t)n_tokens * f * 4) + ws_round((size_t)n_tokens * d * 4) +
                  ws_round(n_tokens * 4u) + ws_round(16);
    rc = ws_begin(ctx, stream, need);
    if (rc) return rc;
    WorkEntry* entries = ws_take<WorkEntry>(ctx, ents);
    uint32_t* n_entries = ws_take<uint32_t>(ctx, 4);
    uint32_t* pair_token = ws_take<uint32_t>(ctx, n_tokens);
    uint32_t* pair_id = ws_take<uint32_t>(ctx, n_tokens);
    float* acts = ws_take<float>(ctx, (size_t)n_tokens * f);
    float* partials = ws_take<float>(ctx, (size_t)n_tokens * d);
    float* gate_logit = ws_take<float>(ctx, n_tokens);
    float* dummy_logits = ws_take<float>(ctx, 4);
    dense_entries_kernel<<<(n_tokens + 255) / 256, 256, 0, s>>>(entries, n_entries, pair_token, pair_id,
                                                              n_tokens, (uint32_t)maxtok, 8u);
    const bool gated = shared_gate && shared_gate->kind;
    if (gated) {
        RouterParams rp{};
        rp.gate = to_desc(shared_gate);
        rp.x = x; rp.x_stride = x_stride; rp.tokens = n_tokens; rp.num_experts = 0; rp.d = d;
        rp.logits = dummy_logits; rp.gate_logit = gate_logit;
        rc = run_router(ctx->act, rp, s);
        if (rc) return rc;
    }
    RowsParams p{};
    p.src.slot[8] = (const uint8_t*)blob;
    p.entries = entries; p.n_entries = n_entries; p.pair_in = pair_token; p.pair_out = pair_id;
    set_phase1(p, *off, d, f);
    p.x = x; p.x_stride = x_stride; p.out = acts; p.out_stride = f;
    launch_rows(ctx->act, bits, true, false, p, maxtok, ents, s);
    RowsParams q = p;
    set_phase2(q, *off, d, f);
    q.pair_in = pair_id;
    q.x = acts; q.x_stride = f; q.out = partials; q.out_stride = d;
    launch_rows(ctx->act, bits, false, true, q, maxtok, ents, s);
    CombineParams cp{};
    cp.partials = partials; cp.w = nullptr; cp.residual = nullptr;
    cp.gate_logit = gated ? gate_logit : nullptr;
    cp.has_shared = 1; cp.tokens = n_tokens; cp.top_k = 0; cp.d = d; cp.res_stride = 0;
    cp.y_stride = y_stride; cp.y = y;
    run_combine(ctx->act, cp, s);
    return launch_status();
}

// ---------------------------------------------------------------------------
// fused decode layer
// ---------------------------------------------------------------------------
namespace {

// Intermediate buffers of a decode step, cut from one block by a bump pointer.
struct Carver {
    uint8_t* base;
    size_t used;
    template <typename T>
    T* take(size_t count) {
        T* p = reinterpret_cast<T*>(base + used);
        used += ws_round(count * sizeof(T));
        return p;
    }
};

// The residual add + RMSNorm that opens the MoE block, done by the router launch (every block of it
// norms its token row for itself) instead of a launch of its own.  x of the layer call is then the
// residual stream; the normed rows land in `normed` for the launches that follow.
struct PreNorm {
    const void* delta; uint32_t delta_stride;      // may be null: norm only
    const uint16_t* weight; float eps;
    void* hidden_out; uint32_t hidden_out_stride;
    void* normed; uint32_t normed_stride;
};

// After the block: stream += y, next = rmsnorm(stream) * weight (the residual add that closes the layer
// and the norm that opens the next one).
struct PostNorm {
    void* stream; uint32_t stream_stride;
    const uint16_t* weight; float eps;
    void* next; uint32_t next_stride;
    bool done;                                     // set when the combine launch took it along
};

// fixed_ws == nullptr: the buffers come from the context's workspace (grown when needed);
// otherwise from the fixed_cap bytes at fixed_ws, and a step that needs more is refused.
int decode_layer_impl(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_moe_layer* L, const void* x,
                      uint32_t x_stride, uint32_t n_tokens, void* y, uint32_t y_stride, uint32_t* out_idx,
                      uint16_t* out_w, uint32_t* stats, uint8_t* fixed_ws, size_t fixed_cap,
                      const PreNorm* pre = nullptr, PostNorm* post = nullptr) {
    if (!ctx || !L || !x || !y) return NVMAI_ERR_INVALID_ARG;
    int rc = check_shape(L->d, L->f, L->bits);
    if (rc) return rc;
    rc = check_offsets(&L->offsets);
    if (rc) return rc;
    rc = check_rows_desc(&L->router, L->d, false);
    if (rc) return rc;
    rc = check_rows_desc(&L->shared_gate, L->d, true);
    if (rc) return rc;
    const uint32_t T = n_tokens, K = L->top_k, E = L->num_experts, D = L->d, F = L->f;
    if (E == 0 || E > 64 * TOPK_MAX_PER_LANE || K == 0 || K > 64 || K > E) return NVMAI_ERR_INVALID_ARG;
    if (!L->experts_base || x_stride < D || y_stride < D) return NVMAI_ERR_INVALID_ARG;
    if ((uint64_t)T * K > 4096) return NVMAI_ERR_INVALID_ARG;   // work list is built in LDS
    if (!aligned16(L->experts_base) || (L->expert_stride & 15u) || !aligned16(x) || (x_stride % 8) ||
        (L->shared_blob && !aligned16(L->shared_blob)))
        return NVMAI_ERR_ALIGNMENT;
    if (T == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const bool has_shared = L->shared_blob != nullptr;
    const bool gated = has_shared && L->shared_gate.kind != 0;
    const int maxtok = T == 1 ? 1 : MAX_TOK;
    const uint32_t pairs = T * K;
    const uint32_t rows_total = pairs + (has_shared ? T : 0);
    uint32_t routed_ents = pairs;
    if (maxtok > 1) routed_ents = pairs < E + pairs / maxtok ? pairs : E + pairs / maxtok;
    const uint32_t max_entries = routed_ents + (has_shared ? (T + maxtok - 1) / maxtok : 0);
    size_t need = ws_round((size_t)T * E * 4) + ws_round(T * 4u) + ws_round(pairs * 4u) +
                  ws_round(pairs * 2u) + ws_round(max_entries * sizeof(WorkEntry)) + ws_round(16) +
                  2 * ws_round(rows_total * 4u) + ws_round((size_t)rows_total * F * 4) +
                  ws_round((size_t)rows_total * D * 4);
    Carver cv{fixed_ws, 0};
    if (fixed_ws) {
        if (need > fixed_cap) return NVMAI_ERR_SCRATCH;
    } else {
        rc = ws_begin(ctx, stream, need);
        if (rc) return rc;
        cv.base = ctx->ws;
    }
    float* logits = cv.take<float>((size_t)T * E);
    float* gate_logit = cv.take<float>(T);
    uint32_t* idx = cv.take<uint32_t>(pairs);
    uint16_t* wts = cv.take<uint16_t>(pairs);
    WorkEntry* entries = cv.take<WorkEntry>(max_entries);
    uint32_t* n_entries = cv.take<uint32_t>(4);
    uint32_t* pair_token = cv.take<uint32_t>(rows_total);
    uint32_t* pair_id = cv.take<uint32_t>(rows_total);
    float* acts = cv.take<float>((size_t)rows_total * F);
    float* partials = cv.take<float>((size_t)rows_total * D);
    if (out_idx) idx = out_idx;
    if (out_w) wts = out_w;

    RouterParams rp{};
    rp.router = to_desc(&L->router);
    if (gated) rp.gate = to_desc(&L->shared_gate);
    rp.x = x; rp.eff_scale = L->eff_scale; rp.x_stride = x_stride; rp.tokens = T;
    rp.num_experts = E; rp.d = D; rp.logits = logits; rp.gate_logit = gate_logit;
    if (pre) {
        rp.pre_delta = (const uint16_t*)pre->delta; rp.pre_delta_stride = pre->delta_stride;
        rp.pre_weight = pre->weight; rp.pre_eps = pre->eps;
        rp.pre_hidden_out = (uint16_t*)pre->hidden_out; rp.pre_hidden_stride = pre->hidden_out_stride;
        rp.pre_normed_out = (uint16_t*)pre->normed; rp.pre_normed_stride = pre->normed_stride;
        x = pre->normed; x_stride = pre->normed_stride;     // what the expert launches read
    }
    SelectParams sp{logits, L->per_expert_scale, T, E, K, idx, wts};
    GroupParams gp{sp, (uint32_t)maxtok, has_shared ? 1 : 0, entries, n_entries, stats, pair_token, pair_id,
                   ctx->tickets};
    if (fused_decode_ok(T, K, has_shared, D, F, L->bits)) {
        { ProfScope ps(ctx, NVMAI_PROF_ROUTER, s); rc = run_router(ctx->act, rp, s); }
        if (rc) return rc;
        RowsParams p{};
        p.src.pool_base = (const uint8_t*)L->experts_base;
        p.src.pool_stride = L->expert_stride;
        p.src.slot[8] = (const uint8_t*)L->shared_blob;
        set_phase1(p, L->offsets, D, F);
        p.x = x; p.x_stride = x_stride; p.out = acts; p.out_stride = F;
        const RoutedStats rs{stats, has_shared ? 1 : 0};
        {
            ProfScope ps(ctx, NVMAI_PROF_PHASE1, s);
            launch_routed(ctx->act, L->bits, p, sp, rs, K + (has_shared ? 1u : 0u), s);
        }
        DownCombineParams dc{};
        dc.src = p.src;
        dc.wA = L->offsets.down_w; dc.sA = L->offsets.down_s; dc.bA = L->offsets.down_b;
        dc.acts = acts; dc.idx = idx; dc.w = wts; dc.gate_logit = gated ? gate_logit : nullptr;
        dc.has_shared = has_shared ? 1 : 0; dc.tokens = T; dc.top_k = K; dc.rows = D; dc.n = F;
        dc.y_stride = y_stride; dc.y = y;
        { ProfScope ps(ctx, NVMAI_PROF_PHASE2, s); launch_down_combine(ctx->act, L->bits, dc, s); }
        return launch_status();
    }
    // Two launches on purpose: one that also selects and groups in its last blocks needs a
    // device-scope release (an L2 write-back on this multi-die part) from every one of its
    // hundreds of producer blocks, and measured 18 us slower per step.
    { ProfScope ps(ctx, NVMAI_PROF_ROUTER, s); rc = run_router(ctx->act, rp, s); }
    if (rc) return rc;
    {
        ProfScope ps(ctx, NVMAI_PROF_GROUP, s);
        if (T <= 4) select_group_one_block_kernel<<<1, 256, (4 * E + 8 + pairs) * 4, s>>>(gp);
        else select_group_kernel<<<(T + 3) / 4, 256, (4 * E + 8 + pairs) * 4, s>>>(gp);
    }

    RowsParams p{};
    p.src.pool_base = (const uint8_t*)L->experts_base;
    p.src.pool_stride = L->expert_stride;
    p.src.slot[8] = (const uint8_t*)L->shared_blob;
    p.entries = entries; p.n_entries = n_entries; p.pair_in = pair_token; p.pair_out = pair_id;
    set_phase1(p, L->offsets, D, F);
    p.x = x; p.x_stride = x_stride; p.out = acts; p.out_stride = F;
    { ProfScope ps(ctx, NVMAI_PROF_PHASE1, s); launch_rows(ctx->act, L->bits, true, false, p, maxtok, max_entries, s); }
    RowsParams q = p;
    set_phase2(q, L->offsets, D, F);
    q.pair_in = pair_id;
    q.x = acts; q.x_stride = F; q.out = partials; q.out_stride = D;
    { ProfScope ps(ctx, NVMAI_PROF_PHASE2, s); launch_rows(ctx->act, L->bits, false, true, q, maxtok, max_entries, s); }
    CombineParams cp{};
    cp.partials = partials; cp.w = wts; cp.residual = nullptr; cp.gate_logit = gated ? gate_logit : nullptr;
    cp.has_shared = has_shared ? 1 : 0; cp.tokens = T; cp.top_k = K; cp.d = D; cp.res_stride = 0;
    cp.y_stride = y_stride; cp.y = y;
    if (post && D % 8 == 0 && D <= 8 * 256 * ROUTER_PRE_PIECES && aligned16(post->stream) && post->stream_stride % 8 == 0 &&
        aligned16(post->next) && post->next_stride % 8 == 0 && aligned16(post->weight) && aligned16(y) && y_stride % 8 == 0) {
        // the combine, the residual add and the next norm in one launch, one block per token
        const PostNormArgs pa{(uint16_t*)post->stream, post->stream_stride, post->weight, post->eps, (uint16_t*)post->next, post->next_stride};
        ProfScope ps(ctx, NVMAI_PROF_COMBINE, s);
        if (ctx->act == ACT_BF16) combine_postnorm_kernel<ACT_BF16><<<T, 256, D * 2, s>>>(cp, pa);
        else combine_postnorm_kernel<ACT_FP16><<<T, 256, D * 2, s>>>(cp, pa);
        post->done = true;
        return launch_status();
    }
    { ProfScope ps(ctx, NVMAI_PROF_COMBINE, s); run_combine(ctx->act, cp, s); }
    return launch_status();
}

}  // namespace

extern "C" int nvmai_hip_moe_decode_layer(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                          const nvmai_moe_layer* L, const void* x, uint32_t x_stride,
                                          uint32_t n_tokens, void* y, uint32_t y_stride,
                                          uint32_t* out_idx, uint16_t* out_w, uint32_t* stats) {
    return decode_layer_impl(ctx, stream, L, x, x_stride, n_tokens, y, y_stride, out_idx, out_w, stats, nullptr, 0);
}

extern "C" int nvmai_hip_moe_decode_layer_prenorm(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_moe_layer* L,
                                                  const void* hidden, uint32_t hidden_stride, const void* delta,
                                                  uint32_t delta_stride, const uint16_t* norm_weight, float eps,
                                                  void* hidden_out, uint32_t hidden_out_stride, void* normed,
                                                  uint32_t normed_stride, uint32_t n_tokens, void* y,
                                                  uint32_t y_stride, uint32_t* out_idx, uint16_t* out_w,
                                                  uint32_t* stats) {
    if (!ctx || !L || !hidden || !norm_weight || !hidden_out || !normed || !y) return NVMAI_ERR_INVALID_ARG;
    const uint32_t D = L->d;
    if (hidden_stride < D || hidden_out_stride < D || normed_stride < D || (delta && delta_stride < D))
        return NVMAI_ERR_INVALID_ARG;
    if (n_tokens == 0) return NVMAI_OK;
    const bool rows16 = aligned16(hidden) && hidden_stride % 8 == 0 && aligned16(hidden_out) && hidden_out_stride % 8 == 0 &&
                        aligned16(normed) && normed_stride % 8 == 0 && aligned16(norm_weight) && D % 8 == 0 &&
                        (!delta || (aligned16(delta) && delta_stride % 8 == 0));
    // the router launch norms for itself when it is the per-token kernel, the rows can be moved 16 bytes
    // at a time and the updated residual rows do not overwrite the ones other blocks still read
    if (n_tokens < 64 && rows16 && D <= 8192 && hidden_out != hidden && normed != hidden && normed != hidden_out) {
        const PreNorm pre{delta, delta_stride, norm_weight, eps, hidden_out, hidden_out_stride, normed, normed_stride};
        return decode_layer_impl(ctx, stream, L, hidden, hidden_stride, n_tokens, y, y_stride, out_idx, out_w, stats,
                                 nullptr, 0, &pre);
    }
    // otherwise the two steps one after the other
    if (hidden_out != hidden) {
        const hipError_t e = hipMemcpy2DAsync(hidden_out, (size_t)hidden_out_stride * 2, hidden, (size_t)hidden_stride * 2,
                                              (size_t)D * 2, n_tokens, hipMemcpyDeviceToDevice, (hipStream_t)stream);
        if (e != hipSuccess) return NVMAI_ERR_HIP;
    }
    int rc = delta ? nvmai_hip_residual_add_rmsnorm(ctx, stream, hidden_out, hidden_out_stride, delta, delta_stride,
                                                    norm_weight, normed, normed_stride, n_tokens, D, eps)
                   : nvmai_hip_rmsnorm(ctx, stream, hidden_out, hidden_out_stride, norm_weight, normed, normed_stride,
                                       n_tokens, D, eps);
    if (rc) return rc;
    return decode_layer_impl(ctx, stream, L, normed, normed_stride, n_tokens, y, y_stride, out_idx, out_w, stats, nullptr, 0);
}

// The block of a layer between two norms: residual add + norm before it (as the entry point above), and
// after it the residual add that closes the layer with the norm that opens the next one:
// hidden_out += y, next_normed = rmsnorm(hidden_out) * next_norm_weight.  With the work-list path
// (five tokens or more) the last of these rides in the combine launch; otherwise it is the
// residual-add-norm kernel after the block.  Same bits as the separate calls either way.
extern "C" int nvmai_hip_moe_decode_layer_norms(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_moe_layer* L,
                                                const void* hidden, uint32_t hidden_stride, const void* delta,
                                                uint32_t delta_stride, const uint16_t* norm_weight, float eps,
                                                void* hidden_out, uint32_t hidden_out_stride, void* normed,
                                                uint32_t normed_stride, uint32_t n_tokens, void* y, uint32_t y_stride,
                                                uint32_t* out_idx, uint16_t* out_w, uint32_t* stats,
                                                const uint16_t* next_norm_weight, void* next_normed,
                                                uint32_t next_normed_stride) {
    if (!ctx || !L || !hidden || !norm_weight || !hidden_out || !normed || !y || !next_norm_weight || !next_normed)
        return NVMAI_ERR_INVALID_ARG;
    const uint32_t D = L->d;
    if (hidden_stride < D || hidden_out_stride < D || normed_stride < D || next_normed_stride < D || (delta && delta_stride < D))
        return NVMAI_ERR_INVALID_ARG;
    if (n_tokens == 0) return NVMAI_OK;
    const bool rows16 = aligned16(hidden) && hidden_stride % 8 == 0 && aligned16(hidden_out) && hidden_out_stride % 8 == 0 &&
                        aligned16(normed) && normed_stride % 8 == 0 && aligned16(norm_weight) && D % 8 == 0 &&
                        (!delta || (aligned16(delta) && delta_stride % 8 == 0));
    PostNorm post{hidden_out, hidden_out_stride, next_norm_weight, eps, next_normed, next_normed_stride, false};
    int rc;
    if (n_tokens < 64 && rows16 && D <= 8192 && hidden_out != hidden && normed != hidden && normed != hidden_out &&
        next_normed != hidden_out && next_normed != y) {
        const PreNorm pre{delta, delta_stride, norm_weight, eps, hidden_out, hidden_out_stride, normed, normed_stride};
        rc = decode_layer_impl(ctx, stream, L, hidden, hidden_stride, n_tokens, y, y_stride, out_idx, out_w, stats,
                               nullptr, 0, &pre, &post);
    } else {
        rc = nvmai_hip_moe_decode_layer_prenorm(ctx, stream, L, hidden, hidden_stride, delta, delta_stride, norm_weight, eps,
                                                hidden_out, hidden_out_stride, normed, normed_stride, n_tokens, y, y_stride,
                                                out_idx, out_w, stats);
    }
    if (rc || post.done) return rc;
    return nvmai_hip_residual_add_rmsnorm(ctx, stream, hidden_out, hidden_out_stride, y, y_stride, next_norm_weight,
                                          next_normed, next_normed_stride, n_tokens, D, eps);
}

extern "C" size_t nvmai_hip_moe_decode_layer_noalloc_scratch_bytes(void) { return STATIC_SCRATCH_BYTES; }

// The same step with its intermediate buffers in the library's static device array: no hipMalloc,
// no hipFree, no memset, nothing but kernel launches.  The array's device address was fetched when
// the context was created; every call on a device shares that device's one array.
extern "C" int nvmai_hip_moe_decode_layer_noalloc(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                                  const nvmai_moe_layer* L, const void* x, uint32_t x_stride,
                                                  uint32_t n_tokens, void* y, uint32_t y_stride,
                                                  uint32_t* out_idx, uint16_t* out_w, uint32_t* stats) {
    if (!ctx) return NVMAI_ERR_INVALID_ARG;
    if (!ctx->static_scratch) return NVMAI_ERR_HIP;     // the symbol lookup failed at context creation
    // every device holds its own copy of the array at its own address: the address this context keeps is
    // only good while its device is the current one
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != ctx->device) return NVMAI_ERR_INVALID_ARG;
    return decode_layer_impl(ctx, stream, L, x, x_stride, n_tokens, y, y_stride, out_idx, out_w, stats,
                             ctx->static_scratch, STATIC_SCRATCH_BYTES);
}
