// Host side of the matrix-core GEMV for 5 .. 32 input rows.
#include "ctx.hpp"
#include "gemv_mfma_kernels.hpp"

namespace nvmai {

bool gemv_mfma_ok(const uint8_t* w, const uint16_t* s, const uint16_t* b, uint32_t bits, const void* x,
                  uint32_t x_stride, uint32_t n_tokens, uint32_t m, uint32_t n, const void* y, const float* y_f32,
                  uint32_t y_stride) {
    return w && s && b && x && (y || y_f32) && (bits == 4 || bits == 8) && n_tokens >= 1 && n_tokens <= 32 && m >= 1 &&
           n >= GM_STAGE_CODES && n % GM_STAGE_CODES == 0 && x_stride >= n && x_stride % 8 == 0 && y_stride >= m &&
           aligned16(w) && aligned16(s) && aligned16(b) && aligned16(x) &&
           (uint64_t)m * n * bits / 8 <= 0x7FFFFFFFull;           // 32-bit row offsets, signed record count
}

int gemv_mfma(nvmai_hip_ctx* ctx, hipStream_t s, const uint8_t* w, const uint16_t* scales, const uint16_t* biases,
              uint32_t bits, const void* x, uint32_t x_stride, uint32_t n_tokens, uint32_t m, uint32_t n, void* y,
              float* y_f32, uint32_t y_stride) {
    if (!ctx || !gemv_mfma_ok(w, scales, biases, bits, x, x_stride, n_tokens, m, n, y, y_f32, y_stride))
        return NVMAI_ERR_INVALID_ARG;
    GemvMfmaParams p{w, scales, biases, (const uint16_t*)x, x_stride, n_tokens, m, n, (uint16_t*)y, y_f32, y_stride};
    // rows per block: 64 for a large matrix, 32 or 16 where that would leave compute units without a block
    const int wr = m >= 8192 ? 4 : m >= 4096 ? 2 : 1;
    const dim3 grid((m + 16 * wr - 1) / (16 * wr));
    // eight waves per block for 4-bit rows (8-bit rows would need 200 KB of LDS for them)
#define NVMAI_GM_N(ACT, BITS, TT, NW)                                                          \
    do {                                                                                       \
        if (wr == 4) gemv_mfma_kernel<ACT, BITS, TT, 4, NW><<<grid, 64 * NW, 0, s>>>(p);       \
        else if (wr == 2) gemv_mfma_kernel<ACT, BITS, TT, 2, NW><<<grid, 64 * NW, 0, s>>>(p);  \
        else gemv_mfma_kernel<ACT, BITS, TT, 1, NW><<<grid, 64 * NW, 0, s>>>(p);               \
    } while (0)
#define NVMAI_GM_T(ACT, BITS, TT)                                                              \
    do {                                                                                       \
        NVMAI_GM_N(ACT, BITS, TT, (BITS == 4 ? 8 : 4));                                        \
    } while (0)
#define NVMAI_GM(ACT, BITS)                                                                    \
    do {                                                                                       \
        if (n_tokens <= 16) NVMAI_GM_T(ACT, BITS, 1); else NVMAI_GM_T(ACT, BITS, 2);           \
    } while (0)
    if (ctx->act == ACT_BF16) { if (bits == 8) NVMAI_GM(ACT_BF16, 8); else NVMAI_GM(ACT_BF16, 4); }
    else { if (bits == 8) NVMAI_GM(ACT_FP16, 8); else NVMAI_GM(ACT_FP16, 4); }
#undef NVMAI_GM_T
#undef NVMAI_GM_N
#undef NVMAI_GM
    return launch_status();
}

}  // namespace nvmai
