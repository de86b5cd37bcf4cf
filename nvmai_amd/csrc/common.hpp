// Device helpers shared by every kernel file: 16-bit float conversions,
// wave64 reductions through DPP, packed-code unpacking.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#define NVMAI_GROUP 64
#define NVMAI_WAVE 64

namespace nvmai {

// ---- 16-bit activations ---------------------------------------------------
// Activations are stored as raw 16-bit patterns; ACT selects the format.
enum ActType : int { ACT_BF16 = 0, ACT_FP16 = 1 };

__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}

// Round-to-nearest-even on the upper 16 bits, no NaN special case: the same
// integer formula as Quantization.swift:17-23 of the reference.
__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t bits = __float_as_uint(x);
    uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7FFFu + lsb) >> 16);
}

__device__ __forceinline__ float f16_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// Round an fp32 value to fp16 (v_cvt_f16_f32, nearest even) as a step of its own.  The empty asm
// hides where x came from: left to itself the compiler folds "round(a * b)" into v_fma_mixlo_f16,
// which rounds the exact product once instead of rounding the fp32 product again -- in some kernels
// and not in others, so that two kernels written with the same arithmetic differ in the last bit
// of about one element in eight thousand.
__device__ __forceinline__ uint16_t f32_to_f16(float x) {
    asm("" : "+v"(x));
    return __builtin_bit_cast(uint16_t, (_Float16)x);
}

template <int ACT>
__device__ __forceinline__ float act_to_f32(uint16_t v) {
    return ACT == ACT_BF16 ? bf16_to_f32(v) : f16_to_f32(v);
}

template <int ACT>
__device__ __forceinline__ uint16_t f32_to_act(float v) {
    return ACT == ACT_BF16 ? f32_to_bf16(v) : f32_to_f16(v);
}

// Two packed activations in one dword -> two floats (low half first).
template <int ACT>
__device__ __forceinline__ void act2_to_f32(uint32_t w, float& lo, float& hi) {
    if (ACT == ACT_BF16) {
        lo = __uint_as_float(w << 16);
        hi = __uint_as_float(w & 0xFFFF0000u);
    } else {
        lo = f16_to_f32((uint16_t)(w & 0xFFFFu));
        hi = f16_to_f32((uint16_t)(w >> 16));
    }
}

// ---- DPP reductions ---------------------------------------------------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, true));
}

// Sum over aligned segments of SEG lanes (SEG = 4, 8, 16, 32 or 64).  Up to 16
// lanes every lane of the segment ends with the segment sum; for SEG 32 and 64
// the sum is valid in the LAST lane of each segment only.
template <int SEG>
__device__ __forceinline__ float seg_reduce_sum(float v) {
    static_assert(SEG == 4 || SEG == 8 || SEG == 16 || SEG == 32 || SEG == 64, "SEG");
    v += dpp_mov<0xB1, 0xF>(v);                  // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E, 0xF>(v);                  // quad_perm [2,3,0,1]
    if (SEG >= 8) v += dpp_mov<0x141, 0xF>(v);   // row_half_mirror
    if (SEG >= 16) v += dpp_mov<0x140, 0xF>(v);  // row_mirror
    if (SEG >= 32) v += dpp_mov<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    if (SEG >= 64) v += dpp_mov<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return v;
}

// Wave-wide max / min through the same DPP ladder; lanes a step does not reach
// keep their own value (bound_ctrl off, old = own value), result broadcast.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_keep(int v) {
    return __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xF, false);
}

__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, __int_as_float(dpp_keep<0xB1, 0xF>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_keep<0x4E, 0xF>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_keep<0x141, 0xF>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_keep<0x140, 0xF>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_keep<0x142, 0xA>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_keep<0x143, 0xC>(__float_as_int(v))));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    v = min(v, (uint32_t)dpp_keep<0xB1, 0xF>((int)v));
    v = min(v, (uint32_t)dpp_keep<0x4E, 0xF>((int)v));
    v = min(v, (uint32_t)dpp_keep<0x141, 0xF>((int)v));
    v = min(v, (uint32_t)dpp_keep<0x140, 0xF>((int)v));
    v = min(v, (uint32_t)dpp_keep<0x142, 0xA>((int)v));
    v = min(v, (uint32_t)dpp_keep<0x143, 0xC>((int)v));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// Lane of a SEG-lane segment that holds seg_reduce_sum's result.
template <int SEG>
__device__ __forceinline__ bool seg_result_lane(int lane) {
    return SEG <= 16 ? (lane % SEG) == 0 : (lane % SEG) == SEG - 1;
}

__device__ __forceinline__ float wave_sum_bcast(float v) {
    v = seg_reduce_sum<64>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float readlane_f(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Butterfly exchange, any power-of-two distance below 64.
__device__ __forceinline__ float shfl_xor_f(float v, int mask) {
    return __shfl_xor(v, mask, 64);
}
__device__ __forceinline__ uint32_t shfl_xor_u(uint32_t v, int mask) {
    return (uint32_t)__shfl_xor((int)v, mask, 64);
}

// ---- packed codes -----------------------------------------------------------
// 4 codes of one dword at 8 bits -> floats, element order = byte order.
__device__ __forceinline__ void unpack8(uint32_t w, float* q) {
    q[0] = (float)(w & 0xFFu);
    q[1] = (float)((w >> 8) & 0xFFu);
    q[2] = (float)((w >> 16) & 0xFFu);
    q[3] = (float)(w >> 24);
}

// unpack4 with the two nibble masks kept as they are written: two ANDs and a shift isolate
// the codes as bytes, and each code is then one byte-to-float conversion.  (Left to itself the
// compiler folds the masks into one bit-field extract per code, twice the instructions.)
__device__ __forceinline__ void unpack4_bytes(uint32_t w, float* q) {
    uint32_t lo = w & 0x0F0F0F0Fu;          // elements 0,2,4,6
    uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;   // elements 1,3,5,7
#if defined(__HIP_DEVICE_COMPILE__)          // the host pass parses this body too and knows no "v" registers
    asm("" : "+v"(lo));
    asm("" : "+v"(hi));
#endif
    q[0] = (float)(lo & 0xFFu);
    q[1] = (float)(hi & 0xFFu);
    q[2] = (float)((lo >> 8) & 0xFFu);
    q[3] = (float)((hi >> 8) & 0xFFu);
    q[4] = (float)((lo >> 16) & 0xFFu);
    q[5] = (float)((hi >> 16) & 0xFFu);
    q[6] = (float)(lo >> 24);
    q[7] = (float)(hi >> 24);
}

// 8 codes of one dword at 4 bits -> floats, element j at bits 4j..4j+3
// (element 2k in the low nibble of byte k).
__device__ __forceinline__ void unpack4(uint32_t w, float* q) {
    uint32_t lo = w & 0x0F0F0F0Fu;          // elements 0,2,4,6
    uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;   // elements 1,3,5,7
    q[0] = (float)(lo & 0xFFu);
    q[1] = (float)(hi & 0xFFu);
    q[2] = (float)((lo >> 8) & 0xFFu);
    q[3] = (float)((hi >> 8) & 0xFFu);
    q[4] = (float)((lo >> 16) & 0xFFu);
    q[5] = (float)((hi >> 16) & 0xFFu);
    q[6] = (float)(lo >> 24);
    q[7] = (float)(hi >> 24);
}

// Codes per 16-byte chunk.
// ---- RMSNorm pieces shared by the norm kernels and the kernels that norm their own input ------
// Sum of squares in a stated order: lane l runs acc = fma(x, x, acc) over the elements l, l + 64,
// ..., then this xor butterfly 32, 16, 8, 4, 2, 1; mean, sqrt and the divide are single IEEE steps.
__device__ __forceinline__ float rms_wave_sum(float acc) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc = __fadd_rn(acc, shfl_xor_f(acc, off));
    return acc;
}

__device__ __forceinline__ float rms_inverse(float sum, uint32_t d, float eps) {
    const float mean = __fdiv_rn(sum, (float)d);
    return __fdiv_rn(1.0f, sqrtf(__fadd_rn(mean, eps)));     // sqrtf: correctly rounded (the _rn intrinsic is not)
}

template <int BITS>
struct Chunk { static constexpr int elems = 128 / BITS; };

// Unpack one 16-byte chunk into Chunk<BITS>::elems floats.
template <int BITS>
__device__ __forceinline__ void unpack_chunk(const uint4& w, float* q) {
    if (BITS == 8) {
        unpack8(w.x, q); unpack8(w.y, q + 4); unpack8(w.z, q + 8); unpack8(w.w, q + 12);
    } else {
        unpack4_bytes(w.x, q); unpack4_bytes(w.y, q + 8); unpack4_bytes(w.z, q + 16); unpack4_bytes(w.w, q + 24);
    }
}

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// silu through the hardware exp2 and reciprocal (about 1e-6 relative): for kernels
// whose result is rounded to 16 bits or compared at 1e-3.
__device__ __forceinline__ float silu_fast(float v) {
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

}  // namespace nvmai
