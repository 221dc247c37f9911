// Pieces shared by the row kernels (dynamic quant, RMSNorm, LayerNorm and their quantising forms):
// block reductions, the exact reciprocal-based division and the torch-exact quantisation steps.
#pragma once

#include "fnn_common.h"

// every rounding of the reference's fp32 arithmetic is kept: no contraction into fmas
#pragma clang fp contract(off)

namespace fnn {

constexpr int kRowThreads = 256;

// Block reductions over the four waves of a workgroup.  `red` serves ONE reduction per kernel (nothing
// guards it against being written again while a slow wave still reads it): every kernel here reduces once
// through each of its arrays.
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__device__ __forceinline__ double block_sum(double v, double* red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// two sums at once (one pair of barriers)
__device__ __forceinline__ void block_sum2(double& a, double& b, double* red) {
    a = wave_sum(a);
    b = wave_sum(b);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { red[w] = a; red[4 + w] = b; }
    __syncthreads();
    a = (red[0] + red[1]) + (red[2] + red[3]);
    b = (red[4] + red[5]) + (red[6] + red[7]);
}

// Correctly rounded fp32 quotient x / s from r = RN(1/s) (one IEEE division per row):
// q0 = RN(x*r) is within 2 ulp, e = x - s*q0 is exact in an fma, and RN(q0 + e*r) is the rounded
// quotient (Markstein).  Three instructions instead of the ~10 of a full division sequence.
__device__ __forceinline__ float div_by(float x, float s, float r) {
    const float q0 = x * r;
    const float e = __builtin_fmaf(-q0, s, x);
    return __builtin_fmaf(e, r, q0);
}

// q = round_half_even(round_DT(x / s)) with x/s a correctly rounded fp32 division.
template <int DT> __device__ __forceinline__ int quant_in_dtype(float x, float s, float r) {
    // pinned: the last fma of the division must round to fp32 before the conversion rounds again
    // (fused into v_fma_mixlo_f16 it would round once)
    const float t = rounded_f32(div_by(x, s, r));
    const float th = bits_to_f32<DT>(f32_to_bits<DT>(t));
    return (int)rintf(th);
}

// The same with the result left as an integer-valued float (for the packing below).
template <int DT> __device__ __forceinline__ float quant_in_dtype_f(float x, float s, float r) {
    const float t = rounded_f32(div_by(x, s, r));
    return rintf(bits_to_f32<DT>(f32_to_bits<DT>(t)));
}

// Reciprocal to hand to div_by: 1/s, or 0 for an all-zero row, whose quotients then come out as 0
// instead of 0 * inf (so the per-element test for s == 0 can go).
__device__ __forceinline__ float quant_rcp(float s) { return s == 0.f ? 0.f : 1.0f / s; }

// Byte j of w <- the integer-valued float r as int8, saturated to [-128, 127]: r + 128 is exact, lands in
// [0, 255] as an unsigned byte, and v_cvt_pk_u8_f32 saturates, converts and inserts it in one instruction
// (conversion, clamp and packing took five).  The finished dword still needs its sign bits flipped:
// w ^ 0x80808080.  Used by every quantising kernel: the norm + quant layers clamp in the reference, and plain
// dynamic quantisation is clamped here as well (a bf16 row whose scale rounded down reaches 128, which an
// unclamped cast wraps to -128).
__device__ __forceinline__ uint32_t put_biased_byte(float r, int j, uint32_t w) {
    return __builtin_amdgcn_cvt_pk_u8_f32(r + 128.f, (uint32_t)j, w);
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xFF) | ((uint32_t)(b & 0xFF) << 8) | ((uint32_t)(c & 0xFF) << 16) |
           ((uint32_t)(d & 0xFF) << 24);
}

__device__ __forceinline__ int quant_clamped(float n, float s, float rcp) {
    float r = rintf(div_by(n, s, rcp));
    r = fminf(fmaxf(r, -128.f), 127.f);
    return s == 0.f ? 0 : (int)r;
}

// 8 consecutive gamma values as fp32 (vector loads; the type branch is uniform)
__device__ __forceinline__ void load_gamma8(const void* gamma, int gamma_dtype, int64_t first, float g[8]) {
    if (gamma_dtype == FNN_F32) {
        const v4f a = *(const v4f*)((const float*)gamma + first);
        const v4f b = *(const v4f*)((const float*)gamma + first + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) { g[j] = a[j]; g[4 + j] = b[j]; }
    } else {
        const v4u a = *(const v4u*)((const uint16_t*)gamma + first);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = a[j] & 0xFFFFu, hi = a[j] >> 16;
            g[2 * j] = gamma_dtype == FNN_F16 ? f16_bits_to_f32(lo) : bf16_bits_to_f32(lo);
            g[2 * j + 1] = gamma_dtype == FNN_F16 ? f16_bits_to_f32(hi) : bf16_bits_to_f32(hi);
        }
    }
}

// Vector kernels keep a whole row in registers: up to kRowMaxNV x 8 values per thread (rows of up
// to 40960 values), 16-byte aligned rows.
constexpr int kRowMaxNV = 20;
inline bool vec_ok(const void* x, const void* q, int64_t K, int64_t ldx, int64_t ldq) {
    return K % 8 == 0 && K <= 8 * kRowThreads * kRowMaxNV && ldx % 8 == 0 && ldq % 8 == 0 &&
           ((uintptr_t)x % 16) == 0 && ((uintptr_t)q % 8) == 0;
}

// Launches KERNEL<..., NV, ...> with the smallest NV of the list that holds `nv` vectors per thread.
#define FNN_ROW_DISPATCH_NV(nv, LAUNCH)                   \
    do {                                                  \
        if ((nv) <= 1) { LAUNCH(1); }                     \
        else if ((nv) <= 2) { LAUNCH(2); }                \
        else if ((nv) <= 4) { LAUNCH(4); }                \
        else if ((nv) <= 8) { LAUNCH(8); }                \
        else if ((nv) <= 12) { LAUNCH(12); }              \
        else if ((nv) <= 16) { LAUNCH(16); }              \
        else { LAUNCH(20); }                              \
    } while (0)


}  // namespace fnn
