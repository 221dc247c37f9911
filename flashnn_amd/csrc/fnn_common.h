// Shared device/host helpers for the flashnn_amd HIP kernels (gfx950 / CDNA4 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/flashnn_hip.h"

namespace fnn {

constexpr int kWave = 64;  // CDNA wavefront width

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// ---- 16-bit float <-> fp32 on raw bit patterns -------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// round-to-nearest-even through the hardware conversion (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    const v2bf t = __builtin_convertvector(v2f{f, f}, v2bf);
    return __builtin_bit_cast(uint32_t, t) & 0xFFFFu;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    union { uint16_t u; _Float16 f; } c;
    c.u = (uint16_t)h;
    return (float)c.f;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    union { uint16_t u; _Float16 f; } c;
    c.f = (_Float16)f;  // v_cvt_f16_f32, round-to-nearest-even
    return c.u;
}

// Pins an fp32 value: the compiler otherwise fuses a multiplication with the conversion that
// follows it into v_fma_mixlo_f16, which rounds once where the reference rounds twice.
__device__ __forceinline__ float rounded_f32(float f) {
    asm volatile("" : "+v"(f));
    return f;
}

template <int DT> __device__ __forceinline__ float bits_to_f32(uint32_t h) {
    if constexpr (DT == FNN_F16) return f16_bits_to_f32(h);
    else return bf16_bits_to_f32(h);
}
template <int DT> __device__ __forceinline__ uint32_t f32_to_bits(float f) {
    if constexpr (DT == FNN_F16) return f32_to_f16_bits(f);
    else return f32_to_bf16_bits(f);
}

// Load element i of an array whose element type is only known at run time (uniform branch).
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dtype) {
    if (dtype == FNN_F32) return ((const float*)p)[i];
    uint32_t h = ((const uint16_t*)p)[i];
    return dtype == FNN_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}

__device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v, int dtype) {
    if (dtype == FNN_F32) ((float*)p)[i] = v;
    else ((uint16_t*)p)[i] = (uint16_t)(dtype == FNN_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v));
}

// ---- wave / block reductions -------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// ---- host side ----------------------------------------------------------------------
void set_error(const char* fmt, ...);

// Brackets the launches of one entry point: construct before the first launch, return done() after the
// last.  done() reports an error only if the thread's last HIP error changed in between, and only then
// takes it off the thread: an error that the caller's own HIP calls left before this call is neither
// reported as ours nor cleared.  (A launch failing with the very code already pending goes unseen.)
struct Call {
    const char* fn;
    hipError_t prior;
    explicit Call(const char* fn);
    int done() const;
};

// Raises a kernel's dynamic-LDS limit to the 160 KB of a gfx950 CU, once per device: `raised` is the launch
// site's own bit mask of the devices done (function attributes are kept per device).
void allow_large_lds(const void* kernel, std::atomic<uint64_t>& raised);

// Records the kernel a launch site is about to run, with up to three numbers that tell its variants apart
// (tile rows, tile columns, waves ...): fnn_last_kernel() returns the last one noted on the calling thread.
// With FLASHNN_HIP_LOG=1 in the environment the first launch of every variant prints one line on stderr.
// `name` must be a string literal (it is kept by pointer).
void note_kernel(const char* name, int a = 0, int b = 0, int c = 0);

inline bool is16(int dt) { return dt == FNN_F16 || dt == FNN_BF16; }
inline bool isflt(int dt) { return dt == FNN_F16 || dt == FNN_BF16 || dt == FNN_F32; }

}  // namespace fnn
