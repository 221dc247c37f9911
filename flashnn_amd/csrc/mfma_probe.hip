// Measurement aid: the rate at which this GPU sustains back-to-back int8 MFMAs when nothing else
// runs - no loads, no LDS, operands held in registers.  The chip's clock follows its power draw,
// and the draw of the matrix cores follows how many operand bits toggle between instructions, so
// the rate is measured for operands of random bytes (what a GEMM on quantised data feeds them) and
// for constant operands (which reach the datasheet rate).  The A8W8 kernels are judged against the
// datasheet peak; this number says how much of the gap any kernel can close.
#include <hip/hip_runtime.h>

#include "fnn_common.h"

namespace fnn {

typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(256) void mfma_rate_kernel(int* __restrict__ sink, int random_operands, int iters) {
    // four operand pairs, used in turn: consecutive MFMAs see different bytes, as in a GEMM
    v4i a[4], b[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t id = (threadIdx.x * 4 + q) * 8 + j;
            a[q][j] = random_operands ? (int)mix32(2 * id + 1) : 0x01010101;
            b[q][j] = random_operands ? (int)mix32(2 * id + 0x9e3779b9u) : 0x01010101;
        }
    v16i c[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) c[q][r] = 0;
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int q = 0; q < 4; ++q) c[q] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q], b[q], c[q], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += c[q][r];
    if (s == 0x5a5a5a5a && iters < 0) sink[0] = s;   // never true: keeps the accumulators alive
}

}  // namespace fnn

extern "C" int fnn_debug_mfma_rate(void* sink, int random_operands, int iters, int launches,
                                   double* tops, void* stream) {
    using namespace fnn;
    if (!sink || !tops || iters <= 0 || launches <= 0) {
        set_error("fnn_debug_mfma_rate: bad argument");
        return FNN_ERR_ARG;
    }
    hipStream_t st = (hipStream_t)stream;
    int dev = 0, cus = 0;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        set_error("fnn_debug_mfma_rate: %s", hipGetErrorString(hipGetLastError()));
        return FNN_ERR_HIP;
    }
    const int wgs = cus * 2;   // two waves per SIMD: one alone leaves issue gaps between dependent MFMAs
    mfma_rate_kernel<<<wgs, 256, 0, st>>>((int*)sink, random_operands, iters);   // warm-up
    (void)hipEventRecord(e0, st);
    for (int l = 0; l < launches; ++l) mfma_rate_kernel<<<wgs, 256, 0, st>>>((int*)sink, random_operands, iters);
    (void)hipEventRecord(e1, st);
    float ms = 0.f;
    const hipError_t err = hipEventSynchronize(e1) == hipSuccess ? hipEventElapsedTime(&ms, e0, e1) : hipGetLastError();
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess || ms <= 0.f) {
        set_error("fnn_debug_mfma_rate: %s", hipGetErrorString(err));
        return FNN_ERR_HIP;
    }
    // 32x32x32 MFMA = 2 * 32^3 operations; 4 waves per workgroup, 4 MFMAs per iteration
    *tops = (double)wgs * 4 * 4 * (double)iters * launches * 65536.0 / ((double)ms * 1e-3) * 1e-12;
    return FNN_OK;
}
