// Measurement aid: the rate at which this GPU sustains back-to-back int8 MFMAs when nothing else
// runs - no loads, no LDS, operands held in registers.  The chip's clock follows its power draw,
// and the draw of the matrix cores follows how many operand bits toggle between instructions, so
// the rate is measured for operands of random bytes (what a GEMM on quantised data feeds them) and
// for constant operands (which reach the datasheet rate).  The A8W8 kernels are judged against the
// datasheet peak; this number says how much of the gap any kernel can close.
//
// Built into libfnn_probe.so, a library of its own that only bench.py loads: it creates events and waits
// for them, which the product library never does.
//   int fnn_probe_mfma_rate(void* sink, int random_operands, int iters, int launches, double* tops,
//                           void* stream);
// returns 0, or a hipError_t; sink: 4 bytes of device memory (never written); *tops: 1e12 int8
// operations per second over `launches` kernels of `iters` loop iterations on `stream`.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fnn {

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

// The MFMA shape and order of the tiled A8W8 kernel's 256x192 tile: per wave 6 weight fragments against
// 8 activation fragments of v_mfma_i32_16x16x64_i8, the weight fragment fixed over the inner loop.  (The
// shape matters: on random bytes the device sustains about 4.0 POP/s of these and about 3.35 POP/s of
// v_mfma_i32_32x32x32_i8 in the same order.)
__global__ __launch_bounds__(256) void mfma_rate_kernel(int* __restrict__ sink, int random_operands, int iters) {
    constexpr int FN = 6, FM = 8;
    v4i wf[FN], af[FM];
#pragma unroll
    for (int q = 0; q < FN; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            wf[q][j] = random_operands ? (int)mix32(2 * ((threadIdx.x * 8 + q) * 8 + j) + 1) : 0x01010101;
#pragma unroll
    for (int q = 0; q < FM; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            af[q][j] = random_operands ? (int)mix32(2 * ((threadIdx.x * 8 + q) * 8 + j) + 0x9e3779b9u) : 0x01010101;
    v4i c[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j) c[i][j] = v4i{0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < FN; ++i)
#pragma unroll
            for (int j = 0; j < FM; ++j)
                // (written as asm: around the builtin the compiler shuffles the loop-carried accumulators
                // through a hundred register moves per iteration)
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c[i][j]) : "v"(wf[i]), "v"(af[j]));
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) s += c[i][j][r];
    if (s == 0x5a5a5a5a && iters < 0) sink[0] = s;   // never true: keeps the accumulators alive
}

}  // namespace fnn

extern "C" int fnn_probe_mfma_rate(void* sink, int random_operands, int iters, int launches,
                                   double* tops, void* stream) {
    using namespace fnn;
    if (!sink || !tops || iters <= 0 || launches <= 0) return (int)hipErrorInvalidValue;
    hipStream_t st = (hipStream_t)stream;
    int dev = 0, cus = 0;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t err = hipGetDevice(&dev);
    if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err == hipSuccess) err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err != hipSuccess) return (int)err;
    const int wgs = cus;   // one wave per SIMD, as in the tiled kernel; the 48 MFMAs of an iteration are independent
    mfma_rate_kernel<<<wgs, 256, 0, st>>>((int*)sink, random_operands, iters);   // warm-up
    (void)hipEventRecord(e0, st);
    for (int l = 0; l < launches; ++l) mfma_rate_kernel<<<wgs, 256, 0, st>>>((int*)sink, random_operands, iters);
    (void)hipEventRecord(e1, st);
    float ms = 0.f;
    err = hipEventSynchronize(e1);
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return (int)err;
    if (ms <= 0.f) return (int)hipErrorUnknown;
    // 16x16x64 MFMA = 2 * 16 * 16 * 64 operations; 4 waves per workgroup, 48 MFMAs per iteration
    *tops = (double)wgs * 4 * 48 * (double)iters * launches * 32768.0 / ((double)ms * 1e-3) * 1e-12;
    return 0;
}
