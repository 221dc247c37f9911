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

// ---- what the memory side delivers, without arithmetic
// (1) The copy pattern of the tiled A8W8 kernel's 256x192 tile alone: per slab of K, 448 rows x 128 bytes go
// from global memory into the LDS rings by direct-to-LDS loads, 14 per wave and slab, one barrier per slab -
// no fragment reads, no MFMAs.  One workgroup per CU.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

__global__ __launch_bounds__(256) void copy_rate_kernel(const char* __restrict__ src, int64_t rows, int64_t ld,
                                                        int slabs, int tiles, int* __restrict__ sink) {
    // as in the kernel: 256 a-rows in two stages, copied one slab ahead; 192 b-rows in three stages, two ahead
    constexpr int RA = 256, RB = 192, NLA = RA / 32, NLB = RB / 32;   // a wave-load covers 8 rows of 128 bytes; 4 waves
    __shared__ __attribute__((aligned(1024))) char sa[2][RA * 128];
    __shared__ __attribute__((aligned(1024))) char sb[3][RB * 128];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t off[NLA];
#pragma unroll
    for (int j = 0; j < NLA; ++j) off[j] = (uint32_t)(((j * 4 + wave) * 8 + (lane >> 3)) * ld + (lane & 7) * 16);
    for (int t = 0; t < tiles; ++t) {
        // the kernel's sharing: the 32 workgroups of an XCD (ids of equal id & 7) are 8 tile rows x 4 tile
        // columns; an a-tile is read by 4 of them, a b-tile by 8, through that XCD's L2
        const int xcd = blockIdx.x & 7, x = (blockIdx.x >> 3) & 31;
        const int64_t set = (((int64_t)(blockIdx.x >> 8) * tiles + t) * 8 + xcd) * (8 * RA + 4 * RB) % (rows - (8 * RA + 4 * RB));
        const char* a = src + (set + (x >> 2) * RA) * ld;
        const char* b = src + (set + 8 * RA + (x & 3) * RB) * ld;
        auto copy_a = [&](int kt) {
#pragma unroll
            for (int j = 0; j < NLA; ++j)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(a + (int64_t)kt * 128 + off[j]),
                                                 (lds_ptr_t)(sa[kt & 1] + (j * 4 + wave) * 1024), 16, 0, 0);
        };
        auto copy_b = [&](int kt) {
#pragma unroll
            for (int j = 0; j < NLB; ++j)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(b + (int64_t)kt * 128 + off[j]),
                                                 (lds_ptr_t)(sb[kt % 3] + (j * 4 + wave) * 1024), 16, 0, 0);
        };
        copy_a(0);
        copy_b(0);
        copy_b(1);
        for (int kt = 0; kt < slabs; ++kt) {
            // slab kt has landed when everything but the newest b-copies has
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0x0070 | (NLB & 15));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            copy_a(min(kt + 1, slabs - 1));
            copy_b(min(kt + 2, slabs - 1));
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();
    }
    if (slabs < 0) sink[0] = sa[0][threadIdx.x] + sb[0][threadIdx.x];   // never true: keeps the rings alive
}

// (2) A stream of contiguous kilobytes per wave-load with 9 non-temporal 16-byte loads per lane in flight, 8 waves
// per workgroup, one workgroup per CU, each wave walking its own range: the request pattern of the decode
// GEMV on packed weights with the arithmetic taken out.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void stream_rate_kernel(const v4u* __restrict__ src, int64_t vecs_per_wave, int* __restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6);
    const v4u* p = src + wave * vecs_per_wave + lane;
    v4u acc = v4u{0, 0, 0, 0};
    v4u buf[9];
#pragma unroll
    for (int b = 0; b < 9; ++b) buf[b] = __builtin_nontemporal_load(p + b * 64);
    for (int64_t i = 9 * 64; i + 9 * 64 <= vecs_per_wave; i += 9 * 64) {
#pragma unroll
        for (int b = 0; b < 9; ++b) {
            acc ^= buf[b];
            buf[b] = __builtin_nontemporal_load(p + i + b * 64);
        }
    }
#pragma unroll
    for (int b = 0; b < 9; ++b) acc ^= buf[b];
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5a5a5a5au && vecs_per_wave < 0) sink[0] = 1;   // never true
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

// Times `launches` kernels between two events on `stream`; returns milliseconds in *ms.
template <typename F>
static int time_launches(F&& launch, int launches, void* stream, float* ms) {
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err != hipSuccess) return (int)err;
    launch();   // warm-up
    (void)hipEventRecord(e0, st);
    for (int l = 0; l < launches; ++l) launch();
    (void)hipEventRecord(e1, st);
    err = hipEventSynchronize(e1);
    if (err == hipSuccess) err = hipEventElapsedTime(ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err == hipSuccess) err = hipGetLastError();
    return (int)err;
}

// src: `bytes` of device memory read as rows of `ld` bytes (ld a multiple of 128, at least slabs * 128; at
// least 8192 rows, less than 4 GiB); every workgroup copies `tiles` tiles of 448 rows x slabs x 128 bytes.  *gbps_per_cu: bytes a
// CU took in per second, in 1e9.
extern "C" int fnn_probe_copy_rate(const void* src, size_t bytes, int64_t ld, int slabs, int tiles, int launches,
                                   void* sink, double* gbps_per_cu, void* stream) {
    using namespace fnn;
    if (!src || !sink || !gbps_per_cu || ld < 128 || ld % 128 != 0 || slabs < 2 || (int64_t)slabs * 128 > ld || tiles <= 0 ||
        launches <= 0 || bytes / (size_t)ld < 8192 || (bytes / (size_t)ld) * (size_t)ld >= (1ull << 32))
        return (int)hipErrorInvalidValue;
    int dev = 0, cus = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess) return (int)err;
    const int64_t rows = (int64_t)(bytes / (size_t)ld);
    float ms = 0.f;
    const int rc = time_launches([&] {
        copy_rate_kernel<<<cus, 256, 0, (hipStream_t)stream>>>((const char*)src, rows, ld, slabs, tiles, (int*)sink);
    }, launches, stream, &ms);
    if (rc != 0) return rc;
    if (ms <= 0.f) return (int)hipErrorUnknown;
    *gbps_per_cu = 448.0 * 128.0 * slabs * tiles * launches / ((double)ms * 1e-3) * 1e-9;
    return 0;
}

// src: `bytes` of device memory (a multiple of 16); the waves of one workgroup per CU split it evenly.
// *tbps: bytes read per second, in 1e12, launch gaps included.
extern "C" int fnn_probe_stream_rate(const void* src, size_t bytes, int launches, void* sink, double* tbps, void* stream) {
    using namespace fnn;
    if (!src || !sink || !tbps || launches <= 0 || ((uintptr_t)src % 16) != 0) return (int)hipErrorInvalidValue;
    int dev = 0, cus = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess) return (int)err;
    const int64_t waves = (int64_t)cus * 8;
    const int64_t per_wave = (int64_t)(bytes / 16) / waves / (9 * 64) * (9 * 64);     // whole rounds of 9 loads
    if (per_wave < 9 * 64) return (int)hipErrorInvalidValue;
    float ms = 0.f;
    const int rc = time_launches([&] {
        stream_rate_kernel<<<cus, 512, 0, (hipStream_t)stream>>>((const v4u*)src, per_wave, (int*)sink);
    }, launches, stream, &ms);
    if (rc != 0) return rc;
    if (ms <= 0.f) return (int)hipErrorUnknown;
    *tbps = (double)per_wave * 16.0 * waves * launches / ((double)ms * 1e-3) * 1e-12;
    return 0;
}
