// Row kernels: per-token dynamic int8 quantisation and fused RMSNorm + quantisation.
//
// One 256-thread workgroup owns one row.  The row is read from HBM once (16-byte loads)
// and kept in VGPRs across the reduction(s), so the HBM traffic is the algorithmic
// 2*K bytes in + K bytes out per row.  Rows that cannot use 16-byte accesses (K not a
// multiple of 8, unaligned base/stride, or K > 40960) take a strided path that re-reads
// the row from L2.
//
// Arithmetic follows the reference's torch path exactly:
//   dynamic_quant   flashnn/quant_gemm.py:53-57  (two roundings to the input type)
//   rmsnorm_dquant  flashnn/norm.py:45-60        (fp32 throughout)
#include "row_common.h"

#pragma clang fp contract(off)

namespace fnn {

// ------------------------------------------------------------------ dynamic quant
template <int DT, int NV>
__global__ __launch_bounds__(kRowThreads) void dynamic_quant_vec_kernel(
    int8_t* __restrict__ q, uint16_t* __restrict__ scale, const uint16_t* __restrict__ x, int K,
    int64_t ldx, int64_t ldq) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const v4u* xr = (const v4u*)(x + row * ldx);
    const int nvec = K >> 3;
    v4u v[NV];
    uint32_t amax = 0;  // max of |x| taken on the bit patterns (monotonic for finite values)
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + i * kRowThreads;
        v[i] = idx < nvec ? xr[idx] : v4u{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t w = v[i][j] & 0x7FFF7FFFu;
            amax = max(amax, max(w & 0xFFFFu, w >> 16));
        }
    }
    const float mx = block_max(bits_to_f32<DT>(amax), red);
    const uint32_t sbits = f32_to_bits<DT>(mx / 127.0f);
    const float s = bits_to_f32<DT>(sbits);
    if (threadIdx.x == 0) scale[row] = (uint16_t)(DT == FNN_F16 ? sbits : f32_to_f16_bits(s));
    // The quotient is clamped to [-128, 127] (the saturating byte conversion does it): with bf16 input the
    // scale max/127 can round down so far that the row maximum quantises to 128, which an unclamped
    // conversion to int8 wraps to -128 - the sign of the row's largest activation.  fp16 rows never exceed 127.
    const float rcp = quant_rcp(s);   // 0 for an all-zero row: every quotient is then 0
    v2u* qr = (v2u*)(q + row * ldq);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + i * kRowThreads;
        if (idx < nvec) {
            uint32_t w[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                w[j >> 1] = put_biased_byte(quant_in_dtype_f<DT>(bits_to_f32<DT>(v[i][j] & 0xFFFFu), s, rcp), 2 * (j & 1), w[j >> 1]);
                w[j >> 1] = put_biased_byte(quant_in_dtype_f<DT>(bits_to_f32<DT>(v[i][j] >> 16), s, rcp), 2 * (j & 1) + 1, w[j >> 1]);
            }
            qr[idx] = v2u{w[0] ^ 0x80808080u, w[1] ^ 0x80808080u};
        }
    }
}

template <int DT>
__global__ __launch_bounds__(kRowThreads) void dynamic_quant_any_kernel(
    int8_t* __restrict__ q, uint16_t* __restrict__ scale, const uint16_t* __restrict__ x, int K,
    int64_t ldx, int64_t ldq) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * ldx;
    uint32_t amax = 0;
    for (int k = threadIdx.x; k < K; k += kRowThreads) amax = max(amax, (uint32_t)(xr[k] & 0x7FFFu));
    const float mx = block_max(bits_to_f32<DT>(amax), red);
    const uint32_t sbits = f32_to_bits<DT>(mx / 127.0f);
    const float s = bits_to_f32<DT>(sbits);
    if (threadIdx.x == 0) scale[row] = (uint16_t)(DT == FNN_F16 ? sbits : f32_to_f16_bits(s));
    const float rcp = 1.0f / s;
    int8_t* qr = q + row * ldq;
    for (int k = threadIdx.x; k < K; k += kRowThreads)
        qr[k] = (int8_t)(s == 0.f ? 0 : min(quant_in_dtype<DT>(bits_to_f32<DT>(xr[k]), s, rcp), 127));
}

// ---------------------------------------------------------------- rmsnorm + quant
template <int DT, int NV, bool EARLY>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_dquant_vec_kernel(
    int8_t* __restrict__ q, uint16_t* __restrict__ scale, const uint16_t* __restrict__ x,
    const void* __restrict__ gamma, int gamma_dtype, float eps, int K, int64_t ldx, int64_t ldq) {
    __shared__ double redd[4];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const v4u* xr = (const v4u*)(x + row * ldx);
    const int nvec = K >> 3;
    float n[NV][8];
    // short rows, few of them (EARLY): gamma is requested together with the row, so that its latency is not
    // paid a second time behind the first reduction (a handful of rows is one chain of latencies); with
    // thousands of rows the registers are worth more as resident waves, and the launcher keeps the late load
    constexpr bool PRE = EARLY && NV <= 4;
    float gpre[PRE ? NV : 1][8];
    v4u xv[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + i * kRowThreads;
        xv[i] = idx < nvec ? xr[idx] : v4u{0, 0, 0, 0};
    }
    if constexpr (PRE) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = threadIdx.x + i * kRowThreads;
            if (idx < nvec) load_gamma8(gamma, gamma_dtype, (int64_t)idx * 8, gpre[i]);
        }
    }
    double ssq = 0.0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const v4u v = xv[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            n[i][2 * j] = bits_to_f32<DT>(v[j] & 0xFFFFu);
            n[i][2 * j + 1] = bits_to_f32<DT>(v[j] >> 16);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ssq += (double)(n[i][j] * n[i][j]);  // x*x is exact in fp32
    }
    const float sum = (float)block_sum(ssq, redd);
    const float mean = sum / (float)K;
    const float rs = 1.0f / sqrtf(mean + eps);
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + i * kRowThreads;
        if (idx < nvec) {
            float g[8];
            if constexpr (PRE) {
#pragma unroll
                for (int j = 0; j < 8; ++j) g[j] = gpre[i][j];
            } else {
                load_gamma8(gamma, gamma_dtype, (int64_t)idx * 8, g);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                n[i][j] = (n[i][j] * rs) * g[j];
                mx = fmaxf(mx, fabsf(n[i][j]));
            }
        }
    }
    mx = block_max(mx, red);
    const float s = mx / 127.0f;
    if (threadIdx.x == 0) scale[row] = (uint16_t)f32_to_bits<DT>(s);
    const float rcp = quant_rcp(s);
    v2u* qr = (v2u*)(q + row * ldq);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + i * kRowThreads;
        if (idx < nvec) {
            uint32_t w[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j >> 2] = put_biased_byte(rintf(div_by(n[i][j], s, rcp)), j & 3, w[j >> 2]);
            qr[idx] = v2u{w[0] ^ 0x80808080u, w[1] ^ 0x80808080u};
        }
    }
}

// The same with one wave per row and four rows per workgroup, for launches of many rows of up to 2048
// values: nothing crosses waves, so there is no LDS traffic and no barrier, a wave that has its row starts
// computing without waiting for three others, and a CU holds more rows in flight (times at the launcher).
// NV vectors of 8 values per lane.
template <int DT, int NV>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_dquant_wave_kernel(
    int8_t* __restrict__ q, uint16_t* __restrict__ scale, const uint16_t* __restrict__ x,
    const void* __restrict__ gamma, int gamma_dtype, float eps, int64_t M, int K, int64_t ldx, int64_t ldq) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * (kRowThreads / kWave) + (threadIdx.x >> 6);
    if (row >= M) return;   // wave-uniform
    const v4u* xr = (const v4u*)(x + row * ldx);
    const int nvec = K >> 3;
    float n[NV][8];
    v4u xv[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = lane + i * kWave;
        xv[i] = idx < nvec ? xr[idx] : v4u{0, 0, 0, 0};
    }
    double ssq = 0.0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const v4u v = xv[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            n[i][2 * j] = bits_to_f32<DT>(v[j] & 0xFFFFu);
            n[i][2 * j + 1] = bits_to_f32<DT>(v[j] >> 16);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ssq += (double)(n[i][j] * n[i][j]);  // x*x is exact in fp32
    }
    const float sum = (float)wave_sum(ssq);
    const float mean = sum / (float)K;
    const float rs = 1.0f / sqrtf(mean + eps);
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = lane + i * kWave;
        if (idx < nvec) {
            float g[8];
            load_gamma8(gamma, gamma_dtype, (int64_t)idx * 8, g);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                n[i][j] = (n[i][j] * rs) * g[j];
                mx = fmaxf(mx, fabsf(n[i][j]));
            }
        }
    }
    mx = wave_max(mx);
    const float s = mx / 127.0f;
    if (lane == 0) scale[row] = (uint16_t)f32_to_bits<DT>(s);
    const float rcp = quant_rcp(s);
    v2u* qr = (v2u*)(q + row * ldq);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = lane + i * kWave;
        if (idx < nvec) {
            uint32_t w[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j >> 2] = put_biased_byte(rintf(div_by(n[i][j], s, rcp)), j & 3, w[j >> 2]);
            qr[idx] = v2u{w[0] ^ 0x80808080u, w[1] ^ 0x80808080u};
        }
    }
}

template <int DT>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_dquant_any_kernel(
    int8_t* __restrict__ q, uint16_t* __restrict__ scale, const uint16_t* __restrict__ x,
    const void* __restrict__ gamma, int gamma_dtype, float eps, int K, int64_t ldx, int64_t ldq) {
    __shared__ double redd[4];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * ldx;
    double ssq = 0.0;
    for (int k = threadIdx.x; k < K; k += kRowThreads) {
        const float v = bits_to_f32<DT>(xr[k]);
        ssq += (double)(v * v);
    }
    const float sum = (float)block_sum(ssq, redd);
    const float mean = sum / (float)K;
    const float rs = 1.0f / sqrtf(mean + eps);
    float mx = 0.f;
    for (int k = threadIdx.x; k < K; k += kRowThreads) {
        const float nv = (bits_to_f32<DT>(xr[k]) * rs) * load_as_f32(gamma, k, gamma_dtype);
        mx = fmaxf(mx, fabsf(nv));
    }
    mx = block_max(mx, red);
    const float s = mx / 127.0f;
    if (threadIdx.x == 0) scale[row] = (uint16_t)f32_to_bits<DT>(s);
    const float rcp = 1.0f / s;
    int8_t* qr = q + row * ldq;
    for (int k = threadIdx.x; k < K; k += kRowThreads) {
        const float nv = (bits_to_f32<DT>(xr[k]) * rs) * load_as_f32(gamma, k, gamma_dtype);
        qr[k] = (int8_t)quant_clamped(nv, s, rcp);
    }
}

// --------------------------------------------------------------------- launchers
template <int DT>
static void launch_dq(int8_t* q, uint16_t* scale, const uint16_t* x, int64_t M, int K, int64_t ldx,
                      int64_t ldq, hipStream_t st) {
    const dim3 grid((unsigned)M), block(kRowThreads);
    if (vec_ok(x, q, K, ldx, ldq)) {
        const int nv = (K / 8 + kRowThreads - 1) / kRowThreads;
        note_kernel("dynamic_quant_vec_kernel", nv);
#define FNN_DQ(NV) dynamic_quant_vec_kernel<DT, NV><<<grid, block, 0, st>>>(q, scale, x, K, ldx, ldq)
        FNN_ROW_DISPATCH_NV(nv, FNN_DQ);
#undef FNN_DQ
    } else {
        note_kernel("dynamic_quant_any_kernel");
        dynamic_quant_any_kernel<DT><<<grid, block, 0, st>>>(q, scale, x, K, ldx, ldq);
    }
}

template <int DT>
static void launch_rq(int8_t* q, uint16_t* scale, const uint16_t* x, const void* gamma, int gdt,
                      float eps, int64_t M, int K, int64_t ldx, int64_t ldq, hipStream_t st) {
    const dim3 grid((unsigned)M), block(kRowThreads);
    if (vec_ok(x, q, K, ldx, ldq) && ((uintptr_t)gamma % 16) == 0) {
        // many short rows: one wave per row.  Measured (bf16, rows x values, one wave / one workgroup per
        // row): 32768 x 1024 24.4 / 43.4 us, 8192 x 2048 15.2 / 19.1 us, 8192 x 4096 25.9 / 26.1 us,
        // 8192 x 8192 60.5 / 45.6 us, 2048 x 8192 18.3 / 14.2 us - from 4096 values on the four waves of a
        // workgroup fetch a row faster than one wave does.
        const int nvw = (K / 8 + kWave - 1) / kWave;
        if (M >= 2048 && nvw <= 4) {
            const dim3 wgrid((unsigned)((M + 3) / 4));
            note_kernel("rmsnorm_dquant_wave_kernel", nvw <= 1 ? 1 : nvw <= 2 ? 2 : 4);
#define FNN_RQW(NV) rmsnorm_dquant_wave_kernel<DT, NV><<<wgrid, block, 0, st>>>(q, scale, x, gamma, gdt, eps, M, K, ldx, ldq)
            if (nvw <= 1) FNN_RQW(1);
            else if (nvw <= 2) FNN_RQW(2);
            else FNN_RQW(4);
#undef FNN_RQW
            return;
        }
        const int nv = (K / 8 + kRowThreads - 1) / kRowThreads;
        note_kernel("rmsnorm_dquant_vec_kernel", nv, M <= 1024 && nv <= 4);
#define FNN_RQ(NV)                                                                                          \
    do {                                                                                                    \
        if (M <= 1024 && NV <= 4)                                                                           \
            rmsnorm_dquant_vec_kernel<DT, NV <= 4 ? NV : 1, true><<<grid, block, 0, st>>>(q, scale, x, gamma, gdt, eps, K, ldx, ldq); \
        else rmsnorm_dquant_vec_kernel<DT, NV, false><<<grid, block, 0, st>>>(q, scale, x, gamma, gdt, eps, K, ldx, ldq);             \
    } while (0)
        FNN_ROW_DISPATCH_NV(nv, FNN_RQ);
#undef FNN_RQ
    } else {
        note_kernel("rmsnorm_dquant_any_kernel");
        rmsnorm_dquant_any_kernel<DT><<<grid, block, 0, st>>>(q, scale, x, gamma, gdt, eps, K, ldx, ldq);
    }
}

}  // namespace fnn

using namespace fnn;

static int check_rows(const char* fn, const void* q, const void* scale, const void* x, int64_t M,
                      int64_t K, int64_t ldx, int64_t ldq, int x_dtype) {
    // an empty tensor has no address: pointers are only required when there are rows
    if (M != 0 && (!q || !scale || !x)) { set_error("%s: null pointer argument", fn); return FNN_ERR_ARG; }
    if (M < 0 || K <= 0 || ldx < K || ldq < K) {
        set_error("%s: bad shape M=%lld K=%lld ldx=%lld ldq=%lld", fn, (long long)M, (long long)K,
                  (long long)ldx, (long long)ldq);
        return FNN_ERR_ARG;
    }
    if (!is16(x_dtype)) { set_error("%s: input type must be fp16 or bf16", fn); return FNN_ERR_UNSUPPORTED; }
    if (M > 0x7FFFFFFFLL || K > 0x7FFFFFFFLL) { set_error("%s: shape too large", fn); return FNN_ERR_UNSUPPORTED; }
    return FNN_OK;
}

extern "C" int fnn_dynamic_quant(void* q, void* scale, const void* x, int64_t M, int64_t K,
                                 int64_t ldx, int64_t ldq, int x_dtype, void* stream) {
    int rc = check_rows("fnn_dynamic_quant", q, scale, x, M, K, ldx, ldq, x_dtype);
    if (rc != FNN_OK) return rc;
    if (M == 0) return FNN_OK;
    hipStream_t st = (hipStream_t)stream;
    const Call call("fnn_dynamic_quant");
    if (x_dtype == FNN_F16)
        launch_dq<FNN_F16>((int8_t*)q, (uint16_t*)scale, (const uint16_t*)x, M, (int)K, ldx, ldq, st);
    else
        launch_dq<FNN_BF16>((int8_t*)q, (uint16_t*)scale, (const uint16_t*)x, M, (int)K, ldx, ldq, st);
    return call.done();
}

extern "C" int fnn_rmsnorm_dquant(void* q, void* scale, const void* x, const void* gamma, float eps,
                                  int64_t M, int64_t K, int64_t ldx, int64_t ldq, int x_dtype,
                                  int gamma_dtype, void* stream) {
    int rc = check_rows("fnn_rmsnorm_dquant", q, scale, x, M, K, ldx, ldq, x_dtype);
    if (rc != FNN_OK) return rc;
    if (M != 0 && !gamma) { set_error("fnn_rmsnorm_dquant: null gamma"); return FNN_ERR_ARG; }
    if (!isflt(gamma_dtype)) { set_error("fnn_rmsnorm_dquant: bad gamma type"); return FNN_ERR_UNSUPPORTED; }
    if (M == 0) return FNN_OK;
    hipStream_t st = (hipStream_t)stream;
    const Call call("fnn_rmsnorm_dquant");
    if (x_dtype == FNN_F16)
        launch_rq<FNN_F16>((int8_t*)q, (uint16_t*)scale, (const uint16_t*)x, gamma, gamma_dtype, eps, M, (int)K, ldx, ldq, st);
    else
        launch_rq<FNN_BF16>((int8_t*)q, (uint16_t*)scale, (const uint16_t*)x, gamma, gamma_dtype, eps, M, (int)K, ldx, ldq, st);
    return call.done();
}
