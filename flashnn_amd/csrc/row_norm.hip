// RMSNorm, LayerNorm and LayerNorm + per-token int8 quantisation for gfx950: the producers one step
// before the quantised GEMMs.  One 256-thread workgroup per row; the row is read once with 16-byte
// loads and stays in registers over the reductions.
//
//   rmsnorm            n = x * (1 / sqrt(mean(x^2) + eps)) in fp32, rounded to the input type, times
//                      gamma, rounded to the input type (flashnn/norm.py:25-33)
//   layernorm          y = ((x - mean) * rstd) * gamma + beta in fp32, rounded once to the input type
//                      (torch.nn.functional.layer_norm, flashnn/norm.py:82-85)
//   layernorm + quant  the rounded y, then scale = max|y| / 127 and q = clamp(round(y / scale)), both
//                      evaluated in the input type as torch evaluates them (flashnn/norm.py:112-119)
//
// Sums are taken in fp64 over exactly representable terms (x and x^2 of 16-bit inputs: 22-bit
// products, so a row whose magnitudes span less than 2^15 sums without any rounding); their order
// then does not matter and the kernels are bit-identical to a float64 restatement
// (var = sum(x^2)/K - (sum(x)/K)^2 in fp64, rounded once); torch's own fp32 moments can differ from
// that in their last bit.
#include "row_common.h"

namespace fnn {

enum { OP_RMS = 0, OP_LN = 1, OP_LNQ = 2 };

struct NormArgs {
    void* out;            // 16-bit outputs (OP_RMS, OP_LN) or int8 (OP_LNQ)
    uint16_t* scale;      // OP_LNQ: one scale per row, in the input type
    const uint16_t* x;
    const void* gamma;
    const void* beta;
    int gb_dtype;
    float eps;
    int K;
    int64_t ldx, ldo;
};

// fp32 value -> nearest value of the 16-bit type.  The value is pinned first: the compiler would
// otherwise fuse the multiplication or addition that produced it with the conversion
// (v_fma_mixlo_f16), which rounds once where the reference rounds twice.
template <int DT> __device__ __forceinline__ float round_dt(float v) {
    return bits_to_f32<DT>(f32_to_bits<DT>(rounded_f32(v)));
}

template <int DT, int NV, int OP, bool EARLY>
__global__ __launch_bounds__(kRowThreads) void norm_vec_kernel(const NormArgs p) {
    __shared__ double redd[8];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const v4u* xr = (const v4u*)(p.x + row * p.ldx);
    const int nvec = p.K >> 3;
    float n[NV][8];
    // short rows, few of them (EARLY): gamma and beta are requested together with the row, so that their
    // latency is not paid a second time behind the first reduction - a handful of rows is one chain of
    // latencies (M=1, K=8192: 4.0 -> 3.6 us).  With thousands of rows the registers this takes cost more in
    // resident waves than the latency is worth (layer norm 8192 x 8192: 59 -> 68 us), so the launcher keeps
    // the late loads there.
    constexpr bool PRE = EARLY && NV <= 4;
    float gpre[PRE ? NV : 1][8], bpre[PRE && OP != OP_RMS ? NV : 1][8];
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
            if (idx < nvec) {
                load_gamma8(p.gamma, p.gb_dtype, (int64_t)idx * 8, gpre[i]);
                if constexpr (OP != OP_RMS) load_gamma8(p.beta, p.gb_dtype, (int64_t)idx * 8, bpre[i]);
            }
        }
    }
    double acc = 0.0, acc1 = 0.0;   // sum of squares; sum
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const v4u v = xv[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            n[i][2 * j] = bits_to_f32<DT>(v[j] & 0xFFFFu);
            n[i][2 * j + 1] = bits_to_f32<DT>(v[j] >> 16);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const double xd = (double)n[i][j];
            acc = __builtin_fma(xd, xd, acc);     // the product is exact; one fp64 conversion serves both sums
            if constexpr (OP != OP_RMS) acc1 += xd;
        }
    }
    float mul;   // the row's multiplier: 1/rms or rstd
    if constexpr (OP == OP_RMS) {
        const float sum = (float)block_sum(acc, redd);
        mul = 1.0f / sqrtf(sum / (float)p.K + p.eps);
    } else {
        block_sum2(acc, acc1, redd);
        const double m64 = acc1 / (double)p.K;
        const float mean = (float)m64;
        const float var = (float)fmax(acc / (double)p.K - m64 * m64, 0.0);
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) n[i][j] = n[i][j] - mean;
        mul = 1.0f / sqrtf(var + p.eps);
    }
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + i * kRowThreads;
        if (idx < nvec) {
            float g[8], b[8];
            if constexpr (PRE) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    g[j] = gpre[i][j];
                    if constexpr (OP != OP_RMS) b[j] = bpre[i][j];
                }
            } else {
                load_gamma8(p.gamma, p.gb_dtype, (int64_t)idx * 8, g);
                if constexpr (OP != OP_RMS) load_gamma8(p.beta, p.gb_dtype, (int64_t)idx * 8, b);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if constexpr (OP == OP_RMS) n[i][j] = round_dt<DT>(round_dt<DT>(n[i][j] * mul) * g[j]);
                else n[i][j] = round_dt<DT>((n[i][j] * mul) * g[j] + b[j]);
                mx = fmaxf(mx, fabsf(n[i][j]));
            }
            if constexpr (OP != OP_LNQ) {
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    o[j] = f32_to_bits<DT>(n[i][2 * j]) | (f32_to_bits<DT>(n[i][2 * j + 1]) << 16);
                ((v4u*)((uint16_t*)p.out + row * p.ldo))[idx] = v4u{o[0], o[1], o[2], o[3]};
            }
        }
    }
    if constexpr (OP == OP_LNQ) {
        mx = block_max(mx, red);
        const uint32_t sbits = f32_to_bits<DT>(mx / 127.0f);
        const float s = bits_to_f32<DT>(sbits);
        if (threadIdx.x == 0) p.scale[row] = (uint16_t)sbits;
        const float rcp = quant_rcp(s);
        v2u* qr = (v2u*)((int8_t*)p.out + row * p.ldo);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = threadIdx.x + i * kRowThreads;
            if (idx < nvec) {
                uint32_t w[2] = {0, 0};
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    w[j >> 2] = put_biased_byte(quant_in_dtype_f<DT>(n[i][j], s, rcp), j & 3, w[j >> 2]);
                qr[idx] = v2u{w[0] ^ 0x80808080u, w[1] ^ 0x80808080u};
            }
        }
    }
}

// Any K and alignment: the row is re-read for every pass.
template <int DT, int OP>
__global__ __launch_bounds__(kRowThreads) void norm_any_kernel(const NormArgs p) {
    __shared__ double redd[8];
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = p.x + row * p.ldx;
    double acc = 0.0, acc1 = 0.0;
    for (int k = threadIdx.x; k < p.K; k += kRowThreads) {
        const float v = bits_to_f32<DT>(xr[k]);
        acc += (double)(v * v);
        acc1 += (double)v;
    }
    float mean = 0.f, mul;
    if constexpr (OP == OP_RMS) {
        const float sum = (float)block_sum(acc, redd);
        mul = 1.0f / sqrtf(sum / (float)p.K + p.eps);
    } else {
        block_sum2(acc, acc1, redd);
        const double m64 = acc1 / (double)p.K;
        mean = (float)m64;
        const float var = (float)fmax(acc / (double)p.K - m64 * m64, 0.0);
        mul = 1.0f / sqrtf(var + p.eps);
    }
    auto value = [&](int k) -> float {
        const float v = bits_to_f32<DT>(xr[k]);
        const float g = load_as_f32(p.gamma, k, p.gb_dtype);
        if constexpr (OP == OP_RMS) return round_dt<DT>(round_dt<DT>(v * mul) * g);
        else return round_dt<DT>(((v - mean) * mul) * g + load_as_f32(p.beta, k, p.gb_dtype));
    };
    if constexpr (OP != OP_LNQ) {
        uint16_t* o = (uint16_t*)p.out + row * p.ldo;
        for (int k = threadIdx.x; k < p.K; k += kRowThreads) o[k] = (uint16_t)f32_to_bits<DT>(value(k));
    } else {
        float mx = 0.f;
        for (int k = threadIdx.x; k < p.K; k += kRowThreads) mx = fmaxf(mx, fabsf(value(k)));
        mx = block_max(mx, red);
        const uint32_t sbits = f32_to_bits<DT>(mx / 127.0f);
        const float s = bits_to_f32<DT>(sbits);
        if (threadIdx.x == 0) p.scale[row] = (uint16_t)sbits;
        const float rcp = 1.0f / s;
        int8_t* o = (int8_t*)p.out + row * p.ldo;
        for (int k = threadIdx.x; k < p.K; k += kRowThreads)
            o[k] = (int8_t)(s == 0.f ? 0 : min(max(quant_in_dtype<DT>(value(k), s, rcp), -128), 127));
    }
}

template <int DT, int OP>
static void launch_norm(const NormArgs& p, int64_t M, hipStream_t st) {
    const dim3 grid((unsigned)M), block(kRowThreads);
    const int esz = OP == OP_LNQ ? 1 : 2;
    const bool vec = p.K % 8 == 0 && p.K <= 8 * kRowThreads * kRowMaxNV && p.ldx % 8 == 0 &&
                     (p.ldo * esz) % (OP == OP_LNQ ? 8 : 16) == 0 && ((uintptr_t)p.x % 16) == 0 &&
                     ((uintptr_t)p.out % (OP == OP_LNQ ? 8 : 16)) == 0 && ((uintptr_t)p.gamma % 16) == 0 &&
                     (OP == OP_RMS || ((uintptr_t)p.beta % 16) == 0);
    if (vec) {
        const int nv = (p.K / 8 + kRowThreads - 1) / kRowThreads;
        note_kernel("norm_vec_kernel", OP, nv, M <= 1024 && nv <= 4);
        // up to four workgroups per CU are "few rows": every row is then resident at once either way
#define FNN_NORM(NV)                                                                   \
    do {                                                                               \
        if (M <= 1024 && NV <= 4) norm_vec_kernel<DT, NV <= 4 ? NV : 1, OP, true><<<grid, block, 0, st>>>(p); \
        else norm_vec_kernel<DT, NV, OP, false><<<grid, block, 0, st>>>(p);            \
    } while (0)
        FNN_ROW_DISPATCH_NV(nv, FNN_NORM);
#undef FNN_NORM
    } else {
        note_kernel("norm_any_kernel", OP);
        norm_any_kernel<DT, OP><<<grid, block, 0, st>>>(p);
    }
}

template <int OP>
static int run_norm(const char* fn, void* out, void* scale, const void* x, const void* gamma,
                    const void* beta, float eps, int64_t M, int64_t K, int64_t ldx, int64_t ldo,
                    int x_dtype, int gb_dtype, void* stream) {
    // an empty tensor has no address: pointers are only required when there are rows
    if (M != 0 && (!out || !x || !gamma || (OP != OP_RMS && !beta) || (OP == OP_LNQ && !scale))) {
        set_error("%s: null pointer argument", fn);
        return FNN_ERR_ARG;
    }
    if (M < 0 || K <= 0 || ldx < K || ldo < K) {
        set_error("%s: bad shape M=%lld K=%lld ldx=%lld ldo=%lld", fn, (long long)M, (long long)K,
                  (long long)ldx, (long long)ldo);
        return FNN_ERR_ARG;
    }
    if (!is16(x_dtype)) { set_error("%s: input type must be fp16 or bf16", fn); return FNN_ERR_UNSUPPORTED; }
    if (!isflt(gb_dtype)) { set_error("%s: bad weight type", fn); return FNN_ERR_UNSUPPORTED; }
    if (M > 0x7FFFFFFFLL || K > 0x7FFFFFFFLL) { set_error("%s: shape too large", fn); return FNN_ERR_UNSUPPORTED; }
    if (M == 0) return FNN_OK;
    NormArgs p{out, (uint16_t*)scale, (const uint16_t*)x, gamma, beta, gb_dtype, eps, (int)K, ldx, ldo};
    const Call call(fn);
    if (x_dtype == FNN_F16) launch_norm<FNN_F16, OP>(p, M, (hipStream_t)stream);
    else launch_norm<FNN_BF16, OP>(p, M, (hipStream_t)stream);
    return call.done();
}

}  // namespace fnn

using namespace fnn;

extern "C" int fnn_rmsnorm(void* out, const void* x, const void* gamma, float eps, int64_t M, int64_t K,
                           int64_t ldx, int64_t ldo, int x_dtype, int gamma_dtype, void* stream) {
    return run_norm<OP_RMS>("fnn_rmsnorm", out, nullptr, x, gamma, nullptr, eps, M, K, ldx, ldo, x_dtype,
                            gamma_dtype, stream);
}

extern "C" int fnn_layernorm(void* out, const void* x, const void* gamma, const void* beta, float eps,
                             int64_t M, int64_t K, int64_t ldx, int64_t ldo, int x_dtype, int gb_dtype,
                             void* stream) {
    return run_norm<OP_LN>("fnn_layernorm", out, nullptr, x, gamma, beta, eps, M, K, ldx, ldo, x_dtype,
                           gb_dtype, stream);
}

extern "C" int fnn_layernorm_dquant(void* q, void* scale, const void* x, const void* gamma, const void* beta,
                                    float eps, int64_t M, int64_t K, int64_t ldx, int64_t ldq, int x_dtype,
                                    int gb_dtype, void* stream) {
    return run_norm<OP_LNQ>("fnn_layernorm_dquant", q, scale, x, gamma, beta, eps, M, K, ldx, ldq, x_dtype,
                            gb_dtype, stream);
}
