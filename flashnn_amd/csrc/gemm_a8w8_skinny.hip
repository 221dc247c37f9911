// A8W8 GEMM for up to 64 activation rows (decode and small-batch shapes, gfx950).
//
// With so few activation rows the work is reading the weights once, so the kernel is laid out
// like the weight-only streaming kernels rather than like the tiled GEMM:
//   * one 512-thread workgroup (8 waves) per 16 weight rows; the waves split K;
//   * lane (i, g) streams 16-byte pieces of weight row i (k = 64 step + 16 g ..) straight from
//     global memory into the "A" operand of v_mfma_i32_16x16x64_i8, kept UN steps ahead in
//     registers; the same bytes of activation row j are the "B" operand (the activation matrix
//     is small and stays in L2);
//   * the 8 partial int32 tiles are added through LDS (integer sums: exact in any order), then
//     the row and column scales are applied exactly as in the tiled kernel,
//     out = ((float)acc * alpha_row[m]) * alpha_col[n], and rounded once.
//
// Reference semantics: flashnn/quant_gemm.py:96-104, flashnn/triton_kernels/gemm_a8w8.py:135,170-173.
#include "a8w8_common.h"

// The scaled output is two fp32 multiplications and one rounding to 16 bits, each rounded on its
// own as in the reference's torch path.
#pragma clang fp contract(off)

namespace fnn {

constexpr int kSkWaves = 8;
constexpr int kSkUN = 8;     // steps in flight per lane

template <int MB, int MODE>
__global__ __launch_bounds__(kSkWaves * 64) void gemm_a8w8_skinny_kernel(const A8W8Args p) {
    __shared__ int red[kSkWaves][MB][4][64];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int n0 = blockIdx.x * 16;

    const int steps = p.K / 64;
    const int s_begin = (int)((int64_t)steps * wave / kSkWaves);
    const int s_end = (int)((int64_t)steps * (wave + 1) / kSkWaves);

    const char* wptr = (const char*)p.b + (int64_t)min(n0 + li, p.N - 1) * p.ldb + lg * 16;
    const char* aptr[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
        aptr[mb] = (const char*)p.a + (int64_t)min(mb * 16 + li, p.M - 1) * p.lda + lg * 16;
    auto load_w = [&](int step) -> v4i {
        return *(const v4i*)(wptr + (int64_t)min(step, s_end - 1) * 64);
    };
    auto load_a = [&](int mb, int step) -> v4i {
        return *(const v4i*)(aptr[mb] + (int64_t)min(step, s_end - 1) * 64);
    };

    v4i acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = v4i{0, 0, 0, 0};

    if (s_begin < s_end) {
        v4i wq[kSkUN], aq[kSkUN][MB];
#pragma unroll
        for (int i = 0; i < kSkUN; ++i) {
            wq[i] = load_w(s_begin + i);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) aq[i][mb] = load_a(mb, s_begin + i);
        }
        for (int sb = s_begin; sb < s_end; sb += kSkUN) {
#pragma unroll
            for (int i = 0; i < kSkUN; ++i) {
                const int step = sb + i;
                if (step < s_end) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wq[i], aq[i][mb], acc[mb], 0, 0, 0);
                }
                wq[i] = load_w(step + kSkUN);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) aq[i][mb] = load_a(mb, step + kSkUN);
            }
        }
    }

    // ---- sum of the 8 partial tiles; lane (j, g) of a wave holds channels 4g .. 4g+3 of row 16 mb + j
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][mb][r][lane] = acc[mb][r];
    __syncthreads();
    // thread e writes channel e & 15 of row e >> 4: 16 consecutive threads fill 16 consecutive outputs
    for (int e = threadIdx.x; e < MB * 256; e += kSkWaves * 64) {
        const int c = e & 15;
        const int ml = e >> 4;
        const int mb = ml >> 4;
        const int src_lane = (c >> 2) * 16 + (ml & 15);
        int v = 0;
#pragma unroll
        for (int w = 0; w < kSkWaves; ++w) v += red[w][mb][c & 3][src_lane];
        const int m = ml, n = n0 + c;
        if (m < p.M && n < p.N) {
            if constexpr (MODE == OUT_I32) {
                ((int32_t*)p.out)[(int64_t)m * p.ldc + n] = v;
            } else {
                const float ar = load_as_f32(p.arow, m, p.arow_dtype);
                const float ac = load_as_f32(p.acol, n, p.acol_dtype);
                const float f = rounded_f32(((float)v * ar) * ac);
                ((uint16_t*)p.out)[(int64_t)m * p.ldc + n] =
                    (uint16_t)(MODE == OUT_F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f));
            }
        }
    }
}

template <int MODE>
static bool launch_skinny_t(A8W8Args& p, hipStream_t st) {
    if (p.M > 64 || p.K % 64 != 0 || p.lda % 16 != 0 || p.ldb % 16 != 0 ||
        ((uintptr_t)p.a % 16) != 0 || ((uintptr_t)p.b % 16) != 0)
        return false;
    const dim3 grid((p.N + 15) / 16), block(kSkWaves * 64);
    if (p.M <= 16) gemm_a8w8_skinny_kernel<1, MODE><<<grid, block, 0, st>>>(p);
    else if (p.M <= 32) gemm_a8w8_skinny_kernel<2, MODE><<<grid, block, 0, st>>>(p);
    else if (p.M <= 48) gemm_a8w8_skinny_kernel<3, MODE><<<grid, block, 0, st>>>(p);
    else gemm_a8w8_skinny_kernel<4, MODE><<<grid, block, 0, st>>>(p);
    return true;
}

bool launch_a8w8_skinny(A8W8Args& p, int mode, hipStream_t st) {
    if (mode == OUT_I32) return launch_skinny_t<OUT_I32>(p, st);
    return mode == OUT_F16 ? launch_skinny_t<OUT_F16>(p, st) : launch_skinny_t<OUT_BF16>(p, st);
}

}  // namespace fnn
