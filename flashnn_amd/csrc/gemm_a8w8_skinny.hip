// A8W8 GEMM for up to 64 activation rows (decode and small-batch shapes, gfx950).
//
// With so few activation rows the work is reading the weights once, so the kernel is laid out
// like the weight-only streaming kernels rather than like the tiled GEMM:
//   * one 512-thread workgroup (8 waves) per 16 weight rows; the waves split K;
//   * a wave streams its 16 weight rows in blocks of 128 bytes per row, kept UN blocks ahead in
//     registers, and reshapes each block through a private LDS staging area into the "A" operand
//     of v_mfma_i32_16x16x64_i8 (two k-steps per block); the same bytes of 16 activation rows,
//     fetched and reshaped the same way, are the "B" operand (the activation matrix is small and
//     stays in L2);
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
constexpr int kSkUN = 4;     // 128-byte k-pairs in flight per lane

template <int MB, int MODE>
__global__ __launch_bounds__(kSkWaves * 64) void gemm_a8w8_skinny_kernel(const A8W8Args p) {
    __shared__ int red[kSkWaves][MB][4][64];
    // per wave: one 16-row x 128-byte block of weights and MB blocks of activations
    __shared__ __attribute__((aligned(16))) char stg[kSkWaves][1 + MB][2048];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int r8 = lane >> 3;
    const int c8 = lane & 7;
    const int n0 = blockIdx.x * 16;

    const int pairs = p.K / 128;
    const int p_begin = (int)((int64_t)pairs * wave / kSkWaves);
    const int p_end = (int)((int64_t)pairs * (wave + 1) / kSkWaves);

    // Load h of a block fetches rows 8h .. 8h+7, eight lanes per row: one full 128-byte line per
    // row, which streams about a third faster from HBM than the operand's own 16 rows x 64 bytes.
    // The block is reshaped through the wave's staging area: row i at i*128, its 16-byte chunk c
    // at slot c ^ ((i >> 1) & 7), so that neither the writes nor the operand reads (16 rows, same
    // chunk) meet in a bank.
    const char* wptr[2];
    const char* aptr[MB][2];
    int swr[2], srd[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        wptr[h] = (const char*)p.b + (int64_t)min(n0 + 8 * h + r8, p.N - 1) * p.ldb + c8 * 16;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            aptr[mb][h] = (const char*)p.a + (int64_t)min(mb * 16 + 8 * h + r8, p.M - 1) * p.lda + c8 * 16;
        swr[h] = (8 * h + r8) * 128 + ((c8 ^ ((4 * h + (r8 >> 1)) & 7)) << 4);
        srd[h] = li * 128 + (((4 * h + lg) ^ ((li >> 1) & 7)) << 4);
    }
    char* const mine = &stg[wave][0][0];

    v4i acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = v4i{0, 0, 0, 0};

    if (p_begin < p_end) {
        v4i wq[kSkUN][2], aq[kSkUN][MB][2];
        auto fetch = [&](int i, int pr) {
            const int64_t off = (int64_t)min(pr, p_end - 1) * 128;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                wq[i][h] = *(const v4i*)(wptr[h] + off);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) aq[i][mb][h] = *(const v4i*)(aptr[mb][h] + off);
            }
        };
#pragma unroll
        for (int i = 0; i < kSkUN; ++i) fetch(i, p_begin + i);
        for (int pb = p_begin; pb < p_end; pb += kSkUN) {
#pragma unroll
            for (int i = 0; i < kSkUN; ++i) {
                const int pr = pb + i;
                if (pr < p_end) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        *(v4i*)(mine + swr[h]) = wq[i][h];
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) *(v4i*)(mine + (1 + mb) * 2048 + swr[h]) = aq[i][mb][h];
                    }
                    if (pr + kSkUN < p_end) fetch(i, pr + kSkUN);
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        const v4i w = *(const v4i*)(mine + srd[s]);
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) {
                            const v4i a = *(const v4i*)(mine + (1 + mb) * 2048 + srd[s]);
                            acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w, a, acc[mb], 0, 0, 0);
                        }
                    }
                }
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
    if (p.M > 64 || p.K % 128 != 0 || p.lda % 16 != 0 || p.ldb % 16 != 0 ||
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
