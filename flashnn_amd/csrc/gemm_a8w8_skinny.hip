// A8W8 GEMM for up to 64 activation rows (decode and small-batch shapes, gfx950): two kernels, one
// in which every wave fetches its own activations (a single row, and shapes the other does not take)
// and one in which the waves of a workgroup share activation slabs through LDS.
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

// ---------------------------------------------------------------- shared activation slabs
// Same job, for matrices with enough rows and K: 8 waves = RT tiles of 16 weight rows x KS = 8 / RT
// parts of K.  The RT waves of a K part share each slab of activations (16 MB rows x 128 bytes),
// which is copied global -> LDS by direct-to-LDS loads into a ring of 4 stages (3 slabs ahead; row r
// keeps its 16-byte chunk c in slot c ^ ((r >> 1) & 7)); the weights take the route of the kernel
// above (full 128-byte lines into registers, 4 slabs ahead, reshaped through a private LDS area).
// Every iteration issues its loads in a fixed order (copies, then weights), so "slab j has landed" is
// one s_waitcnt vmcnt(X) with a compile-time X, followed by a bare s_barrier.  K parts may differ by
// one slab: every wave runs the same number of iterations and skips the slabs it does not have.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

template <int MB, int RT, int MODE, bool MOE = false>
__global__ __launch_bounds__(512) void gemm_a8w8_panel_kernel(const A8W8Args p, const int passes, const MoeArgs q) {
    constexpr int KS = 8 / RT;
    constexpr int SLAB = MB * 16 * 128;
    constexpr int STG = KS * SLAB;
    constexpr int RED = (KS - 1) * RT * MB * 4 * 64 * 4;
    constexpr int STG0 = STG > RED ? STG : RED;
    constexpr int NCP = MB * 2 / RT;            // copies per wave and slab
    static_assert(MB * 2 % RT == 0 && NCP >= 1, "the waves of a K part must share a slab's copies evenly");
    __shared__ __attribute__((aligned(16))) char st0[STG0];
    __shared__ __attribute__((aligned(16))) char st1[STG];
    __shared__ __attribute__((aligned(16))) char st2[STG];
    __shared__ __attribute__((aligned(16))) char st3[STG];
    __shared__ __attribute__((aligned(16))) char wst[8 * 2048];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rt = wave % RT;
    const int ks = wave / RT;
    const int li = lane & 15;
    const int lg = lane >> 4;

    const int tiles = p.N / (16 * RT);
    const int y = blockIdx.x >> 3;
    const int pass = y % passes;
    const int tile = (y / passes) * 8 + (blockIdx.x & 7);
    if (tile >= tiles) return;
    const int m_base = pass * (MB * 16);
    const int row0 = (tile * RT + rt) * 16;
    // mixture of experts: the pass covers sorted rows m_base .. of one expert; passes beyond the rows
    // in use have nothing to do
    int expert = 0;
    if constexpr (MOE) {
        if (m_base >= q.ntpp[0]) return;
        expert = q.expert_ids[m_base / q.block_m];
    }
    // activation row and validity of local row r of this pass
    auto token_of = [&](int r) -> int {
        const int sidx = m_base + r;
        return sidx < q.EM ? q.sorted_ids[sidx] : q.num_valid;
    };

    // K = 128 * (KT - 1) + tail.  The last slab may be partial (tail = 32, 64 or 96 bytes): the lanes
    // whose 16-byte chunk lies beyond K fetch the first chunk of their row piece instead (bytes that
    // exist), and the weights of those chunks are replaced by zeros before they reach the MFMAs, so
    // whatever the activation copies fetched there is multiplied by zero.
    const int KT = (p.K + 127) / 128;
    const int tail = p.K - (KT - 1) * 128;
    const bool part_tail = tail < 128 && ks == KS - 1;   // wave-uniform: this K part ends in the partial slab
    const int sl0 = KT * ks / KS;
    const int nsl = KT * (ks + 1) / KS - sl0;
    const int n_iter = ((KT + KS - 1) / KS + 3) / 4 * 4;

    const int r8 = lane >> 3, c8 = lane & 7;
    const char* wptr = (const char*)p.b + (MOE ? (int64_t)expert * q.stride_be : 0) + (int64_t)(row0 + r8) * p.ldb +
                       c8 * 16 + (int64_t)sl0 * 128;
    const int64_t w_half = 8 * p.ldb;
    const bool wzero = c8 * 16 >= tail;
    const int wfix = wzero ? -(c8 * 16) : 0;
    auto load_w = [&](int jj, int half) -> v4i {
        const int s = min(jj, nsl - 1);
        const int fix = part_tail && s == nsl - 1 ? wfix : 0;
        return *(const v4i*)(wptr + (int64_t)s * 128 + half * w_half + fix);
    };
    char* const wmine = wst + wave * 2048;
    int wwr[2], wrd[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        wwr[h] = (8 * h + r8) * 128 + ((c8 ^ ((4 * h + (r8 >> 1)) & 7)) << 4);
        wrd[h] = li * 128 + (((4 * h + lg) ^ ((li >> 1) & 7)) << 4);
    }

    // activation copies: the 64 RT lanes of a K part cover 8 RT rows per copy
    const int t = rt * 64 + lane;
    const char* act_part = (const char*)p.a + (int64_t)sl0 * 128;
    int64_t goff[NCP];
    int afix[NCP];
#pragma unroll
    for (int i = 0; i < NCP; ++i) {
        const int row = i * (8 * RT) + (t >> 3);
        const int chunk = (t & 7) ^ ((row >> 1) & 7);
        if constexpr (MOE) {
            const int tok = token_of(row);
            goff[i] = (int64_t)(tok < q.num_valid ? tok / q.top_k : 0) * p.lda + chunk * 16;
        } else {
            goff[i] = (int64_t)min(m_base + row, p.M - 1) * p.lda + chunk * 16;
        }
        afix[i] = chunk * 16 >= tail ? -(chunk * 16) : 0;
    }
    auto copy_act = [&](char* stage, int jj) {
        const int s = min(jj, nsl - 1);
        const char* src = act_part + (int64_t)s * 128;
        const bool last = part_tail && s == nsl - 1;
#pragma unroll
        for (int i = 0; i < NCP; ++i)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + goff[i] + (last ? afix[i] : 0)),
                                             (lds_ptr_t)(stage + ks * SLAB + (i * RT * 64 + rt * 64) * 16), 16, 0, 0);
    };
    int rd[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) rd[s] = ks * SLAB + li * 128 + (((4 * s + lg) ^ ((li >> 1) & 7)) << 4);

    v4i acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = v4i{0, 0, 0, 0};

    constexpr int C = NCP + 2;
    constexpr int X = (C - NCP) + 2 * C;
    auto wait_barrier = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070 | (X & 15) | ((X >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    v4i wq[4][2];

#define FNN_A8_ITER(W, CUR, FREE, JJ)                                                   \
    do {                                                                                \
        wait_barrier();                                                                 \
        copy_act(FREE, (JJ) + 3);                                                       \
        const bool mine_ = (JJ) < nsl;   /* wave-uniform */                             \
        if (mine_) {                                                                    \
            const bool z_ = part_tail && (JJ) == nsl - 1 && wzero;                      \
            *(v4i*)(wmine + wwr[0]) = z_ ? v4i{0, 0, 0, 0} : wq[W][0];                  \
            *(v4i*)(wmine + wwr[1]) = z_ ? v4i{0, 0, 0, 0} : wq[W][1];                  \
        }                                                                               \
        wq[W][0] = load_w((JJ) + 4, 0);                                                 \
        wq[W][1] = load_w((JJ) + 4, 1);                                                 \
        __builtin_amdgcn_sched_barrier(0);                                              \
        if (mine_) {                                                                    \
            _Pragma("unroll") for (int s = 0; s < 2; ++s) {                             \
                const v4i w = *(const v4i*)(wmine + wrd[s]);                            \
                _Pragma("unroll") for (int mb = 0; mb < MB; ++mb) {                     \
                    const v4i a = *(const v4i*)((CUR) + rd[s] + mb * 2048);             \
                    acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w, a, acc[mb], 0, 0, 0); \
                }                                                                       \
            }                                                                           \
        }                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                              \
    } while (0)

    // prologue: the same issue order as the three iterations before the first one
    wq[0][0] = load_w(0, 0);
    wq[0][1] = load_w(0, 1);
    __builtin_amdgcn_sched_barrier(0);
    copy_act(st0, 0);
    wq[1][0] = load_w(1, 0);
    wq[1][1] = load_w(1, 1);
    __builtin_amdgcn_sched_barrier(0);
    copy_act(st1, 1);
    wq[2][0] = load_w(2, 0);
    wq[2][1] = load_w(2, 1);
    __builtin_amdgcn_sched_barrier(0);
    copy_act(st2, 2);
    wq[3][0] = load_w(3, 0);
    wq[3][1] = load_w(3, 1);
    __builtin_amdgcn_sched_barrier(0);
    for (int jj = 0; jj < n_iter; jj += 4) {
        FNN_A8_ITER(0, st0, st3, jj);
        FNN_A8_ITER(1, st1, st0, jj + 1);
        FNN_A8_ITER(2, st2, st1, jj + 2);
        FNN_A8_ITER(3, st3, st2, jj + 3);
    }
#undef FNN_A8_ITER

    // add the K parts (integers: exact in any order); the stages are idle once every copy has landed
    if constexpr (KS > 1) {
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        int* red = (int*)st0;
        if (ks > 0) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 4; ++r) red[((((ks - 1) * RT + rt) * MB + mb) * 4 + r) * 64 + lane] = acc[mb][r];
        }
        __syncthreads();
        if (ks > 0) return;
#pragma unroll
        for (int k2 = 1; k2 < KS; ++k2)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[mb][r] += red[((((k2 - 1) * RT + rt) * MB + mb) * 4 + r) * 64 + lane];
    }

    // lane (li, lg) holds channels n0 .. n0+3 of row 16 mb + li
    const int n0 = row0 + 4 * lg;
    float ac[4];
    if constexpr (MODE != OUT_I32) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            ac[r] = load_as_f32(p.acol, (MOE ? (int64_t)expert * q.stride_scale_be : 0) + n0 + r, p.acol_dtype);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        int m = m_base + mb * 16 + li;     // output row; for gathered rows the token id
        int arow_idx = m;
        float wroute = 1.f;
        if constexpr (MOE) {
            m = token_of(mb * 16 + li);
            if (m >= q.num_valid) continue;
            arow_idx = m / q.top_k;
            if (q.mul_w) wroute = load_as_f32(q.topk_w, m, q.topk_w_dtype);
        } else {
            if (m >= p.M) continue;
        }
        if constexpr (MODE == OUT_I32) {
            int32_t* dst = (int32_t*)p.out + (int64_t)m * p.ldc + n0;
            if ((p.ldc & 3) == 0 && ((uintptr_t)p.out & 15) == 0) *(v4i*)dst = acc[mb];
            else {
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[r] = acc[mb][r];
            }
        } else {
            const float ar = load_as_f32(p.arow, arow_idx, p.arow_dtype);
            uint32_t h[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float f = rounded_f32(((float)acc[mb][r] * ar) * ac[r]);
                if constexpr (MOE) {
                    if (q.mul_w) f = rounded_f32(f * wroute);
                }
                h[r] = MODE == OUT_F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f);
            }
            uint16_t* dst = (uint16_t*)p.out + (int64_t)m * p.ldc + n0;
            if ((p.ldc & 3) == 0 && ((uintptr_t)p.out & 7) == 0) {
                *(v2u*)dst = v2u{(h[0] & 0xFFFFu) | (h[1] << 16), (h[2] & 0xFFFFu) | (h[3] << 16)};
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[r] = (uint16_t)h[r];
            }
        }
    }
}

template <int MODE>
static bool launch_a8_panel_t(A8W8Args& p, hipStream_t st) {
    if (p.M > kA8PanelRowsNarrow || p.N % 16 != 0 || p.K % 32 != 0 || p.K < 8 * 128 || p.lda % 16 != 0 || p.ldb % 16 != 0 ||
        ((uintptr_t)p.a % 16) != 0 || ((uintptr_t)p.b % 16) != 0)
        return false;
    // Rows per workgroup (16 rt) and 16-row activation blocks per pass (RT = 4 takes 2 or 4, RT = 2 takes 1 or
    // 2, RT = 1 takes 1; fewer blocks than the rows allow make more, cheaper passes): the cheapest under the model of the weight-only panel kernel - a workgroup costs
    // about eight loop iterations of start-up and wind-down plus ceil(KT * rt / 8) iterations, dearer with
    // more row blocks, and the grid runs in rounds of 256 workgroups.
    int rt = 0, mb = 1;
    double best = 0.0;
    const int KT = (int)((p.K + 127) / 128);
    static const double per_iter[5] = {0, 1.0, 1.2, 0, 1.8};
    const int need = p.M <= 16 ? 1 : p.M <= 32 ? 2 : 4;
    for (int cand = 4; cand >= 1; cand >>= 1) {
        if (p.N % (16 * cand) != 0) continue;
        const int m_lo = cand == 4 ? 2 : 1;                   // the kernel is built for (4,4) (4,2) (2,2) (2,1) (1,1)
        for (int m = cand == 1 ? 1 : cand; m >= m_lo; m >>= 1) {
            if (m > need && m > m_lo) continue;               // more row blocks than there are rows
            const int64_t wgs = (int64_t)(p.N / (16 * cand)) * ((p.M + m * 16 - 1) / (m * 16));
            double cost = (double)((wgs + 255) / 256) * (8.0 + (double)((KT * cand + 7) / 8) * per_iter[m]);
            // Weight rows a multiple of 8 KiB apart: a workgroup's 64 rows then start in the same few memory channels,
            // and 32-row workgroups stream them better (forced pairs under a captured graph, M=16, K=8192, 64 / 32
            // rows per workgroup, us: N=12288 25.6 / 24.1, N=16384 33.8 / 26.1, N=28672 50.8 / 47.0, N=32768 58.5 /
            // 49.8; at K=4096 and K=11008 the 64-row workgroups are level or ahead: N=16384 14.9 / 16.3, 38.6 / 38.8)
            // (measured for up to 16 rows only)
            if (cand == 4 && p.M <= 16 && p.ldb % 8192 == 0) cost *= 1.3;
            if (rt == 0 || cost < best) { best = cost; rt = cand; mb = m; }
        }
    }
    const int passes = (p.M + mb * 16 - 1) / (mb * 16);
    const int tiles = p.N / (16 * rt);
    const dim3 grid(((tiles + 7) / 8) * 8 * passes), block(512);
    note_kernel("gemm_a8w8_panel_kernel", mb, rt);
    if (rt == 4) {
        if (mb == 2) gemm_a8w8_panel_kernel<2, 4, MODE><<<grid, block, 0, st>>>(p, passes, MoeArgs{});
        else gemm_a8w8_panel_kernel<4, 4, MODE><<<grid, block, 0, st>>>(p, passes, MoeArgs{});
    } else if (rt == 2) {
        if (mb == 1) gemm_a8w8_panel_kernel<1, 2, MODE><<<grid, block, 0, st>>>(p, passes, MoeArgs{});
        else gemm_a8w8_panel_kernel<2, 2, MODE><<<grid, block, 0, st>>>(p, passes, MoeArgs{});
    } else {
        gemm_a8w8_panel_kernel<1, 1, MODE><<<grid, block, 0, st>>>(p, passes, MoeArgs{});
    }
    return true;
}

template <int MODE>
static bool launch_skinny_t(A8W8Args& p, hipStream_t st) {
    // a single activation row gains nothing from shared slabs (measured 14.0 against 16.5 us at K = N = 8192)
    // (it takes the shared-slab kernel all the same when K is no multiple of 128, which only that one handles)
    const bool skinny_ok = p.M <= 64 && p.K % 128 == 0 && p.lda % 16 == 0 && p.ldb % 16 == 0 &&
                           ((uintptr_t)p.a % 16) == 0 && ((uintptr_t)p.b % 16) == 0;
    // Up to 16 rows, two kinds of shapes on which this kernel (16 channels per workgroup, K split over its waves,
    // no barrier per slab) beats the shared-slab kernel; both kernels timed over 60 shapes under a captured graph
    // with rotating weights, shared-slab / this kernel, us.  Few workgroups - N <= 4096, one per CU or fewer, at any
    // K (N=K=2048 4.6 / 3.5, N=K=4096 M=2..8 6.7 / 6.3, M=16 7.1 / 6.8, N=4096 K=11008 11.5 / 10.5, N=1536 K=8960
    // 7.8 / 6.0), or N <= 8192 with K <= 3072 (N=8192 K=2048 6.3 / 5.3): the call is a handful of latencies.  And up
    // to 8 rows of K >= 8192 over N >= 8192: N=12288 25.6 / 20.0, N=16384 33.7 / 25.1, N=28672 49.3 / 40.1, N=32768
    // 58.4 / 44.7; K=11008 N=12288 33.3 / 28.7.  Elsewhere the shared-slab kernel is level or ahead (N=4608 K=4096
    // 6.8 / 7.2, N=12288 K=4096 11.9 / 13.5, N=28672 K=4096 23.7 / 25.9; from 17 rows on everywhere).
    const bool few_workgroups = p.N <= 4096 || (p.N <= 8192 && p.K <= 3072);
    const bool long_rows = p.M <= 8 && p.K >= 8192 && p.N >= 8192;
    const bool prefer = skinny_ok && p.M <= 16 && (few_workgroups || long_rows);
    if (!prefer && (p.M > 1 || p.K % 128 != 0) && launch_a8_panel_t<MODE>(p, st)) return true;
    if (!skinny_ok) return false;
    const dim3 grid((p.N + 15) / 16), block(kSkWaves * 64);
    note_kernel("gemm_a8w8_skinny_kernel", (p.M + 15) / 16);
    if (p.M <= 16) gemm_a8w8_skinny_kernel<1, MODE><<<grid, block, 0, st>>>(p);
    else if (p.M <= 32) gemm_a8w8_skinny_kernel<2, MODE><<<grid, block, 0, st>>>(p);
    else if (p.M <= 48) gemm_a8w8_skinny_kernel<3, MODE><<<grid, block, 0, st>>>(p);
    else gemm_a8w8_skinny_kernel<4, MODE><<<grid, block, 0, st>>>(p);
    return true;
}

// ------------------------------------------------------------------ mixture of experts
// Any shape: one thread per output value, the row dotted byte by byte (4 at a time where aligned).
template <int MODE>
__global__ __launch_bounds__(256) void moe_a8w8_any_kernel(const A8W8Args p, const MoeArgs q) {
    const int sidx = blockIdx.x;
    if (sidx >= q.ntpp[0]) return;
    const int tok = q.sorted_ids[sidx];
    if (tok >= q.num_valid) return;
    const int n = blockIdx.y * 256 + threadIdx.x;
    if (n >= p.N) return;
    const int expert = q.expert_ids[sidx / q.block_m];
    const int8_t* a = p.a + (int64_t)(tok / q.top_k) * p.lda;
    const int8_t* b = p.b + (int64_t)expert * q.stride_be + (int64_t)n * p.ldb;
    int acc = 0;
    int k = 0;
    if ((((uintptr_t)a | (uintptr_t)b) & 3) == 0)
        for (; k + 4 <= p.K; k += 4) acc = __builtin_amdgcn_sdot4(*(const int*)(a + k), *(const int*)(b + k), acc, false);
    for (; k < p.K; ++k) acc += (int)a[k] * (int)b[k];
    const float ar = load_as_f32(p.arow, tok / q.top_k, p.arow_dtype);
    const float ac = load_as_f32(p.acol, (int64_t)expert * q.stride_scale_be + n, p.acol_dtype);
    float f = rounded_f32(((float)acc * ar) * ac);
    if (q.mul_w) f = rounded_f32(f * load_as_f32(q.topk_w, tok, q.topk_w_dtype));
    ((uint16_t*)p.out)[(int64_t)tok * p.ldc + n] = (uint16_t)(MODE == OUT_F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f));
}

template <int MODE>
static bool launch_moe_t(A8W8Args& p, const MoeArgs& q, hipStream_t st) {
    const bool fast = p.N % 16 == 0 && p.K % 32 == 0 && p.K >= 8 * 128 && p.lda % 16 == 0 && p.ldb % 16 == 0 &&
                      q.stride_be % 16 == 0 && ((uintptr_t)p.a % 16) == 0 && ((uintptr_t)p.b % 16) == 0 &&
                      q.block_m % 16 == 0 && q.EM % q.block_m == 0;
    if (!fast) {
        note_kernel("moe_a8w8_any_kernel");
        moe_a8w8_any_kernel<MODE><<<dim3(q.EM, (p.N + 255) / 256), dim3(256), 0, st>>>(p, q);
        return true;
    }
    // a pass must stay within one expert's block: 16 * MB rows divide block_m
    const int mb_max = q.block_m % 64 == 0 ? 4 : q.block_m % 32 == 0 ? 2 : 1;
    int rt = 0;
    double best = 0.0;
    for (int cand = 4; cand >= 1; cand >>= 1) {
        if (p.N % (16 * cand) != 0) continue;
        if (cand == 4 && mb_max < 2) continue;          // RT = 4 shares slabs of at least 32 rows
        const int t = p.N / (16 * cand);
        const double fill = (double)t / (((t + 255) / 256) * 256);
        const double score = fill * (cand == 4 ? 1.0 : cand == 2 ? 0.9 : 0.6);
        if (score > best) { best = score; rt = cand; }
    }
    const int mb = rt == 4 ? (mb_max >= 4 ? 4 : 2) : rt == 2 ? (mb_max >= 2 ? 2 : 1) : 1;
    const int passes = q.EM / (mb * 16);
    const int tiles = p.N / (16 * rt);
    const dim3 grid(((tiles + 7) / 8) * 8 * passes), block(512);
    note_kernel("gemm_a8w8_panel_kernel(moe)", mb, rt);
    if (rt == 4) {
        if (mb == 2) gemm_a8w8_panel_kernel<2, 4, MODE, true><<<grid, block, 0, st>>>(p, passes, q);
        else gemm_a8w8_panel_kernel<4, 4, MODE, true><<<grid, block, 0, st>>>(p, passes, q);
    } else if (rt == 2) {
        if (mb == 1) gemm_a8w8_panel_kernel<1, 2, MODE, true><<<grid, block, 0, st>>>(p, passes, q);
        else gemm_a8w8_panel_kernel<2, 2, MODE, true><<<grid, block, 0, st>>>(p, passes, q);
    } else {
        gemm_a8w8_panel_kernel<1, 1, MODE, true><<<grid, block, 0, st>>>(p, passes, q);
    }
    return true;
}

bool launch_a8w8_moe(A8W8Args& p, const MoeArgs& q, int mode, hipStream_t st) {
    return mode == OUT_F16 ? launch_moe_t<OUT_F16>(p, q, st) : launch_moe_t<OUT_BF16>(p, q, st);
}

bool launch_a8w8_skinny(A8W8Args& p, int mode, hipStream_t st) {
    if (mode == OUT_I32) return launch_skinny_t<OUT_I32>(p, st);
    return mode == OUT_F16 ? launch_skinny_t<OUT_F16>(p, st) : launch_skinny_t<OUT_BF16>(p, st);
}

}  // namespace fnn
