// A8W8 GEMM for gfx950:  acc[m,n] = sum_k a[m,k] * b[n,k]  (int8 x int8 -> int32, exact),
// out = float(acc) * alpha_row[m] * alpha_col[n]  -> fp16 / bf16   (or the raw int32).
//
// Main kernel (K % 128 == 0, 16-byte aligned rows)
//   * one 256-thread workgroup (4 waves, 2x2) per BM x BN output tile, one workgroup per CU;
//   * K is walked in slabs of 128 bytes.  A slab of the a-rows and b-rows of the tile is
//     copied global -> LDS with direct-to-LDS 16-byte loads (no VGPR staging) into one of
//     two static LDS stages while the MFMAs of the previous slab run;
//   * both operands are K-contiguous, so a lane's 16-byte LDS read is directly one
//     v_mfma_i32_32x32x32_i8 operand.  The 16-byte chunks of each 128-byte LDS row are
//     XOR-swizzled with (row & 7) so that the 8 lanes served together hit 8 distinct
//     bank groups.  The swizzle is applied on the global side of the copy (the LDS side
//     of a direct-to-LDS load is linear in the lane id);
//   * the weight rows feed the MFMA "A" operand and the activation rows the "B"
//     operand, so a lane ends up with 4 consecutive n for one m: the epilogue scales in
//     fp32 and writes 8-byte (16-bit out) or 16-byte (int32 out) pieces;
//   * workgroup ids are remapped so that each XCD (ids congruent mod 8 share an L2) works
//     on a contiguous band of tiles with the m index fastest, which keeps the b-panel and
//     the whole a-panel slab of the moment resident in that XCD's L2.
//
// Any other shape takes a small guarded LDS kernel built on v_dot4_i32_i8.
//
// Reference for the semantics: flashnn/triton_kernels/gemm_a8w8.py:74-179.
#include "fnn_common.h"

namespace fnn {

constexpr int BK = 128;  // bytes of K per LDS slab row

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

enum { OUT_SCALED = 0, OUT_I32 = 1 };

template <int BM, int BN>
struct Stage {
    // a rows first, then b rows; every row is 128 bytes of K
    char bytes[(BM + BN) * BK];
};

struct A8W8Args {
    const int8_t* a;
    const int8_t* b;
    void* out;
    const void* arow;
    const void* acol;
    int M, N, K;
    int64_t lda, ldb, ldc;
    int out_dtype, arow_dtype, acol_dtype;
    int tiles_m, tiles_n, tiles_per_xcd;
};

template <int BM, int BN, int MODE>
__global__ __launch_bounds__(256) void gemm_a8w8_mfma_kernel(const A8W8Args p) {
    constexpr int NWAVES = 4;
    constexpr int WTM = BM / 2;        // wave tile extent in m
    constexpr int WTN = BN / 2;        // wave tile extent in n
    constexpr int FM = WTM / 32;       // 32x32 fragments along m per wave
    constexpr int FN = WTN / 32;
    constexpr int ROWS = BM + BN;      // LDS rows per stage
    constexpr int NLD = ROWS / (8 * NWAVES);  // direct-to-LDS loads per wave per slab
    static_assert(ROWS % (8 * NWAVES) == 0, "tile rows must split evenly over the waves");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");

    __shared__ __attribute__((aligned(1024))) Stage<BM, BN> stage0;
    __shared__ __attribute__((aligned(1024))) Stage<BM, BN> stage1;

    // ---- tile assignment (XCD-aware) ----
    const int xcd = blockIdx.x & 7;
    const int t = xcd * p.tiles_per_xcd + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= p.tiles_per_xcd || t >= p.tiles_m * p.tiles_n) return;
    const int tile_m = t % p.tiles_m;
    const int tile_n = t / p.tiles_m;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave & 1;   // wave position along m
    const int wn = wave >> 1;  // wave position along n

    // ---- global -> LDS copy plan ----
    // load j of this wave fills LDS rows rg*8 .. rg*8+7 with rg = j*NWAVES + wave;
    // lane L writes physical chunk (L & 7) of row rg*8 + (L >> 3), which must hold the
    // logical chunk (L & 7) ^ (row & 7) = (L & 7) ^ (L >> 3).
    const int lrow = lane >> 3;
    const int lchunk = (lane & 7) ^ lrow;
    // Row offsets fit 32 bits (checked on the host), so a load is "uniform base + lane offset".
    uint32_t goff[NLD];
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
        const int rr = (j * NWAVES + wave) * 8 + lrow;
        if (rr < BM) goff[j] = (uint32_t)min(m0 + rr, p.M - 1) * (uint32_t)p.lda + lchunk * 16;
        else goff[j] = (uint32_t)min(n0 + rr - BM, p.N - 1) * (uint32_t)p.ldb + lchunk * 16;
    }

    auto issue_loads = [&](char* stage_bytes, int kt) {
        const char* a_slab = (const char*)p.a + (int64_t)kt * BK;
        const char* b_slab = (const char*)p.b + (int64_t)kt * BK;
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            char* dst = stage_bytes + (j * NWAVES + wave) * (8 * BK);
            // rows of one load are all a-rows or all b-rows: BM is a multiple of 8*NWAVES
            const char* src = ((j * NWAVES) * 8 < BM ? a_slab : b_slab) + goff[j];
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)dst, 16, 0, 0);
        }
        // keep the copies ahead of the MFMAs that follow: they need the whole compute phase to land
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- LDS read plan ----
    // lane reads row (lane & 31) of a fragment, logical chunk 2*s + (lane >> 5) for k-step s
    const int frow = lane & 31;
    const int hsel = lane >> 5;
    int rd_off[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) rd_off[s] = frow * BK + (((2 * s + hsel) ^ (frow & 7)) * 16);
    const int a_base = wm * WTM * BK;               // activation rows of this wave
    const int b_base = (BM + wn * WTN) * BK;        // weight rows of this wave

    v16i acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    auto compute = [&](const char* stage_bytes) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v4i wf[FN], af[FM];
#pragma unroll
            for (int i = 0; i < FN; ++i)
                wf[i] = *(const v4i*)(stage_bytes + b_base + i * 32 * BK + rd_off[s]);
#pragma unroll
            for (int j = 0; j < FM; ++j)
                af[j] = *(const v4i*)(stage_bytes + a_base + j * 32 * BK + rd_off[s]);
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], af[j], acc[i][j], 0, 0, 0);
        }
    };

    const int KT = p.K / BK;
    auto wait_and_sync = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's copies have landed
        __syncthreads();                     // everyone's have, and everyone left the other stage
    };
    // slab kt lives in stage (kt & 1); its copy is issued one compute phase ahead
    issue_loads(stage0.bytes, 0);
    int kt = 0;
    for (; kt + 2 < KT; kt += 2) {
        wait_and_sync();
        issue_loads(stage1.bytes, kt + 1);
        compute(stage0.bytes);
        wait_and_sync();
        issue_loads(stage0.bytes, kt + 2);
        compute(stage1.bytes);
    }
    wait_and_sync();
    if (kt + 1 < KT) {
        issue_loads(stage1.bytes, kt + 1);
        compute(stage0.bytes);
        wait_and_sync();
        compute(stage1.bytes);
    } else {
        compute(stage0.bytes);
    }

    // ---- epilogue ----
    // acc[i][j][r]: n = wn0 + i*32 + 8*(r/4) + 4*(lane>>5) + (r&3),  m = wm0 + j*32 + (lane&31)
    const int wm0 = m0 + wm * WTM;
    const int wn0 = n0 + wn * WTN;
#pragma unroll
    for (int j = 0; j < FM; ++j) {
        const int m = wm0 + j * 32 + frow;
        if (m >= p.M) continue;
        float ar = 1.f;
        if constexpr (MODE == OUT_SCALED) ar = load_as_f32(p.arow, m, p.arow_dtype);
#pragma unroll
        for (int i = 0; i < FN; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = wn0 + i * 32 + 8 * g + 4 * hsel;
                if (n >= p.N) continue;
                if constexpr (MODE == OUT_I32) {
                    int32_t* o = (int32_t*)p.out + (int64_t)m * p.ldc + n;
                    if (n + 3 < p.N && (p.ldc & 3) == 0) {
                        *(v4i*)o = v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                                       acc[i][j][4 * g + 3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < p.N) o[e] = acc[i][j][4 * g + e];
                    }
                } else {
                    uint32_t h[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float ac = n + e < p.N ? load_as_f32(p.acol, n + e, p.acol_dtype) : 0.f;
                        const float v = ((float)acc[i][j][4 * g + e] * ar) * ac;
                        h[e] = p.out_dtype == FNN_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
                    }
                    uint16_t* o = (uint16_t*)p.out + (int64_t)m * p.ldc + n;
                    if (n + 3 < p.N && (p.ldc & 3) == 0) {
                        *(v2u*)o = v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < p.N) o[e] = (uint16_t)h[e];
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------ guarded fallback
// 64x64 tile, 256 threads, each thread a 4x4 block; any M, N, K and strides.
template <int MODE>
__global__ __launch_bounds__(256) void gemm_a8w8_any_kernel(const A8W8Args p) {
    constexpr int T = 64, KS = 64, LD = KS + 4;
    __shared__ __attribute__((aligned(16))) int8_t sa[T * LD];
    __shared__ __attribute__((aligned(16))) int8_t sb[T * LD];
    const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    int acc[4][4] = {};
    for (int k0 = 0; k0 < p.K; k0 += KS) {
        for (int e = threadIdx.x; e < T * KS; e += 256) {
            const int r = e / KS, c = e % KS;
            const int k = k0 + c;
            sa[r * LD + c] = (m0 + r < p.M && k < p.K) ? p.a[(int64_t)(m0 + r) * p.lda + k] : (int8_t)0;
            sb[r * LD + c] = (n0 + r < p.N && k < p.K) ? p.b[(int64_t)(n0 + r) * p.ldb + k] : (int8_t)0;
        }
        __syncthreads();
#pragma unroll 4
        for (int c = 0; c < KS; c += 4) {
            int av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = *(const int*)&sa[(ty * 4 + i) * LD + c];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = *(const int*)&sb[(tx * 4 + j) * LD + c];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_sdot4(av[i], bv[j], acc[i][j], false);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= p.M) continue;
        float ar = 1.f;
        if constexpr (MODE == OUT_SCALED) ar = load_as_f32(p.arow, m, p.arow_dtype);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= p.N) continue;
            if constexpr (MODE == OUT_I32) {
                ((int32_t*)p.out)[(int64_t)m * p.ldc + n] = acc[i][j];
            } else {
                const float v = ((float)acc[i][j] * ar) * load_as_f32(p.acol, n, p.acol_dtype);
                store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
            }
        }
    }
}

// ------------------------------------------------------------------------ dispatch
struct TileChoice { int bm, bn; };

// Pick the tile whose last, partly filled round of workgroups costs least on 256 CUs.
static TileChoice choose_tile(int64_t M, int64_t N) {
    static const struct { int bm, bn; double eff; } cand[] = {
        {256, 256, 1.00}, {256, 192, 0.97}, {256, 128, 0.88}, {128, 128, 0.70}};
    double best = 1e300;
    TileChoice c{128, 128};
    for (const auto& t : cand) {
        const int64_t tiles = ((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn);
        const int64_t rounds = (tiles + 255) / 256;
        const double cost = (double)rounds * t.bm * t.bn / t.eff;
        if (cost < best) { best = cost; c = {t.bm, t.bn}; }
    }
    return c;
}

template <int BM, int BN, int MODE>
static void launch_mfma(A8W8Args& p, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int tiles = p.tiles_m * p.tiles_n;
    p.tiles_per_xcd = (tiles + 7) / 8;
    gemm_a8w8_mfma_kernel<BM, BN, MODE><<<dim3(p.tiles_per_xcd * 8), dim3(256), 0, st>>>(p);
}

template <int MODE>
static void dispatch(A8W8Args& p, hipStream_t st, int force_bm, int force_bn) {
    const bool fast = p.K % BK == 0 && p.lda % 16 == 0 && p.ldb % 16 == 0 &&
                      ((uintptr_t)p.a % 16) == 0 && ((uintptr_t)p.b % 16) == 0 &&
                      ((uintptr_t)p.out % 16) == 0 && (int64_t)p.M * p.lda < (1LL << 31) &&
                      (int64_t)p.N * p.ldb < (1LL << 31);
    if (!fast) {
        gemm_a8w8_any_kernel<MODE><<<dim3((p.N + 63) / 64, (p.M + 63) / 64), dim3(256), 0, st>>>(p);
        return;
    }
    TileChoice c = choose_tile(p.M, p.N);
    if (force_bm > 0) c = {force_bm, force_bn};
    if (c.bm == 256 && c.bn == 256) launch_mfma<256, 256, MODE>(p, st);
    else if (c.bm == 256 && c.bn == 192) launch_mfma<256, 192, MODE>(p, st);
    else if (c.bm == 256 && c.bn == 128) launch_mfma<256, 128, MODE>(p, st);
    else launch_mfma<128, 128, MODE>(p, st);
}

static int check_args(const char* fn, const void* out, const void* a, const void* b, int64_t M,
                      int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
    if (!out || !a || !b) { set_error("%s: null pointer argument", fn); return FNN_ERR_ARG; }
    if (M < 0 || N < 0 || K <= 0 || lda < K || ldb < K || ldc < N) {
        set_error("%s: bad shape M=%lld N=%lld K=%lld lda=%lld ldb=%lld ldc=%lld", fn, (long long)M,
                  (long long)N, (long long)K, (long long)lda, (long long)ldb, (long long)ldc);
        return FNN_ERR_ARG;
    }
    if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) {
        set_error("%s: shape too large", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    return FNN_OK;
}

}  // namespace fnn

using namespace fnn;

// Test hook: force a tile shape (bm, bn) for the next calls on any thread; (0, 0) = automatic.
static int g_force_bm = 0, g_force_bn = 0;
extern "C" int fnn_debug_force_a8w8_tile(int bm, int bn) {
    const bool ok = (bm == 0 && bn == 0) || (bm == 256 && (bn == 256 || bn == 192 || bn == 128)) ||
                    (bm == 128 && bn == 128);
    if (!ok) { set_error("fnn_debug_force_a8w8_tile: no such tile %dx%d", bm, bn); return FNN_ERR_ARG; }
    g_force_bm = bm;
    g_force_bn = bn;
    return FNN_OK;
}

extern "C" int fnn_gemm_a8w8(void* out, const void* a, const void* b, const void* alpha_row,
                             const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                             int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                             int alpha_col_dtype, void* stream) {
    int rc = check_args("fnn_gemm_a8w8", out, a, b, M, N, K, lda, ldb, ldc);
    if (rc != FNN_OK) return rc;
    if (!alpha_row || !alpha_col) { set_error("fnn_gemm_a8w8: null scale pointer"); return FNN_ERR_ARG; }
    if (!is16(out_dtype)) { set_error("fnn_gemm_a8w8: Output type must be float16 or bfloat16"); return FNN_ERR_UNSUPPORTED; }
    if (!isflt(alpha_row_dtype) || !isflt(alpha_col_dtype)) { set_error("fnn_gemm_a8w8: bad scale type"); return FNN_ERR_UNSUPPORTED; }
    if (M == 0 || N == 0) return FNN_OK;
    A8W8Args p{};
    p.a = (const int8_t*)a; p.b = (const int8_t*)b; p.out = out; p.arow = alpha_row; p.acol = alpha_col;
    p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.out_dtype = out_dtype; p.arow_dtype = alpha_row_dtype; p.acol_dtype = alpha_col_dtype;
    dispatch<OUT_SCALED>(p, (hipStream_t)stream, g_force_bm, g_force_bn);
    return check_launch("fnn_gemm_a8w8");
}

extern "C" int fnn_gemm_a8w8_i32(int32_t* acc, const void* a, const void* b, int64_t M, int64_t N,
                                 int64_t K, int64_t lda, int64_t ldb, int64_t ldc, void* stream) {
    int rc = check_args("fnn_gemm_a8w8_i32", acc, a, b, M, N, K, lda, ldb, ldc);
    if (rc != FNN_OK) return rc;
    if (M == 0 || N == 0) return FNN_OK;
    A8W8Args p{};
    p.a = (const int8_t*)a; p.b = (const int8_t*)b; p.out = acc;
    p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    dispatch<OUT_I32>(p, (hipStream_t)stream, g_force_bm, g_force_bn);
    return check_launch("fnn_gemm_a8w8_i32");
}
