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

enum { OUT_F16 = 0, OUT_BF16 = 1, OUT_I32 = 2 };

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


// ------------------------------------------------------------------ pipelined main kernel
// K % 256 == 0.  Slabs of 64 bytes of K; four static LDS stages form a ring, the copy of
// slab j+3 is issued while slab j-1 is being finished, so a copy has three slabs of MFMA time
// (about 1 us) to land.  One barrier per slab, placed at the start of the LAST k-step of the
// previous slab: by then every fragment of that slab is in registers, which frees its stage
// for the copy issued right after the barrier, and the barrier also publishes the next slab,
// whose first fragments are read while the last MFMAs of the previous slab run.  Fragments
// are double-buffered in registers; LDS reads and MFMAs are interleaved one to one.
//
// LDS rows are 64 bytes (4 chunks of 16); chunk c of row r is stored at slot c ^ ((r >> 1) & 3),
// which spreads the 8 rows read together over all 32 banks.
constexpr int BK4 = 64;

template <int BM, int BN>
struct Stage4 {
    char bytes[(BM + BN) * BK4];
};

template <int BM, int BN, int MODE>
__global__ __launch_bounds__(256) void gemm_a8w8_mfma4_kernel(const A8W8Args p) {
    constexpr int NWAVES = 4;
    constexpr int WTM = BM / 2, WTN = BN / 2;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int ROWS = BM + BN;
    constexpr int NLD = ROWS / (16 * NWAVES);   // a wave-load covers 16 rows of 64 bytes
    static_assert(ROWS % (16 * NWAVES) == 0 && BM % (16 * NWAVES) == 0, "tile rows must split evenly");

    __shared__ __attribute__((aligned(1024))) Stage4<BM, BN> st0;
    __shared__ __attribute__((aligned(1024))) Stage4<BM, BN> st1;
    __shared__ __attribute__((aligned(1024))) Stage4<BM, BN> st2;
    __shared__ __attribute__((aligned(1024))) Stage4<BM, BN> st3;
    __shared__ __attribute__((aligned(16))) float sc_row[BM];   // alpha_row of the tile's rows, fp32
    __shared__ __attribute__((aligned(16))) float sc_col[BN];   // alpha_col of the tile's columns

    const int xcd = blockIdx.x & 7;
    const int t = xcd * p.tiles_per_xcd + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= p.tiles_per_xcd || t >= p.tiles_m * p.tiles_n) return;
    const int tile_m = t % p.tiles_m;
    const int tile_n = t / p.tiles_m;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave & 1;
    const int wn = wave >> 1;

    // Scales of the tile go to LDS as fp32 before anything else is in flight (their loads are the
    // oldest, so waiting for them does not wait for the copies issued below); the epilogue then
    // needs no global loads at all.
    if constexpr (MODE != OUT_I32) {
        for (int e = threadIdx.x; e < BM + BN; e += 256) {
            const bool is_row = e < BM;
            const int idx = is_row ? min(m0 + e, p.M - 1) : min(n0 + e - BM, p.N - 1);
            const float v = load_as_f32(is_row ? p.arow : p.acol, idx, is_row ? p.arow_dtype : p.acol_dtype);
            if (is_row) sc_row[e] = v; else sc_col[e - BM] = v;
        }
    }

    // copy plan: load j of this wave fills rows rg*16 .. rg*16+15, rg = j*NWAVES + wave; lane L
    // writes slot (L & 3) of row rg*16 + (L >> 2), which holds logical chunk (L & 3) ^ ((row >> 1) & 3)
    const int lrow = lane >> 2;
    const int lchunk = (lane & 3) ^ ((lrow >> 1) & 3);
    uint32_t goff[NLD];
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
        const int rr = (j * NWAVES + wave) * 16 + lrow;
        if (rr < BM) goff[j] = (uint32_t)min(m0 + rr, p.M - 1) * (uint32_t)p.lda + lchunk * 16;
        else goff[j] = (uint32_t)min(n0 + rr - BM, p.N - 1) * (uint32_t)p.ldb + lchunk * 16;
    }
    auto issue_loads = [&](char* stage_bytes, int kt) {
        const char* a_slab = (const char*)p.a + (int64_t)kt * BK4;
        const char* b_slab = (const char*)p.b + (int64_t)kt * BK4;
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            char* dst = stage_bytes + (j * NWAVES + wave) * (16 * BK4);
            const char* src = ((j * NWAVES) * 16 < BM ? a_slab : b_slab) + goff[j];
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)dst, 16, 0, 0);
        }
    };

    // read plan: lane reads row (lane & 31) of a fragment, logical chunk 2*s + (lane >> 5)
    const int frow = lane & 31;
    const int hsel = lane >> 5;
    int rd_off[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) rd_off[s2] = frow * BK4 + (((2 * s2 + hsel) ^ ((frow >> 1) & 3)) * 16);
    const int a_base = wm * WTM * BK4;
    const int b_base = (BM + wn * WTN) * BK4;

    v16i acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    v4i wf[2][FN], af[2][FM];   // fragment double buffer, indexed by k-step parity
    auto read_frags = [&](const char* stage_bytes, int s2) {
#pragma unroll
        for (int i = 0; i < FN; ++i) wf[s2][i] = *(const v4i*)(stage_bytes + b_base + i * 32 * BK4 + rd_off[s2]);
#pragma unroll
        for (int j = 0; j < FM; ++j) af[s2][j] = *(const v4i*)(stage_bytes + a_base + j * 32 * BK4 + rd_off[s2]);
    };
    auto mfmas = [&](int s2) {
#pragma unroll
        for (int i = 0; i < FN; ++i)
#pragma unroll
            for (int j = 0; j < FM; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[s2][i], af[s2][j], acc[i][j], 0, 0, 0);
    };
    // ask the scheduler for: MFMA, LDS read, MFMA, LDS read, ... then the remaining MFMAs
    auto interleave = [&]() {
#pragma unroll
        for (int q = 0; q < FN + FM; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, FN * FM - (FN + FM), 0);
    };

    const int KT = p.K / BK4;   // multiple of 4, >= 8 (checked on the host)
    // Wait until at most `newer` of this wave's copies are outstanding and all its LDS reads have
    // returned, then cross the workgroup barrier.  A bare s_barrier is used: __syncthreads() would
    // add a fence that waits for every outstanding copy and collapse the ring to depth one.
    auto wait_barrier = [&](int newer) {
        asm volatile("" ::: "memory");
        if (newer == 2 * NLD) __builtin_amdgcn_s_waitcnt(0x0070 | ((2 * NLD) & 15) | (((2 * NLD) >> 4) << 14));
        else if (newer == NLD) __builtin_amdgcn_s_waitcnt(0x0070 | (NLD & 15) | ((NLD >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // One slab = two k-steps.  Step 0 overlaps the fragment reads of step 1.  Step 1 (the last of
    // the slab) first waits for the next slab and crosses the barrier, then reads the next slab's
    // first fragments and re-arms the stage it has just finished, all under its own MFMAs.
    //   newer  : copies that may stay outstanding at the barrier (-1: there is no next slab)
    //   refill : slab index to copy into `cur`, or -1
    auto slab = [&](char* cur, const char* nxt, int newer, int refill) {
        read_frags(cur, 1);
        mfmas(0);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
        if (newer >= 0) {
            wait_barrier(newer);
            read_frags(nxt, 0);
            if (refill >= 0) issue_loads(cur, refill);
        }
        mfmas(1);
        if (newer >= 0) interleave();
        __builtin_amdgcn_sched_barrier(0);
    };

    issue_loads(st0.bytes, 0);
    issue_loads(st1.bytes, 1);
    issue_loads(st2.bytes, 2);
    issue_loads(st3.bytes, 3);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | ((3 * NLD) & 15) | (((3 * NLD) >> 4) << 14));   // slab 0 landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_frags(st0.bytes, 0);
    int kt = 0;
    for (; kt + 8 <= KT; kt += 4) {
        slab(st0.bytes, st1.bytes, 2 * NLD, kt + 4);
        slab(st1.bytes, st2.bytes, 2 * NLD, kt + 5);
        slab(st2.bytes, st3.bytes, 2 * NLD, kt + 6);
        slab(st3.bytes, st0.bytes, 2 * NLD, kt + 7);
    }
    // last four slabs: nothing left to copy, the outstanding count runs down
    slab(st0.bytes, st1.bytes, 2 * NLD, -1);
    slab(st1.bytes, st2.bytes, NLD, -1);
    slab(st2.bytes, st3.bytes, 0, -1);
    slab(st3.bytes, st3.bytes, -1, -1);

    // ---- epilogue ----
    // acc[i][j][r]: n = wn0 + i*32 + 8*(r/4) + 4*(lane>>5) + (r&3),  m = wm0 + j*32 + (lane&31).
    // A lane owns 4 consecutive n of ONE row, so storing straight from registers would touch 32
    // rows per instruction with 16 bytes each.  Instead every wave transposes its sub-tile through
    // LDS (the ring stage with its own index, free now) 64 rows at a time and writes whole rows:
    // 16 bytes per lane, consecutive lanes on consecutive addresses.
    const int wm0 = m0 + wm * WTM;
    const int wn0 = n0 + wn * WTN;
    if constexpr (MODE == OUT_I32) {
        const bool vec_ok = (p.ldc & 3) == 0;
#pragma unroll
        for (int j = 0; j < FM; ++j) {
            const int m = wm0 + j * 32 + frow;
#pragma unroll
            for (int i = 0; i < FN; ++i) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = wn0 + i * 32 + 8 * g + 4 * hsel;
                    if (m >= p.M || n >= p.N) continue;
                    int32_t* o = (int32_t*)p.out + (int64_t)m * p.ldc + n;
                    if (n + 3 < p.N && vec_ok) {
                        *(v4i*)o = v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                                       acc[i][j][4 * g + 3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < p.N) o[e] = acc[i][j][4 * g + e];
                    }
                }
            }
        }
    } else {
        constexpr int TSTRIDE = WTN * 2 + 16;      // bytes per staged row; the pad staggers the banks
        constexpr int PR = WTN * 2 / 16;           // 16-byte pieces per row
        static_assert(64 * TSTRIDE <= (int)sizeof(Stage4<BM, BN>), "transpose buffer must fit a stage");
        char* tbuf = wave == 0 ? st0.bytes : wave == 1 ? st1.bytes : wave == 2 ? st2.bytes : st3.bytes;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070);   // all copies and LDS reads of this wave are done
        __builtin_amdgcn_s_barrier();         // ... and everybody else's: the stages are free
        asm volatile("" ::: "memory");
        const bool vec_ok = (p.ldc & 7) == 0;
#pragma unroll
        for (int jc = 0; jc < FM; jc += 2) {
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int j = jc + jj;
                const float ar = sc_row[wm * WTM + j * 32 + frow];
#pragma unroll
                for (int i = 0; i < FN; ++i) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int nl = i * 32 + 8 * g + 4 * hsel;   // column within the wave tile
                        const v4f ac = *(const v4f*)&sc_col[wn * WTN + nl];
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = ((float)acc[i][j][4 * g + e] * ar) * ac[e];
                        uint32_t lo, hi;
                        if constexpr (MODE == OUT_BF16) {
                            lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[0], v[1]}, v2bf));
                            hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[2], v[3]}, v2bf));
                        } else {
                            lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[0], v[1]}, v2h));
                            hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[2], v[3]}, v2h));
                        }
                        *(v2u*)(tbuf + (jj * 32 + frow) * TSTRIDE + nl * 2) = v2u{lo, hi};
                    }
                }
            }
            // rows jc*32 .. jc*32+63 of the wave tile are staged; write them out row by row
#pragma unroll
            for (int it = 0; it < (64 * PR + 63) / 64; ++it) {
                const int e = it * 64 + lane;
                const int row = e / PR, c = e % PR;
                if (e < 64 * PR) {
                    const v4u val = *(const v4u*)(tbuf + row * TSTRIDE + c * 16);
                    const int m = wm0 + jc * 32 + row;
                    const int n = wn0 + c * 8;
                    if (m < p.M && n < p.N) {
                        uint16_t* o = (uint16_t*)p.out + (int64_t)m * p.ldc + n;
                        if (n + 7 < p.N && vec_ok) {
                            __builtin_nontemporal_store(val, (v4u*)o);
                        } else {
#pragma unroll
                            for (int q = 0; q < 8; ++q)
                                if (n + q < p.N) o[q] = (uint16_t)(val[q >> 1] >> (16 * (q & 1)));
                        }
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
        if constexpr (MODE != OUT_I32) ar = load_as_f32(p.arow, m, p.arow_dtype);
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
    gemm_a8w8_mfma4_kernel<BM, BN, MODE><<<dim3(p.tiles_per_xcd * 8), dim3(256), 0, st>>>(p);
}

template <int MODE>
static void dispatch(A8W8Args& p, hipStream_t st, int force_bm, int force_bn) {
    // the MFMA kernel walks K in four-slab rounds of 64 bytes and addresses rows with 32-bit offsets
    const bool fast = p.K % 256 == 0 && p.K >= 512 && p.lda % 16 == 0 && p.ldb % 16 == 0 &&
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
    if (out_dtype == FNN_F16) dispatch<OUT_F16>(p, (hipStream_t)stream, g_force_bm, g_force_bn);
    else dispatch<OUT_BF16>(p, (hipStream_t)stream, g_force_bm, g_force_bn);
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
