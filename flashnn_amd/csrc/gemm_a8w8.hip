// A8W8 GEMM for gfx950:  acc[m,n] = sum_k a[m,k] * b[n,k]  (int8 x int8 -> int32, exact),
// out = float(acc) * alpha_row[m] * alpha_col[n]  -> fp16 / bf16   (or the raw int32).
//
// Main kernel (K % 32 == 0, K >= 512, 16-byte aligned rows)
//   * one 256-thread workgroup (4 waves, 2x2) per BM x BN output tile; one workgroup per CU for the
//     256-row tiles, two for the 64x128 tile and for the pair version of the 128x128 tile;
//   * K is walked in slabs of 128 bytes.  A slab of the a-rows and b-rows of the tile is
//     copied global -> LDS with direct-to-LDS 16-byte loads (no VGPR staging) into a ring of
//     LDS stages, one or two slabs ahead of the MFMAs;
//   * both operands are K-contiguous, so a lane's 16-byte LDS read is directly one
//     v_mfma_i32_16x16x64_i8 operand (with random operands the device sustains a fifth more of
//     these than of the 32x32x32 shape: 4.0 against 3.35 POP/s).  The 16-byte chunks of each
//     128-byte LDS row are XOR-swizzled with ((row >> 1) & 7) so that the 16 lanes served together
//     hit distinct banks.  The swizzle is applied on the global side of the copy (the LDS side
//     of a direct-to-LDS load is linear in the lane id);
//   * the weight rows feed the MFMA "A" operand and the activation rows the "B"
//     operand, so a lane ends up with 4 consecutive n for one m: the epilogue scales in
//     fp32, transposes through LDS and writes whole rows;
//   * workgroup ids are remapped so that each XCD (ids congruent mod 8 share an L2) works
//     on a contiguous band of tiles, numbered so that the workgroups it runs at a time cover
//     8 tile rows x 4 tile columns and share their operand rows through that XCD's L2.
//
// Any other shape takes a small guarded LDS kernel built on v_dot4_i32_i8.
//
// Reference for the semantics: flashnn/triton_kernels/gemm_a8w8.py:74-179.
#include <type_traits>

#include "a8w8_common.h"

#include <atomic>

// The scaled output is two fp32 multiplications and one rounding to 16 bits, each rounded on its
// own as in the reference's torch path.
#pragma clang fp contract(off)

namespace fnn {

constexpr int BK = 128;  // bytes of K per LDS slab row

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;



// ------------------------------------------------------------------ main MFMA kernel
// K % 32 == 0, K >= 512.  K is walked in slabs of 128 bytes: every row piece a copy fetches
// is one full 128-byte line, which is what the L2 -> LDS path needs to run at speed (64-byte
// pieces reach little more than half the rate).  The LDS holds a ring of stages per operand.  The
// 256x192 tile has three for the b-rows (the weights, streamed from HBM, copied two slabs ahead) and
// two for the a-rows (L2 hits after their first use, copied one slab ahead): 2*BM + 3*BN rows of 128
// bytes = 136 KB.  The smaller tiles have room for three stages of both and copy both two slabs ahead
// (3 to 20 % faster).  There is one barrier per slab; the loop around it is described where it is written.
// Chunk c (16 bytes) of LDS row r is stored at slot c ^ ((r >> 1) & 7).  A 16-byte LDS read serves
// 16 lanes (16 consecutive rows, same chunk) per cycle out of 64 banks = 256 bytes; two rows fill
// that period, so rows of equal parity must land in 8 different slots.  (r & 7 instead gives
// two-way conflicts: measured 8 instead of 4 cycles per read.)  The swizzle is applied on the
// global side of the copy; the LDS side of a direct-to-LDS load is linear in the lane id.

// An LDS stage that exists only in some instantiations (a zero-length array is not allowed).
template <bool HAS, int BYTES>
struct OptionalStage {
    static __device__ __forceinline__ char* get() {
        __shared__ __attribute__((aligned(1024))) char buf[BYTES];
        return buf;
    }
};
template <int BYTES>
struct OptionalStage<false, BYTES> {
    static __device__ __forceinline__ char* get() { return nullptr; }
};

// SPLIT: the workgroups of the grid are units, kparts per tile, each the tile's product over its own range
// of K (k_chunk bytes per row, a multiple of the slab; the last part takes the rest).  A unit that is done
// counts itself arrived at the tile's counter.  If it is the last to arrive and finds every other unit's
// accumulators complete in the workspace, it adds them to its registers and goes on to the ordinary
// epilogue.  Otherwise it stores its accumulators, as they lie in registers, in its slot, counts the slot
// complete, and leaves - unless that was the last of all kparts slots: then it is the one that adds up the
// others.  Exactly one unit per tile does, whatever the order; every slot it reads was complete before the
// count that chose it; nobody waits for anybody.  Integer sums do not depend on the order, so the result is
// the unsplit kernel's bit for bit.  The unit that adds up sets the counter back to zero: the counters are
// zero whenever no call is in flight.
// MOE: the mixture-of-experts form for many routed rows per expert (flashnn/triton_kernels/fused_moe_a8w8.py:37-173).
// The M dimension is the list of sorted routed rows (moe.EM of them, padded per expert to blocks of moe.block_m, a
// multiple of BM): tile row r multiplies activation row sorted_ids[r] / top_k with the weight matrix of the
// expert its block belongs to, and the result goes to output row sorted_ids[r], times the routing weight on
// request.  Tiles beyond the rows in use return at once; padding rows read activation row 0 and store nothing.
template <int BM, int BN, int MODE, bool PAIR = false, int WGM = 2, bool SPLIT = false, bool MOE = false>
__global__ __launch_bounds__(WGM * 128) void gemm_a8w8_ring_kernel(const A8W8Args p, const MoeArgs moe) {
    static_assert(!MOE || (!SPLIT && MODE != OUT_I32), "the gathered form has no split and no raw output");
    // WGM x 2 waves.  Only WGM = 2 (one wave per SIMD) is instantiated: with WGM = 4 the two waves of a SIMD
    // meet at the same barrier every slab and never filled each other's gaps (256x192: 81.6 us with four
    // waves, 83.9 with eight; never faster on any shape tried).
    constexpr int NWAVES = WGM * 2, NT = NWAVES * 64;
    constexpr int WTM = BM / WGM, WTN = BN / 2;
    constexpr int FM = WTM / 16, FN = WTN / 16;   // 16x16 fragments per wave tile
    constexpr int HN = FN / 2;
    static_assert(WTM % 16 == 0 && WTN % 32 == 0, "wave tile must split into 16-row fragments, the weight rows in two halves");
    constexpr int NLA = BM / (8 * NWAVES);   // a wave-load covers 8 rows of 128 bytes
    constexpr int NLB = BN / (8 * NWAVES);
    static_assert(BM % (8 * NWAVES) == 0 && BN % (8 * NWAVES) == 0, "tile rows must split evenly");

    __shared__ __attribute__((aligned(1024))) char sa0[BM * BK];
    __shared__ __attribute__((aligned(1024))) char sa1[BM * BK];
    // tiles too large for three stages of both operands give the third stage to the b-rows (the
    // weights, streamed from HBM) and copy the a-rows (L2 hits after their first use) one slab ahead
    // PAIR (128x128 tile, more than 256 tiles): the same arrangement although three stages of both would
    // fit - with two a-stages the tile needs exactly 80 KB, and two workgroups share a CU: each one's
    // prologue, epilogue and barrier waits then run under the other's MFMAs (17 to 25 % faster).  With at
    // most 256 tiles every workgroup has a CU to itself and the three-stage version is the faster one
    // (by 3 % at K = 8192, by 20 % at K = 18944).
    static_assert(!PAIR || 2 * ((2 * BM + 3 * BN) * BK) <= 160 * 1024, "a pair of workgroups must fit the LDS");
    constexpr bool BDEEP = 3 * (BM + BN) * BK + 4 * (BM + BN) + 1024 > 160 * 1024 || PAIR;
    char* const sa2 = OptionalStage<!BDEEP, BM * BK>::get();   // no third a-stage, and no LDS for it, where BDEEP
    __shared__ __attribute__((aligned(1024))) char sb0[BN * BK];
    __shared__ __attribute__((aligned(1024))) char sb1[BN * BK];
    // a third b-stage where the tile leaves room for it (3 * (BM + BN) rows <= 160 KB): the b-rows are
    // then copied two slabs ahead like the a-rows; with two stages their copy has exactly one slab
    // to land, which is about the loaded L2 latency
    constexpr int NSB = 3 * (BM + BN) * BK + 4 * (BM + BN) + 1024 <= 160 * 1024 ? 3 : 2;
    __shared__ __attribute__((aligned(1024))) char sb2[NSB == 3 || BDEEP ? BN * BK : 16];
    // alpha_row of the tile's rows and alpha_col of its columns as fp32: staged only before the epilogue, in
    // the third b-stage, which is free by then and which the epilogue's transposition does not use
    static_assert(NSB == 3 || BDEEP, "the scales live in the third b-stage");
    float* const sc_row = (float*)sb2;
    float* const sc_col = sc_row + BM;

    const int xcd = blockIdx.x & 7;
    const int unit = xcd * p.tiles_per_xcd + (blockIdx.x >> 3);   // (tiles_per_xcd counts units where SPLIT)
    if ((blockIdx.x >> 3) >= p.tiles_per_xcd || unit >= p.tiles_m * p.tiles_n * (SPLIT ? p.kparts : 1)) return;
    // the units of a tile are neighbours in this numbering: they run on one XCD, at about the same time
    const int t = SPLIT ? unit / p.kparts : unit;
    const int kpart = SPLIT ? unit - t * p.kparts : 0;
    const int8_t* const pa = SPLIT ? p.a + (int64_t)kpart * p.k_chunk : p.a;
    const int8_t* pb = SPLIT ? p.b + (int64_t)kpart * p.k_chunk : p.b;
    // (the last part takes what the others leave: a few slabs more, so that it arrives last as a rule)
    const int Kl = SPLIT ? (kpart == p.kparts - 1 ? p.K - kpart * p.k_chunk : p.k_chunk) : p.K;
    // tiles are numbered in groups of GN tile columns, the column fastest within a group: the 32 workgroups
    // an XCD runs at a time then cover 32 / GN tile rows x GN tile columns whatever M is, and fetch
    // (32 / GN) * BM + GN * BN operand rows per slab into its L2 instead of tiles_m*BM + BN.  GN = 8 for the tiles
    // of 192 and 256 columns, 4 for the narrower ones (measured, see the launchers).
    const int GN = p.gn;
    const int grp = t / (GN * p.tiles_m);
    const int rem = t - grp * (GN * p.tiles_m);
    const int gw = min(GN, p.tiles_n - grp * GN);
    const int tile_n = grp * GN + rem % gw;
    const int tile_m = rem / gw;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    int expert = 0;
    if constexpr (MOE) {
        if (m0 >= moe.ntpp[0]) return;
        expert = moe.expert_ids[m0 / moe.block_m];
        pb += (int64_t)expert * moe.stride_be;
    }
    // the routed row of tile row r (MOE), and the activation row it reads: padding rows read row 0
    auto routed = [&](int r) -> int { return moe.sorted_ids[min(m0 + r, moe.EM - 1)]; };
    auto act_row = [&](int tok) -> int { return tok < moe.num_valid ? tok / moe.top_k : 0; };

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WGM;
    const int wn = wave / WGM;

    // The tile's scales are requested before anything else, as raw words into registers, and nobody waits
    // for them: they are older than every copy, so they have arrived long before the main loop ends.
    // They are widened and staged in LDS just before the epilogue, which then needs no global loads.
    // (Staged at kernel start, their latency came on top of that of the first copies.)
    constexpr int NSC = (BM + BN + NT - 1) / NT;
    uint32_t sc_raw[NSC];
    if constexpr (MODE != OUT_I32) {
#pragma unroll
        for (int q = 0; q < NSC; ++q) {
            const int e = threadIdx.x + q * NT;
            const bool is_row = e < BM;
            int64_t idx = is_row ? min(m0 + e, p.M - 1) : min(n0 + min(e - BM, BN - 1), p.N - 1);
            if constexpr (MOE) idx = is_row ? act_row(routed(e)) : idx + (int64_t)expert * moe.stride_scale_be;
            const void* base = is_row ? p.arow : p.acol;
            sc_raw[q] = (is_row ? p.arow_dtype : p.acol_dtype) == FNN_F32 ? ((const uint32_t*)base)[idx]
                                                                        : (uint32_t)((const uint16_t*)base)[idx];
        }
    }

    // copy plan: load j of this wave fills rows (j*NWAVES + wave)*8 .. +7; lane L writes slot (L & 7)
    // of row (L >> 3) of that group, which holds logical chunk (L & 7) ^ ((row >> 1) & 7)
    const int lrow = lane >> 3;
    const int lchunk = (lane & 7) ^ ((((wave & 1) << 2) + (lrow >> 1)) & 7);
    uint32_t goa[NLA], gob[NLB];
#pragma unroll
    for (int j = 0; j < NLA; ++j) {
        const int r = (j * NWAVES + wave) * 8 + lrow;
        goa[j] = (uint32_t)(MOE ? act_row(routed(r)) : min(m0 + r, p.M - 1)) * (uint32_t)p.lda + lchunk * 16;
    }
#pragma unroll
    for (int j = 0; j < NLB; ++j)
        gob[j] = (uint32_t)min(n0 + (j * NWAVES + wave) * 8 + lrow, p.N - 1) * (uint32_t)p.ldb + lchunk * 16;
    // The copies of a slab are issued in parts (halves or thirds), one per phase of the loop, so that the
    // copy unit is fed evenly instead of receiving a burst that blocks the wave's issue (and its MFMAs)
    // behind it.  `fix` moves a lane's 16 bytes back to the start of its row piece: the lanes of the last,
    // partial slab whose chunk lies beyond K fetch bytes that exist (and are never used).
    // The address of a copy is a scalar base (matrix + slab) plus the lane's 32-bit row offset, which is the
    // form the copy instruction takes directly; the base is passed through readfirstlane so that it is not
    // folded into per-lane 64-bit pointers that need vector adds before every copy.
    auto slab_base = [&](const int8_t* m, int kt) -> const char* {
        const uint64_t v = (uint64_t)m + (uint64_t)((int64_t)kt * BK);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (const char*)(((uint64_t)hi << 32) | lo);
    };
    auto copy_a_part = [&](char* stage, int kt, int part, int fix = 0) {
        const char* slab = slab_base(pa, kt);
#pragma unroll
        for (int j = 0; j < NLA; ++j)
            if (j * 3 / NLA == part)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(slab + (uint32_t)(goa[j] + fix)),
                                                 (lds_ptr_t)(stage + (j * NWAVES + wave) * (8 * BK)), 16, 0, 0);
    };
    auto copy_a = [&](char* stage, int kt, int fix = 0) {
        copy_a_part(stage, kt, 0, fix);
        copy_a_part(stage, kt, 1, fix);
        copy_a_part(stage, kt, 2, fix);
    };
    auto copy_b = [&](char* stage, int kt) {
        const char* slab = slab_base(pb, kt); const int fix = 0;
#pragma unroll
        for (int j = 0; j < NLB; ++j)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(slab + (uint32_t)(gob[j] + fix)),
                                             (lds_ptr_t)(stage + (j * NWAVES + wave) * (8 * BK)), 16, 0, 0);
    };
    auto copy_a_half = [&](char* stage, int kt, int half, int fix = 0) {
        const char* slab = slab_base(pa, kt);
#pragma unroll
        for (int j = 0; j < NLA; ++j)
            if (j * 2 / NLA == half)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(slab + (uint32_t)(goa[j] + fix)),
                                                 (lds_ptr_t)(stage + (j * NWAVES + wave) * (8 * BK)), 16, 0, 0);
    };
    auto copy_b_half = [&](char* stage, int kt, int half, int fix = 0) {
        const char* slab = slab_base(pb, kt);
#pragma unroll
        for (int j = 0; j < NLB; ++j)
            if (j * 2 / NLB == half)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(slab + (uint32_t)(gob[j] + fix)),
                                                 (lds_ptr_t)(stage + (j * NWAVES + wave) * (8 * BK)), 16, 0, 0);
    };
    auto copy_b_part = [&](char* stage, int kt, int part, int fix = 0) {
        const char* slab = slab_base(pb, kt);
#pragma unroll
        for (int j = 0; j < NLB; ++j)
            if (j * 3 / NLB == part)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(slab + (uint32_t)(gob[j] + fix)),
                                                 (lds_ptr_t)(stage + (j * NWAVES + wave) * (8 * BK)), 16, 0, 0);
    };

    // read plan: a fragment is 16 rows x 64 bytes of K; lane reads row (lane & 15), logical chunk
    // 4*kq + (lane >> 4) of chunk kq (0 or 1) of the slab
    const int frow = lane & 15;
    const int csel = lane >> 4;
    int rd_off[2];
#pragma unroll
    for (int kq = 0; kq < 2; ++kq) rd_off[kq] = frow * BK + (((4 * kq + csel) ^ ((frow >> 1) & 7)) * 16);
    const int a_base = wm * WTM * BK;
    const int b_base = wn * WTN * BK;

    v4i acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    // Fragments of both 64-byte chunks of a slab live in registers, indexed by chunk.  The NRD reads of
    // a chunk are issued in two parts, in the order the MFMAs need them: first half of the weight
    // fragments, the activation fragments, second half of the weight fragments.
    v4i wf[2][FN], af[2][FM];
    constexpr int NRD = FN + FM, NRA = (NRD + 1) / 2;
    auto read_part = [&](const char* sa, const char* sb, int kq, int part) {
#pragma unroll
        for (int r = 0; r < NRD; ++r) {
            if ((r >= NRA) != (part == 1)) continue;
            if (r < HN) wf[kq][r] = *(const v4i*)(sb + b_base + r * 16 * BK + rd_off[kq]);
            else if (r < HN + FM) af[kq][r - HN] = *(const v4i*)(sa + a_base + (r - HN) * 16 * BK + rd_off[kq]);
            else wf[kq][r - FM] = *(const v4i*)(sb + b_base + (r - FM) * 16 * BK + rd_off[kq]);
        }
    };
    // one phase of MFMAs: half h of the weight fragments of chunk kq against all activation fragments
    auto mfmas = [&](int kq, int h) {
#pragma unroll
        for (int i = h * HN; i < (h + 1) * HN; ++i)
#pragma unroll
            for (int j = 0; j < FM; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[kq][i], af[kq][j], acc[i][j], 0, 0, 0);
    };
    // ask the scheduler for: 2 MFMAs, 1 LDS read, 2 MFMAs, 1 LDS read, ... then the remaining MFMAs, so
    // that the reads of a phase are spread over its first half and have its second half to return
    // ncopies > 0 also places that many of the phase's copies behind those groups instead of leaving them
    // to the scheduler, which issues them, with their address arithmetic, ahead of the first MFMA after the
    // barrier.  Worth 1 to 2 % on the 256x192 tile; the tiles with three stages of both operands ran up to
    // 1.5 % slower with it and pass 0.
    auto interleave = [&](int part, auto ncopies) {
        constexpr int NC = decltype(ncopies)::value;
        constexpr int NM = HN * FM;
        constexpr int R0 = NRA, R1 = NRD - NRA;
        constexpr int PER = NM >= 2 * R0 ? 2 : 1;
        if (part == 0) {
#pragma unroll
            for (int q = 0; q < R0; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if constexpr (NC > 0) {
                    constexpr int VPG = (NC + R0 - 1) / R0;   // copies behind each of the first groups
                    if (q < (NC + VPG - 1) / VPG) __builtin_amdgcn_sched_group_barrier(0x010, VPG, 0);
                }
            }
            if constexpr (NM - PER * R0 > 0) __builtin_amdgcn_sched_group_barrier(0x008, NM - PER * R0, 0);
        } else {
#pragma unroll
            for (int q = 0; q < R1; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if constexpr (NC > 0) {
                    constexpr int VPG = (NC + R1 - 1) / R1;   // copies behind each of the first groups
                    if (q < (NC + VPG - 1) / VPG) __builtin_amdgcn_sched_group_barrier(0x010, VPG, 0);
                }
            }
            if constexpr (NM - PER * R1 > 0) __builtin_amdgcn_sched_group_barrier(0x008, NM - PER * R1, 0);
        }
    };
    // Wait until at most `newer` of this wave's copies are outstanding and its LDS reads have
    // returned, then cross the workgroup barrier.  A bare s_barrier: __syncthreads() would add a
    // fence that waits for every outstanding copy and collapse the ring to depth one.
    auto wait_barrier_n = [&](int newer_is_kept, auto nkeep) {
        constexpr int NK = decltype(nkeep)::value;
        asm volatile("" ::: "memory");
        if (newer_is_kept) __builtin_amdgcn_s_waitcnt(0x0070 | (NK & 15) | ((NK >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // K = 128 * (KT - 1) + 32 * last_steps: the last slab may hold fewer than 128 bytes per row
    const int KT = (Kl + BK - 1) / BK;
    const int last_steps = (Kl - (KT - 1) * BK) / 32;
    const int tail_fix = lchunk * 16 >= last_steps * 32 ? -(lchunk * 16) : 0;
    // The last slab, in stages (ca, cb), after its barrier; chunk 1 of the slab before it is in registers.
    // Where K ends in the middle of a 64-byte chunk, the lanes that hold its second half feed zeros
    // as weights (the bytes they read exist, but belong to no product).
    auto mask_half = [&](int kq) {
        if (csel >= 2) {
#pragma unroll
            for (int i = 0; i < FN; ++i) wf[kq][i] = v4i{0, 0, 0, 0};
        }
    };
    auto last_iter = [&](const char* ca, const char* cb) {
        read_part(ca, cb, 0, 0);
        mfmas(1, 0);
        read_part(ca, cb, 0, 1);
        mfmas(1, 1);
        __builtin_amdgcn_sched_barrier(0);
        if (last_steps == 1) mask_half(0);
        if (last_steps >= 3) {
            read_part(ca, cb, 1, 0);
            read_part(ca, cb, 1, 1);
        }
        mfmas(0, 0);
        mfmas(0, 1);
        __builtin_amdgcn_sched_barrier(0);
        if (last_steps >= 3) {
            if (last_steps == 3) mask_half(1);
            mfmas(1, 0);
            mfmas(1, 1);
        }
    };
    // A slab is two 64-byte chunks of K; a chunk's MFMAs run in two phases (one half of the weight
    // fragments each), so an iteration has four phases of HN*FM MFMAs.  Iteration i starts with the one
    // barrier: it publishes slab i and frees the stages of slab i-1, every read of which was issued
    // in the previous iteration.  Phases A and B multiply chunk 1 of slab i-1 (in registers) while chunk 0
    // of slab i is read; phases C and D multiply that chunk 0 while chunk 1 is read.  The reads are so
    // spread evenly: (FN+FM)/2 per phase.  The freed stages take the slab two ahead, copied in parts
    // over the phases (issued in one burst the copies block the wave's MFMAs behind them).
#define FNN_PHASE(ca, cb, kq, part, copies, mq, mh, NC)  \
    read_part(ca, cb, kq, part);                      \
    copies;                                           \
    mfmas(mq, mh);                                    \
    interleave(part, std::integral_constant<int, NC>{});  \
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (BDEEP) {
        // a-rows in two stages: slab i+1 goes into the a-stage of slab i-1 during phases A and B (it must be
        // complete at the next barrier); b-rows in three: slab i+2 follows during phases C and D, and only
        // its copies may be in flight at the next barrier (vmcnt counts in order, so all a-copies come first).
        // (Against all a-copies in phase A and the b-copies over B, C and D: 8192^3 411 -> 402 us, QKV 86.2 ->
        // 85.8 us.  The same split on the tiles with three stages of both operands changed nothing on balance.)
        auto wait_barrierB = [&](bool keep) { wait_barrier_n(keep, std::integral_constant<int, NLB>{}); };
        auto iterB = [&](const char* ca, const char* cb, char* fa, char* fb, int i, bool steady) {
            const bool more = steady || i + 2 < KT;
            const int fix_a = !steady && i + 1 == KT - 1 ? tail_fix : 0;
            const int fix_b = !steady && i + 2 == KT - 1 ? tail_fix : 0;
            wait_barrierB(true);
            FNN_PHASE(ca, cb, 0, 0, copy_a_half(fa, i + 1, 0, fix_a), 1, 0, NLA / 2)
            FNN_PHASE(ca, cb, 0, 1, copy_a_half(fa, i + 1, 1, fix_a), 1, 1, NLA / 2)
            FNN_PHASE(ca, cb, 1, 0, if (more) copy_b_half(fb, i + 2, 0, fix_b), 0, 0, NLB / 2)
            FNN_PHASE(ca, cb, 1, 1, if (more) copy_b_half(fb, i + 2, 1, fix_b), 0, 1, NLB / 2)
        };
        copy_b(sb0, 0);
        copy_a(sa0, 0);
        copy_b(sb1, 1);
        wait_barrierB(true);
        read_part(sa0, sb0, 0, 0);
        read_part(sa0, sb0, 0, 1);
        copy_a(sa1, 1);
        FNN_PHASE(sa0, sb0, 1, 0, copy_b_half(sb2, 2, 0), 0, 0, NLB / 2)
        FNN_PHASE(sa0, sb0, 1, 1, copy_b_half(sb2, 2, 1), 0, 1, NLB / 2)
        int i = 1;
        // (the steady loop stops one slab earlier when the last slab is partial: its copies need the fix)
        for (; i + 8 + (last_steps < 4) <= KT; i += 6) {
            iterB(sa1, sb1, sa0, sb0, i, true);
            iterB(sa0, sb2, sa1, sb1, i + 1, true);
            iterB(sa1, sb0, sa0, sb2, i + 2, true);
            iterB(sa0, sb1, sa1, sb0, i + 3, true);
            iterB(sa1, sb2, sa0, sb1, i + 4, true);
            iterB(sa0, sb0, sa1, sb2, i + 5, true);
        }
        for (; i < KT - 1; i += 6) {
            iterB(sa1, sb1, sa0, sb0, i, false);
            if (i + 1 < KT - 1) iterB(sa0, sb2, sa1, sb1, i + 1, false);
            if (i + 2 < KT - 1) iterB(sa1, sb0, sa0, sb2, i + 2, false);
            if (i + 3 < KT - 1) iterB(sa0, sb1, sa1, sb0, i + 3, false);
            if (i + 4 < KT - 1) iterB(sa1, sb2, sa0, sb1, i + 4, false);
            if (i + 5 < KT - 1) iterB(sa0, sb0, sa1, sb2, i + 5, false);
        }
        wait_barrierB(false);
        const int lb = (KT - 1) % 3;
        last_iter((KT - 1) & 1 ? sa1 : sa0, lb == 0 ? sb0 : lb == 1 ? sb1 : sb2);
    } else {
        // three stages each: slab i+2 of both operands goes into the stages of slab i-1 in three parts
        // during phases A..C; at the next barrier only those parts may be in flight
        auto wait_barrier3 = [&](bool keep) { wait_barrier_n(keep, std::integral_constant<int, NLA + NLB>{}); };
        auto iter3 = [&](const char* ca, const char* cb, char* fa, char* fb, int i, bool steady) {
            const bool more = steady || i + 2 < KT;
            const int fix = !steady && i + 2 == KT - 1 ? tail_fix : 0;
            wait_barrier3(true);
            FNN_PHASE(ca, cb, 0, 0, if (more) { copy_a_part(fa, i + 2, 0, fix); copy_b_part(fb, i + 2, 0, fix); }, 1, 0, 0)
            FNN_PHASE(ca, cb, 0, 1, if (more) { copy_a_part(fa, i + 2, 1, fix); copy_b_part(fb, i + 2, 1, fix); }, 1, 1, 0)
            FNN_PHASE(ca, cb, 1, 0, if (more) { copy_a_part(fa, i + 2, 2, fix); copy_b_part(fb, i + 2, 2, fix); }, 0, 0, 0)
            FNN_PHASE(ca, cb, 1, 1, , 0, 1, 0)
        };
        copy_a(sa0, 0);
        copy_b(sb0, 0);
        copy_a(sa1, 1);
        copy_b(sb1, 1);
        wait_barrier3(true);
        read_part(sa0, sb0, 0, 0);
        read_part(sa0, sb0, 0, 1);
        copy_a_part(sa2, 2, 0);
        copy_b_part(sb2, 2, 0);
        copy_a_part(sa2, 2, 1);
        copy_b_part(sb2, 2, 1);
        FNN_PHASE(sa0, sb0, 1, 0, { copy_a_part(sa2, 2, 2); copy_b_part(sb2, 2, 2); }, 0, 0, 0)
        FNN_PHASE(sa0, sb0, 1, 1, , 0, 1, 0)
        int i = 1;
        for (; i + 5 + (last_steps < 4) <= KT; i += 3) {
            iter3(sa1, sb1, sa0, sb0, i, true);
            iter3(sa2, sb2, sa1, sb1, i + 1, true);
            iter3(sa0, sb0, sa2, sb2, i + 2, true);
        }
        for (; i < KT - 1; i += 3) {
            iter3(sa1, sb1, sa0, sb0, i, false);
            if (i + 1 < KT - 1) iter3(sa2, sb2, sa1, sb1, i + 1, false);
            if (i + 2 < KT - 1) iter3(sa0, sb0, sa2, sb2, i + 2, false);
        }
        wait_barrier3(false);
        const int ls = (KT - 1) % 3;
        last_iter(ls == 0 ? sa0 : ls == 1 ? sa1 : sa2, ls == 0 ? sb0 : ls == 1 ? sb1 : sb2);
    }
#undef FNN_PHASE

    if constexpr (SPLIT) {
        // This unit's accumulators into its slot, in register order: value (i, j) of lane L at 16-byte word
        // (i * FM + j) * NT + L of the slot.  The slots are written and read with device-scope accesses
        // (they pass through L2 to where every XCD sees them), 8 bytes at a time.  A device-scope fence
        // would do for plain stores, but it writes back (release) and invalidates (acquire) the XCD's whole
        // L2, under the other workgroups' operand traffic: the split kernel then ran at half the speed of
        // the unsplit one.
        typedef unsigned long long u64;
        u64* const slots = (u64*)p.ws_part + (int64_t)t * p.kparts * (BM * BN / 2);
        // The tile's counter holds arrivals in its low half and completed slots in its high half.
        int* const word = (int*)sb2 + BM + BN;      // behind the scales' place in the third b-stage
        __syncthreads();                    // every wave has left the main loop: the stages are free
        if (threadIdx.x == 0)
            *word = __hip_atomic_fetch_add(p.ws_count + t, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const int seen = *word;
        // the last unit to arrive that finds every other slot complete adds them up without storing its own
        if (!((seen & 0xffff) == p.kparts - 1 && (seen >> 16) == p.kparts - 1)) {
            // 16 bytes per lane, so that a wave's store covers whole 128-byte lines: written as two 8-byte
            // halves every line went to memory twice, half filled each time (M=256 N=4096 K=8192 in three
            // parts: 27.1 us, with whole lines 24.2 us).  Device scope (sc1) through the buffer form of
            // the store, which takes the cache policy as an argument.
            const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
                (char*)slots + (int64_t)kpart * (BM * BN * 4), 0, BM * BN * 4, 0x00027000);
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[i][j]), mine, threadIdx.x * 16,
                                                           (i * FM + j) * (NT * 16), 16 /* sc1 */);
            // Every wave waits here until all of its slot stores have been acknowledged (vmcnt counts a
            // store until the memory side has taken it); only behind the barrier that follows does one
            // lane count the slot complete.  The order "slot written, then counted" rests on this wait: a
            // workgroup-scope fence promises nothing about when stores reach device scope.
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0x0070);
            asm volatile("" ::: "memory");
            __syncthreads();
            if (threadIdx.x == 0)
                *word = __hip_atomic_fetch_add(p.ws_count + t, 0x10000, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            // whoever completes the last of all kparts slots adds up the others; otherwise this unit is done
            if ((*word >> 16) != p.kparts - 1) return;
        }
        // The count that chose this unit was returned to lane 0 before the barrier above, and the loads
        // below are issued behind that barrier: they reach memory after every slot they read was counted
        // complete.  They are device-scope loads, served where the stores went.
        asm volatile("" ::: "memory");
        for (int q = 0; q < p.kparts; ++q) {
            if (q == kpart) continue;
            const u64* const theirs = slots + (int64_t)q * (BM * BN / 2) + 2 * threadIdx.x;
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j) {
                    const u64* const w = theirs + (i * FM + j) * (2 * NT);
                    const u64 lo = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const u64 hi = __hip_atomic_load(w + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    acc[i][j] += v4i{(int)(uint32_t)lo, (int)(uint32_t)(lo >> 32), (int)(uint32_t)hi, (int)(uint32_t)(hi >> 32)};
                }
        }
        if (threadIdx.x == 0) __hip_atomic_store(p.ws_count + t, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue ----
    // acc[i][j][r]: n = wn0 + i*16 + 4*(lane>>4) + r,  m = wm0 + j*16 + (lane&15).
    // A lane owns 4 consecutive n of ONE row, so storing straight from registers would touch 16
    // rows per instruction with 8 bytes each.  Instead every wave transposes its sub-tile through
    // LDS (one ring stage per wave, free now) 64 rows at a time and writes whole rows:
    // 16 bytes per lane, consecutive lanes on consecutive addresses.
    const int wm0 = m0 + wm * WTM;
    const int wn0 = n0 + wn * WTN;
    if constexpr (MODE == OUT_I32) {
        const bool vec_ok = (p.ldc & 3) == 0;
#pragma unroll
        for (int j = 0; j < FM; ++j) {
            const int m = wm0 + j * 16 + frow;
#pragma unroll
            for (int i = 0; i < FN; ++i) {
                const int n = wn0 + i * 16 + 4 * csel;
                if (m >= p.M || n >= p.N) continue;
                int32_t* o = (int32_t*)p.out + (int64_t)m * p.ldc + n;
                if (n + 3 < p.N && vec_ok) {
                    *(v4i*)o = acc[i][j];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < p.N) o[e] = acc[i][j][e];
                }
            }
        }
    } else {
        // A lane holds 4 consecutive n of one row m per fragment: 8 bytes.  v_permlane16_swap exchanges the
        // odd 16-lane rows of one register with the even rows of another; applied to the packed halves
        // of two neighbouring weight fragments it leaves every lane with 8 consecutive n (16 bytes) of one
        // of the two, so that a store instruction writes 64 contiguous bytes of each of its 16 rows and
        // the three instructions of a fragment row the wave's whole 192-byte (WTN * 2) piece of them.  No
        // LDS transposition, no barrier between the waves.
        static_assert(FN % 2 == 0, "weight fragments are stored in pairs");
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070);   // all copies and LDS reads of this wave are done
        __builtin_amdgcn_s_barrier();         // ... and everybody else's: the stages are free
        asm volatile("" ::: "memory");
#pragma unroll
        for (int q = 0; q < NSC; ++q) {
            const int e = threadIdx.x + q * NT;
            const bool is_row = e < BM;
            const int dt = is_row ? p.arow_dtype : p.acol_dtype;
            const float v = dt == FNN_F32 ? __builtin_bit_cast(float, sc_raw[q])
                                          : dt == FNN_F16 ? f16_bits_to_f32(sc_raw[q]) : bf16_bits_to_f32(sc_raw[q]);
            if (is_row) sc_row[e] = v;
            else if (e < BM + BN) sc_col[e - BM] = v;
        }
        // MOE: the routed row of every tile row (and its routing weight) behind the scales
        int* const sc_tok = (int*)(sc_col + BN) + 4;
        float* const sc_wr = (float*)(sc_tok + BM);
        if constexpr (MOE) {
            for (int e = threadIdx.x; e < BM; e += NT) {
                const int tok = routed(e);
                sc_tok[e] = tok;
                sc_wr[e] = moe.mul_w && tok < moe.num_valid ? load_as_f32(moe.topk_w, tok, moe.topk_w_dtype) : 1.f;
            }
        }
        __syncthreads();
        const int nsel = (csel & 1) * 16 + (csel >> 1) * 8;   // column of this lane's 16 bytes within a fragment pair
        v4f ac[FN];
#pragma unroll
        for (int i = 0; i < FN; ++i) ac[i] = *(const v4f*)&sc_col[wn * WTN + i * 16 + 4 * csel];
        // a tile that lies wholly inside the matrix stores without bounds checks (a uniform choice)
        const bool inside = m0 + BM <= p.M && n0 + BN <= p.N && (p.ldc & 7) == 0;
        // the 16 bytes a lane holds of fragments i and i + 1 (8 consecutive columns of row frow) after the scales,
        // the conversion and the exchange between the two fragments
        auto pair_val = [&](int i, int j, float ar, float wr) __attribute__((always_inline)) -> v4u {
            uint32_t lo[2], hi[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = ((float)acc[i + h][j][e] * ar) * ac[i + h][e];
                    if constexpr (MOE) {
                        if (moe.mul_w) v[e] = v[e] * wr;
                    }
                }
                if constexpr (MODE == OUT_BF16) {
                    lo[h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[0], v[1]}, v2bf));
                    hi[h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[2], v[3]}, v2bf));
                } else {
                    lo[h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[0], v[1]}, v2h));
                    hi[h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[2], v[3]}, v2h));
                }
            }
            const v2u sl = __builtin_amdgcn_permlane16_swap(lo[0], lo[1], false, false);
            const v2u sh = __builtin_amdgcn_permlane16_swap(hi[0], hi[1], false, false);
            return v4u{sl[0], sh[0], sl[1], sh[1]};
        };
        // Inside the matrix: whole 128-byte lines per store instruction.  A fragment pair gives every row 64
        // contiguous bytes; two pairs side by side (fragments i .. i + 3) give 128, held by lanes of the same
        // row in two registers.  A rotation by 8 within each row of 16 lanes moves the second pair's bytes of
        // rows 0..7 to the lanes of rows 8..15 and the first pair's bytes of rows 8..15 the other way, so that
        // one instruction writes rows 0..7 and the next rows 8..15, 128 bytes of each.  (Half lines, written at
        // different times, reached memory as partial writes: 1.45 times the output's bytes by the counters.)
        // RG: rows are checked (the tile's last rows may lie beyond M; MOE: a row goes to its routed row, padding
        // rows are not stored); the columns all lie inside the matrix.
        auto store_full = [&](auto row_guard) {
            constexpr bool RG = decltype(row_guard)::value;
            const int r8 = frow & 7, hsel = frow >> 3;
            // the output row of tile row r, or -1
            auto out_row = [&](int r) __attribute__((always_inline)) -> int64_t {
                if constexpr (MOE) {
                    const int t = sc_tok[r];
                    return t < moe.num_valid ? t : -1;
                } else {
                    return !RG || m0 + r < p.M ? m0 + r : -1;
                }
            };
            uint16_t* const cbase = (uint16_t*)p.out + wn0 + nsel;
            auto quad = [&](int i, int j, float ar, float wr) __attribute__((always_inline)) {
                const v4u x = pair_val(i, j, ar, wr), y = pair_val(i + 2, j, ar, wr);
                v4u v1, v2;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v1[k] = (uint32_t)__builtin_amdgcn_update_dpp((int)x[k], (int)y[k], 0x128, 0xF, 0xC, false);
                    v2[k] = (uint32_t)__builtin_amdgcn_update_dpp((int)y[k], (int)x[k], 0x128, 0xF, 0x3, false);
                }
                const int64_t ra = out_row(wm * WTM + j * 16 + r8), rb = out_row(wm * WTM + j * 16 + 8 + r8);
                if (!RG || ra >= 0) __builtin_nontemporal_store(v1, (v4u*)(cbase + ra * p.ldc + hsel * 32 + i * 16));
                if (!RG || rb >= 0) __builtin_nontemporal_store(v2, (v4u*)(cbase + rb * p.ldc + hsel * 32 + i * 16));
            };
            auto pair = [&](int i, int j, float ar, float wr) __attribute__((always_inline)) {
                const v4u v = pair_val(i, j, ar, wr);
                const int64_t r = out_row(wm * WTM + j * 16 + frow);
                if (!RG || r >= 0) __builtin_nontemporal_store(v, (v4u*)(cbase + r * p.ldc + i * 16));
            };
#pragma unroll
            for (int j = 0; j < FM; ++j) {
                const float ar = sc_row[wm * WTM + j * 16 + frow];
                float wr = 1.f;
                if constexpr (MOE) wr = sc_wr[wm * WTM + j * 16 + frow];
                if constexpr (FN % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < FN; i += 4) quad(i, j, ar, wr);
                } else {
                    // six fragments (192 bytes a row): the wave's lines are its first two pairs (wn = 0) or its
                    // last two (wn = 1); the pair in the middle of the tile's row shares its line with the other
                    // wave (handing the halves over through LDS so that one wave writes it whole gained nothing)
                    static_assert(FN % 4 == 0 || FN == 6, "wave tiles of 64, 96 or 128 columns");
                    if (wn == 0) { quad(0, j, ar, wr); pair(4, j, ar, wr); }
                    else { pair(0, j, ar, wr); quad(2, j, ar, wr); }
                }
            }
        };
        auto store_rows = [&]() {
#pragma unroll
            for (int j = 0; j < FM; ++j) {
                const float ar = sc_row[wm * WTM + j * 16 + frow];
                int m = wm0 + j * 16 + frow;
                float wr = 1.f;
                bool row_ok = true;
                if constexpr (MOE) {        // the output row is the routed row; padding rows store nothing
                    m = sc_tok[wm * WTM + j * 16 + frow];
                    wr = sc_wr[wm * WTM + j * 16 + frow];
                    row_ok = m < moe.num_valid;
                }
#pragma unroll
                for (int i = 0; i < FN; i += 2) {
                    const v4u val = pair_val(i, j, ar, wr);
                    const int n = wn0 + i * 16 + nsel;
                    if ((MOE ? row_ok : m < p.M) && n < p.N) {
                        uint16_t* o = (uint16_t*)p.out + (int64_t)m * p.ldc + n;
                        if (n + 7 < p.N && (p.ldc & 7) == 0) {
                            __builtin_nontemporal_store(val, (v4u*)o);
                        } else {
#pragma unroll
                            for (int q = 0; q < 8; ++q)
                                if (n + q < p.N) o[q] = (uint16_t)(val[q >> 1] >> (16 * (q & 1)));
                        }
                    }
                }
            }
        };
        const bool cols_inside = n0 + BN <= p.N && (p.ldc & 7) == 0;
        if (inside && !MOE) store_full(std::false_type{});
        else if (cols_inside) store_full(std::true_type{});
        else store_rows();
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
                const float v = rounded_f32(((float)acc[i][j] * ar) * load_as_f32(p.acol, n, p.acol_dtype));
                store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
            }
        }
    }
}

// ------------------------------------------------------------------------ dispatch
struct TileChoice { int bm, bn; };

// With 256x192 tiles, the number of 192-wide tile columns to give a first launch when the rest is better done
// by a second launch of 256x128 tiles, or 0.  A round of 256 workgroups takes one tile time however few of
// them exist, so a last round that is mostly empty is expensive; the columns are then cut where the first
// launch ends on a full round.  Costs in 256x192 tile times: a 256x128 tile takes 128/192/0.85 of one, the
// second launch about 0.08 (its launch gap and start-up).
static int split_columns_192(int64_t M, int64_t N, double* cost_out = nullptr) {
    const int64_t tm = (M + 255) / 256, c = (N + 191) / 192;
    const double single = (double)((tm * c + 255) / 256);
    double best = single - 0.1;      // worth a second launch only from a tenth of a round
    int best_c1 = 0;
    if (cost_out) *cost_out = single;
    for (int64_t c1 = c - 1; c1 >= 1 && c1 >= c - 64; --c1) {
        const int64_t rem = N - 192 * c1;
        const int64_t r1 = (tm * c1 + 255) / 256, r2 = (tm * ((rem + 127) / 128) + 255) / 256;
        const double cost = (double)r1 + (double)r2 * (128.0 / 192.0 / 0.85) + 0.08;
        if (cost < best) { best = cost; best_c1 = (int)c1; }
    }
    if (cost_out && best_c1 > 0) *cost_out = best;
    return best_c1;
}

// Pick the tile whose last, partly filled round of workgroups costs least on 256 CUs.
static TileChoice choose_tile(int64_t M, int64_t N) {
    static const struct { int bm, bn; double eff; } cand[] = {
        {256, 192, 1.00}, {256, 256, 1.17}, {256, 128, 0.85}, {128, 128, 0.72}, {64, 128, 0.62}};
    // eff = throughput per tile area relative to the 256x192 tile, measured with every round full.  The
    // 256x256 tile (all 256 accumulator registers of a lane beside 256 others, all 160 KB of LDS: two a-stages,
    // three b-stages) takes 1.13 of a 256x192 tile's time for 1.33 of its outputs - the kernel is bound by the
    // operand bytes a CU takes in per slab, (rows + columns) * 128, and the square tile needs fewest per
    // output - so it wins where its rounds are full (M = K = N = 8192: 390 -> 366 us, gate_up 154 -> 149 us)
    // and loses where they are not (QKV: 384 tiles, 82 -> 94 us).  It
    // depends on the shape: the 256x128 tile reaches 1.0 at M=2048, K=4096, N=12288, 0.93 at N=22016 and
    // 0.74 at M=K=N=8192; 128x128 0.71 to 0.76; 64x128 0.64 to 0.67 (a 64x128 tile takes 0.55 to 0.6 of
    // the time of a 128x128 one, so it pays where it doubles the workgroups without adding a round).
    // The 128x128 figure is that of one workgroup per CU; the pairs are priced below.
    // Up to 128 rows over 32769 .. 38912 channels: 257 .. 304 tiles of 128 columns, of which the pricing below
    // makes pairs - fewer than a fifth of the CUs then run two workgroups and set the time while the others
    // stream their weights at the rate of one.  One round of 256x192 tiles (the rows beyond M copy the last
    // row again: L1 hits) is faster: M=128 N=35584 K=13312 116 against 144 us, M=65 110 / 128; N=36864 K=8192
    // 78 / 90 and 75 / 81; N=37888 K=3584 38 / 43 and 39 / 37; N=33792 K=4096 44 / 49 and 44 / 45.  From 320
    // tiles on the pairs are level again or ahead (N=40960 K=4096 M=128 49 / 51, N=49152 53 / 52).
    if (M <= 128 && N > 32768 && N <= 38912) return TileChoice{256, 192};
    double best = 1e300;
    TileChoice c{128, 128};
    for (const auto& t : cand) {
        const int64_t tiles = ((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn);
        const int64_t rounds = (tiles + 255) / 256;
        const double cost = (double)rounds * t.bm * t.bn / t.eff;
        if (cost < best) { best = cost; c = {t.bm, t.bn}; }
    }
    // The 128x128 tile in pairs (two workgroups per CU from 257 tiles on: a round holds 512 of them at 0.85,
    // a last round of at most 256 leaves every workgroup a CU of its own and takes 0.64 of a shared one)
    // replaces a smaller or narrower tile where it is cheaper.  It never replaces the 256x192 tile: the two
    // shapes where this pricing did so were slower on the box (116 -> 122 us, 118 -> 121 us).
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128);
    if (t128 > 256 && !(c.bm == 256 && c.bn >= 192)) {
        const int64_t rem = t128 % 512;
        const double pair = ((double)(t128 / 512) + (rem == 0 ? 0.0 : rem <= 256 ? 0.64 : 1.0)) * 2.0 * 128 * 128 / 0.85;
        if (pair < best) c = {128, 128};
    }
    return c;
}

// The same problem restricted to columns [n0, n0 + n) of the output (rows [n0, n0 + n) of B) ...
static A8W8Args columns_from(const A8W8Args& p, int64_t n0, int n, int mode) {
    A8W8Args q = p;
    q.N = n;
    q.b = p.b + n0 * p.ldb;
    q.out = (char*)p.out + n0 * (mode == OUT_I32 ? 4 : 2);
    if (p.acol) q.acol = (const char*)p.acol + n0 * (p.acol_dtype == FNN_F32 ? 4 : 2);
    return q;
}
// ... and to rows [m0, m0 + m) of A and of the output.
static A8W8Args rows_from(const A8W8Args& p, int64_t m0, int m, int mode) {
    A8W8Args q = p;
    q.M = m;
    q.a = p.a + m0 * p.lda;
    q.out = (char*)p.out + m0 * p.ldc * (mode == OUT_I32 ? 4 : 2);
    if (p.arow) q.arow = (const char*)p.arow + m0 * (p.arow_dtype == FNN_F32 ? 4 : 2);
    return q;
}

// Tile columns per group of the tile numbering (the kernel's GN).  Both libraries on one box, bf16 out, us,
// groups of 4 / 8 / 16 columns: QKV (256x192 tiles) 83.7 / 81.6 / 85.1, gate_up (256x256) 157.2 / 153.2 / 157.5,
// 8192^3 (256x256) 370.4 / 368.9 / 384.8; with 256x128 tiles: down (K = 11008) 78.6 / 80.9 / 84.6, O 32.3 / 32.0 /
// 31.9, M = 1024 N = 8192 33.1 / 32.9 / 33.9; 128x128: M = 512 K = N = 8192 40.8 / 40.9 / 42.0.
// Over a long K the wider groups lose again (M = 8192 N = 17792 K = 13312: 1349 / 1442; M = 2048 N = 35584 K = 13312:
// 732 / 741; K = 7392 .. 8896: within 1 %), so they are taken up to K = 8192.
static int group_columns(int bn, int k) { return bn >= 192 && k <= 8192 ? 8 : 4; }

template <int BM, int BN, int MODE, bool PAIR = false, int WGM = 2>
static void launch_mfma(A8W8Args& p, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int tiles = p.tiles_m * p.tiles_n;
    p.tiles_per_xcd = (tiles + 7) / 8;
    p.gn = group_columns(BN, p.K);
    note_kernel("gemm_a8w8_ring_kernel", BM, BN, WGM * 2);
    gemm_a8w8_ring_kernel<BM, BN, MODE, PAIR, WGM><<<dim3(p.tiles_per_xcd * 8), dim3(WGM * 128), 0, st>>>(p, MoeArgs{});
}

// The same tiles with K cut into p.kparts ranges (p.kparts, p.k_chunk, p.ws_count, p.ws_part set by the caller).
template <int BM, int BN, int MODE, bool PAIR = false>
static void launch_mfma_split(A8W8Args& p, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int units = p.tiles_m * p.tiles_n * p.kparts;
    p.tiles_per_xcd = (units + 7) / 8;
    p.gn = group_columns(BN, p.K);
    note_kernel("gemm_a8w8_ring_kernel(split K)", BM, BN, p.kparts);
    gemm_a8w8_ring_kernel<BM, BN, MODE, PAIR, 2, true><<<dim3(p.tiles_per_xcd * 8), dim3(256), 0, st>>>(p, MoeArgs{});
}

// The tiles that exist: (rows, columns, waves per workgroup).
static bool valid_tile(int bm, int bn, int waves) {
    if (bm == 0 && bn == 0) return waves == 0;
    if (waves == 0 || waves == 4)
        return (bm == 256 && (bn == 256 || bn == 192 || bn == 128)) || (bm == 128 && bn == 128) || (bm == 64 && bn == 128);
    return false;
}

template <int MODE>
static void launch_tile(A8W8Args& p, hipStream_t st, int bm, int bn, int waves) {
    if (bm == 256 && bn == 192) launch_mfma<256, 192, MODE>(p, st);
    else if (bm == 256 && bn == 256) launch_mfma<256, 256, MODE>(p, st);
    else if (bm == 256 && bn == 128) launch_mfma<256, 128, MODE>(p, st);
    else if (bm == 64 && bn == 128) launch_mfma<64, 128, MODE>(p, st);
    else if ((int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) > 256) launch_mfma<128, 128, MODE, true>(p, st);
    else launch_mfma<128, 128, MODE>(p, st);
}

// ---- K split over several workgroups per tile (needs a workspace) ----
// Workspace: kWsCounters ticket counters (zero between calls), then per tile kparts slots of tile-rows x
// tile-columns accumulators.
constexpr int kWsCounters = 1024;
constexpr size_t kWsHeader = kWsCounters * sizeof(int);

struct SplitPlan { int bm, bn, kparts, k_chunk; double us; };

// Slabs per part: the last part gets kStagger slabs more than the others (and the remainder), so that the
// others have stored their accumulators by the time it arrives and it can add them up at once.
constexpr int kStagger = 4;
static int split_chunk_slabs(int KT, int parts) { return (KT - kStagger) / parts; }

static size_t split_ws_bytes(const SplitPlan& s, int64_t M, int64_t N) {
    const int64_t tiles = ((M + s.bm - 1) / s.bm) * ((N + s.bn - 1) / s.bn);
    return kWsHeader + (size_t)tiles * s.kparts * s.bm * s.bn * sizeof(int32_t);
}

// Whether to split K for this shape, and how.  The tile is 128x128 in pairs of workgroups per CU: with few
// activation rows the weights stream from HBM, and two workgroups per CU keep twice the bytes in flight; a
// workgroup's chain of slabs is bound by the latency of the weights, and the split shortens it (the 256-row
// tiles were slower split than the small tiles unsplit).  Measured, bf16 out, microseconds, unsplit -> split
// (parts; units = 128x128 tiles x parts):
//   M = 256  N = 4096 K = 8192   27.1 -> 24.2 (3; 192)      M = 128  N = 2048 K = 16384  54.9 -> 30.2 (8; 128)
//   M = 512  N = 2048 K = 8192   29.3 -> 22.9 (4; 256)      M = 256  N = 4096 K = 6144   24.6 -> 20.9 (4; 256)
//   M = 1024 N = 1920 K = 13312  48.3 -> 39.5 (2; 240)      M = 512  N = 4096 K = 11008  41.4 -> 35.5 (2; 256)
//   M = 384  N = 3584 K = 18944  68.6 -> 44.1 (3; 252)      M = 1024 N = 2048 K = 8192   29.7 -> 27.2 (2; 256)
// About one unit per CU is the best count (84 tiles: 3 parts 44.1, 2 parts 52.8, 4 parts 49.0), a part
// needs 8 slabs and K at least 6144 (K = 4096: 17.0 -> 17.8 and worse).  Up to two units per CU - every CU
// holding a pair - pay only over a long K, from about 40 slabs per part:
//   M = 764  N = 3584 K = 18944  85.8 -> 63.0 (3; 504)      M = 1024 N = 3584 K = 18944  86.3 -> 71.1 (2; 448)
//   M = 1024 N = 4096 K = 11008  53.3 -> 51.7 (2; 512)      M = 512  N = 8192 K = 8192   40.7 -> 45.1 (2; 512: not taken)
static SplitPlan plan_split(int64_t M, int64_t N, int64_t K, size_t ws_bytes) {
    const int KT = (int)((K + 127) / 128);
    const TileChoice u = choose_tile(M, N);
    const SplitPlan none{u.bm, u.bn, 1, 0, 0.0};
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128);
    if (KT < 48 || t128 > 256) return none;
    int parts = 1;
    for (int q = 2; q <= 8; ++q) {
        const int64_t units = t128 * q;
        const int slabs = split_chunk_slabs(KT, q);
        // More than one round of units (two per CU on some or all CUs) pays with two to four tile rows: their
        // tiles stream the weights with little reuse, and a second workgroup on the CU keeps that stream going.
        // With five and more rows the unsplit tiles share their weights through the L2 and are level or ahead,
        // and with a single row most CUs would run one unit and the rest two, no shorter than before (under a
        // captured graph, rotating weights, two parts / unsplit: M=256 N=8960 K=13312 52 / 64 us, M=384 N=8192
        // K=14784 67 / 88, M=512 N=8192 K=28672 125 / 134; but M=640 N=3584 K=18944 66 / 61, M=764 N=4096
        // K=11008 42.6 / 37.7, M=896 N=3584 K=18944 70 / 59, M=1024 N=4096 K=11008 48 / 43, M=1280 N=1920
        // K=13312 48.5 / 42.3, M=128 N=17792 K=13312 81 / 72).
        const int64_t mrows = (M + 127) / 128;
        const bool pairs_pay = mrows >= 2 && mrows <= 4;
        if ((units <= 256 && slabs >= 8) || (units <= 512 && slabs >= 40 && pairs_pay)) parts = q;
    }
    // (a workspace too small for the best count takes the largest one it holds)
    for (; parts >= 2; --parts) {
        const SplitPlan s{128, 128, parts, split_chunk_slabs(KT, parts) * 128, 0.0};
        if (ws_bytes == 0 || split_ws_bytes(s, M, N) <= ws_bytes) return s;
    }
    return none;
}

template <int MODE>
static void launch_split(A8W8Args& p, hipStream_t st, const SplitPlan& s, void* workspace) {
    p.kparts = s.kparts;
    p.k_chunk = s.k_chunk;
    p.ws_count = (int*)workspace;
    p.ws_part = (int32_t*)((char*)workspace + kWsHeader);
    if (s.bm == 128) launch_mfma_split<128, 128, MODE, true>(p, st);   // two workgroups per CU
    else if (s.bn == 192) launch_mfma_split<256, 192, MODE>(p, st);
    else launch_mfma_split<256, 128, MODE>(p, st);
}

// One launch plan for operands whose row offsets fit 32 bits (M * lda and N * ldb below 2^31 bytes).
struct Workspace { void* ptr; size_t bytes; int force_kparts; };

template <int MODE>
static void dispatch_band(A8W8Args& p, hipStream_t st, bool aligned, int force_bm, int force_bn, int force_waves,
                          const Workspace& ws = Workspace{nullptr, 0, 0}) {
    // the MFMA kernel walks K in slabs of 128 bytes
    const bool fast = aligned && p.K % 32 == 0 && p.K >= 512;
    // few activation rows: stream the weights once (unless the caller names a tile of the tiled kernel)
    // ... and up to 256 rows over a narrow weight matrix with long rows, where the tiled kernel has a handful
    // of tiles and splits K to fill the machine: 64-row passes of the few-row kernel stream the weights through
    // all CUs instead (bf16 out, tiled / passes: M=128 N=2048 K=8192 19.8 / 11.6 us, M=256 23.3 / 17.5; M=128
    // N=1920 K=13312 25.3 / 17.4; M=128 N=1024 K=4096 10.1 / 8.7; from N = 3584 on the tiled kernel wins:
    // M=128 N=3584 K=18944 30.5 / 34.5, N=K=8192 23.3 / 24.7).  The same bits either way.
    const bool narrow = p.M <= kA8PanelRowsNarrow && p.N <= 2048 && p.K >= 4096;
    // 17 .. 64 rows over more than 16384 and fewer than 32768 channels: the few-row kernel's workgroups own 64
    // channels, so there are between 257 and 511 of them - one round of the 256 CUs and a part of a second -
    // where the tiled kernel has one round of 64x128 tiles (under a captured graph, rotating weights, bf16 out,
    // M=64, few-row / tiled: N=16384 K=4096 17.8 / 20.7 us, N=16640 26.6 / 21.1, N=20480 27.7 / 22.6, N=24576
    // 28.8 / 24.6, N=28672 30.0 / 29.8 on one box and 30.4 / 25.4 on another; N=24576 K=8192 55.3 / 45.1;
    // N=17792 K=13312 86.0 / 60.0; M=33 alike; M=24: N=24576 K=4096 30.4 / 25.3, N=17792 K=13312 60.9 / 55.9,
    // elsewhere within a few percent, the tiled kernel never behind)
    const bool between_rounds = fast && p.M > 16 && p.M <= 64 && p.N > 16384 && p.N < 32768;
    if (force_bm == 0 && !between_rounds && (p.M <= 64 || narrow) && launch_a8w8_skinny(p, MODE, st)) return;
    if (fast && ws.ptr) {
        if (ws.force_kparts > 1) {          // (the entry point has checked tile, parts and workspace size)
            const int chunk = split_chunk_slabs((p.K + 127) / 128, ws.force_kparts) * 128;
            launch_split<MODE>(p, st, SplitPlan{force_bm, force_bn, ws.force_kparts, chunk, 0.0}, ws.ptr);
            return;
        }
        if (force_bm == 0 && ws.force_kparts == 0) {
            const SplitPlan s = plan_split(p.M, p.N, p.K, ws.bytes);
            if (s.kparts > 1) {
                launch_split<MODE>(p, st, s, ws.ptr);
                return;
            }
        }
    }
    if (!fast) {
        note_kernel("gemm_a8w8_any_kernel");
        gemm_a8w8_any_kernel<MODE><<<dim3((p.N + 63) / 64, (p.M + 63) / 64), dim3(256), 0, st>>>(p);
        return;
    }
    if (force_bm > 0) {
        launch_tile<MODE>(p, st, force_bm, force_bn, force_waves);
        return;
    }
    TileChoice c = choose_tile(p.M, p.N);
    if (c.bm == 256 && c.bn >= 192) {
        // the 256x256 tile in full rounds against 256x192 tiles with their column split, in 256x192 tile times
        double cost192 = 0.0;
        const int c1 = split_columns_192(p.M, p.N, &cost192);
        const int64_t t256 = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256);
        const double cost256 = (double)((t256 + 255) / 256) * (256.0 / 192.0 / 1.17);
        // (by a margin: a partly filled last round is cheaper than the model's whole tile time, for either tile;
        // the cases within 7 % measured between 0.955 and 1.04)
        c.bn = cost256 < 0.93 * cost192 ? 256 : 192;
    }
    if (c.bm == 256 && c.bn == 192) {
        const int c1 = split_columns_192(p.M, p.N);
        if (c1 > 0) {
            // columns [0, 192 c1) in 192-wide tiles, the rest in 128-wide ones
            A8W8Args q = p;
            q.N = 192 * c1;
            launch_tile<MODE>(q, st, 256, 192, 0);
            launch_tile<MODE>(q = columns_from(p, q.N, p.N - q.N, MODE), st, 256, 128, 0);
            return;
        }
    }
    launch_tile<MODE>(p, st, c.bm, c.bn, 0);
}

// The kernels address a row of A or B as base + 32-bit byte offset.  Operands beyond that (M * lda or
// N * ldb of 2^31 bytes and more: a long prefill, a very wide head) are cut on the host into bands of rows
// and of columns that fit, each band a problem of its own on the same kernels.
template <int MODE>
static void dispatch(A8W8Args& p, hipStream_t st, int force_bm, int force_bn, int force_waves,
                     const Workspace& ws = Workspace{nullptr, 0, 0}) {
    const bool aligned = p.lda % 16 == 0 && p.ldb % 16 == 0 && ((uintptr_t)p.a % 16) == 0 &&
                         ((uintptr_t)p.b % 16) == 0 && ((uintptr_t)p.out % 16) == 0;
    constexpr int64_t kLimit = (1LL << 31) - 1;
    const int64_t m_fit = kLimit / p.lda, n_fit = kLimit / p.ldb;
    if (p.M <= m_fit && p.N <= n_fit) {
        dispatch_band<MODE>(p, st, aligned, force_bm, force_bn, force_waves, ws);
        return;
    }
    // bands in whole tiles of every shape (rows: 256; columns: 768 = lcm(256, 192, 128)), so that the bands
    // tile like the undivided problem and every band keeps the operands' alignment
    const int64_t m_band = m_fit >= 256 ? m_fit / 256 * 256 : m_fit, n_band = n_fit >= 768 ? n_fit / 768 * 768 : n_fit;
    for (int64_t m0 = 0; m0 < p.M; m0 += m_band)
        for (int64_t n0 = 0; n0 < p.N; n0 += n_band) {
            A8W8Args q = columns_from(p, n0, (int)(p.N - n0 < n_band ? p.N - n0 : n_band), MODE);
            q = rows_from(q, m0, (int)(p.M - m0 < m_band ? p.M - m0 : m_band), MODE);
            dispatch_band<MODE>(q, st, aligned && ((uintptr_t)q.out % 16) == 0, force_bm, force_bn, force_waves);
        }
}

// Mixture of experts with many routed rows per expert: the MFMA tiles over the sorted rows.  A tile must lie
// within one expert's rows, so its height divides block_m.  Returns false where this form does not apply (the
// few-row kernels then take the call).
template <int BM, int BN, int MODE, bool PAIR = false>
static void launch_mfma_moe(A8W8Args& p, const MoeArgs& q, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.tiles_per_xcd = (p.tiles_m * p.tiles_n + 7) / 8;
    p.gn = 4;
    note_kernel("gemm_a8w8_ring_kernel(moe)", BM, BN, 4);
    gemm_a8w8_ring_kernel<BM, BN, MODE, PAIR, 2, false, true><<<dim3(p.tiles_per_xcd * 8), dim3(256), 0, st>>>(p, q);
}

template <int MODE>
static bool launch_moe_tiled_t(A8W8Args& p, const MoeArgs& q, hipStream_t st) {
    if (q.block_m % 256 == 0) launch_mfma_moe<256, 256, MODE>(p, q, st);
    else if (q.block_m % 128 == 0) launch_mfma_moe<128, 128, MODE, true>(p, q, st);
    else launch_mfma_moe<64, 128, MODE>(p, q, st);
    return true;
}

static bool launch_a8w8_moe_tiled(A8W8Args& p, const MoeArgs& q, int mode, hipStream_t st) {
    constexpr int64_t kLimit = (1LL << 31) - 1;
    const int64_t rows = (q.num_valid + q.top_k - 1) / q.top_k;          // activation rows
    const bool ok = q.block_m % 64 == 0 && q.EM % q.block_m == 0 && p.K % 32 == 0 && p.K >= 1024 &&
                    p.lda % 16 == 0 && p.ldb % 16 == 0 && q.stride_be % 16 == 0 && ((uintptr_t)p.a % 16) == 0 &&
                    ((uintptr_t)p.b % 16) == 0 && ((uintptr_t)p.out % 16) == 0 && rows * p.lda <= kLimit &&
                    (int64_t)p.N * p.ldb <= kLimit && (int64_t)(p.M / 64) * ((p.N + 127) / 128) <= kLimit;
    // The few-row kernel reads an expert's weights once per 64 sorted rows.  Measured on 8 experts of
    // 28672 x 4096, 2 per token, microseconds over S sorted rows in use: few-row kernel 100 + 0.18 S; tiles of
    // 64 rows 110 + 0.14 S, of 128 rows 105 + 0.10 S, of 256 rows 57 + 0.092 S.  Blocks of 128 rows or more
    // always take the tiles; blocks of 64 from about 512 routed rows on.
    if (!ok || (q.block_m % 128 != 0 && q.num_valid < 512)) return false;
    return mode == OUT_F16 ? launch_moe_tiled_t<OUT_F16>(p, q, st) : launch_moe_tiled_t<OUT_BF16>(p, q, st);
}

static int check_args(const char* fn, const void* out, const void* a, const void* b, int64_t M,
                      int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
    // an empty tensor has no address: pointers are only required when there is something to compute
    if (M != 0 && N != 0 && (!out || !a || !b)) { set_error("%s: null pointer argument", fn); return FNN_ERR_ARG; }
    if (M < 0 || N < 0 || K <= 0 || lda < K || ldb < K || ldc < N) {
        set_error("%s: bad shape M=%lld N=%lld K=%lld lda=%lld ldb=%lld ldc=%lld", fn, (long long)M,
                  (long long)N, (long long)K, (long long)lda, (long long)ldb, (long long)ldc);
        return FNN_ERR_ARG;
    }
    if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30) || lda > (1LL << 30) || ldb > (1LL << 30)) {
        set_error("%s: shape or row stride too large", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    return FNN_OK;
}

}  // namespace fnn

using namespace fnn;

static int gemm_a8w8_entry(const char* fn, void* out, const void* a, const void* b, const void* alpha_row,
                           const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                           int64_t ldc, int out_dtype, int alpha_row_dtype, int alpha_col_dtype, int tile_m,
                           int tile_n, int waves, void* stream, const Workspace& ws = Workspace{nullptr, 0, 0}) {
    int rc = check_args(fn, out, a, b, M, N, K, lda, ldb, ldc);
    if (rc != FNN_OK) return rc;
    if (M != 0 && N != 0 && (!alpha_row || !alpha_col)) { set_error("%s: null scale pointer", fn); return FNN_ERR_ARG; }
    if (!is16(out_dtype)) { set_error("%s: Output type must be float16 or bfloat16", fn); return FNN_ERR_UNSUPPORTED; }
    if (!isflt(alpha_row_dtype) || !isflt(alpha_col_dtype)) { set_error("%s: bad scale type", fn); return FNN_ERR_UNSUPPORTED; }
    if (!valid_tile(tile_m, tile_n, waves)) {
        set_error("%s: no such tile %dx%d with %d waves", fn, tile_m, tile_n, waves);
        return FNN_ERR_ARG;
    }
    if (ws.force_kparts < 0 || (ws.bytes > 0 && !ws.ptr)) {
        set_error("%s: bad workspace or number of parts (%d)", fn, ws.force_kparts);
        return FNN_ERR_ARG;
    }
    if (ws.ptr && (((uintptr_t)ws.ptr % 16) != 0 || ws.bytes < kWsHeader)) {
        set_error("%s: the workspace must be 16-byte aligned and hold at least %zu bytes", fn, kWsHeader);
        return FNN_ERR_ARG;
    }
    if (ws.force_kparts > 1) {
        // a named split: one of the two large tiles, parts of at least 4 slabs, a workspace that holds it
        const int KT = (int)((K + 127) / 128), chunk = split_chunk_slabs(KT, ws.force_kparts);
        const SplitPlan s{tile_m, tile_n, ws.force_kparts, chunk * 128, 0.0};
        const bool tile_ok = ((tile_m == 256 && (tile_n == 128 || tile_n == 192)) || (tile_m == 128 && tile_n == 128)) &&
                             (waves == 0 || waves == 4);
        const bool shape_ok = K % 32 == 0 && lda % 16 == 0 && ldb % 16 == 0 && ((uintptr_t)a % 16) == 0 &&
                              ((uintptr_t)b % 16) == 0 && ((uintptr_t)out % 16) == 0 && M * lda < (1LL << 31) &&
                              N * ldb < (1LL << 31);
        if (!tile_ok || !shape_ok || chunk < 4 ||
            ((M + tile_m - 1) / (tile_m ? tile_m : 1)) * ((N + tile_n - 1) / (tile_n ? tile_n : 1)) > kWsCounters) {
            set_error("%s: K = %lld cannot be split %d ways on a %dx%d tile for these operands", fn, (long long)K,
                      ws.force_kparts, tile_m, tile_n);
            return FNN_ERR_ARG;
        }
        if (!ws.ptr || split_ws_bytes(s, M, N) > ws.bytes) {
            set_error("%s: workspace of %zu bytes, the split needs %zu", fn, ws.bytes, split_ws_bytes(s, M, N));
            return FNN_ERR_ARG;
        }
    }
    if (M == 0 || N == 0) return FNN_OK;
    A8W8Args p{};
    p.a = (const int8_t*)a; p.b = (const int8_t*)b; p.out = out; p.arow = alpha_row; p.acol = alpha_col;
    p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.out_dtype = out_dtype; p.arow_dtype = alpha_row_dtype; p.acol_dtype = alpha_col_dtype;
    const Call call(fn);
    if (out_dtype == FNN_F16) dispatch<OUT_F16>(p, (hipStream_t)stream, tile_m, tile_n, waves, ws);
    else dispatch<OUT_BF16>(p, (hipStream_t)stream, tile_m, tile_n, waves, ws);
    return call.done();
}

static int gemm_a8w8_i32_entry(const char* fn, int32_t* acc, const void* a, const void* b, int64_t M, int64_t N,
                               int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int tile_m, int tile_n,
                               int waves, void* stream) {
    int rc = check_args(fn, acc, a, b, M, N, K, lda, ldb, ldc);
    if (rc != FNN_OK) return rc;
    if (!valid_tile(tile_m, tile_n, waves)) {
        set_error("%s: no such tile %dx%d with %d waves", fn, tile_m, tile_n, waves);
        return FNN_ERR_ARG;
    }
    if (M == 0 || N == 0) return FNN_OK;
    A8W8Args p{};
    p.a = (const int8_t*)a; p.b = (const int8_t*)b; p.out = acc;
    p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    const Call call(fn);
    dispatch<OUT_I32>(p, (hipStream_t)stream, tile_m, tile_n, waves);
    return call.done();
}

extern "C" int fnn_gemm_a8w8(void* out, const void* a, const void* b, const void* alpha_row,
                             const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                             int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                             int alpha_col_dtype, void* stream) {
    return gemm_a8w8_entry("fnn_gemm_a8w8", out, a, b, alpha_row, alpha_col, M, N, K, lda, ldb, ldc, out_dtype,
                           alpha_row_dtype, alpha_col_dtype, 0, 0, 0, stream);
}

extern "C" int fnn_gemm_a8w8_tiled(void* out, const void* a, const void* b, const void* alpha_row,
                                   const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                                   int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                                   int alpha_col_dtype, int tile_m, int tile_n, int waves, void* stream) {
    return gemm_a8w8_entry("fnn_gemm_a8w8_tiled", out, a, b, alpha_row, alpha_col, M, N, K, lda, ldb, ldc, out_dtype,
                           alpha_row_dtype, alpha_col_dtype, tile_m, tile_n, waves, stream);
}

extern "C" size_t fnn_gemm_a8w8_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 64 || N <= 0 || K < 512 || K % 32 != 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return 0;
    // (a narrow weight matrix under up to 256 rows goes to the few-row kernel in passes: see dispatch_band)
    if (M <= kA8PanelRowsNarrow && N <= 2048 && K >= 4096 && N % 16 == 0) return 0;
    const SplitPlan s = plan_split(M, N, K, 0);
    return s.kparts > 1 ? split_ws_bytes(s, M, N) : 0;
}

namespace fnn {
__global__ __launch_bounds__(256) void clear_words_kernel(int* w, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) w[i] = 0;
}
}  // namespace fnn

static int static_scratch(const char* fn, void** out);

extern "C" int fnn_workspace_init(void* workspace, size_t ws_bytes, void* stream) {
    const char* fn = "fnn_workspace_init";
    if (!workspace && ws_bytes == 0) {
        // the library's own workspace on the current device (fnn_gemm_a8w8_static)
        const int rc = static_scratch(fn, &workspace);
        if (rc != FNN_OK) return rc;
    } else if (!workspace || ((uintptr_t)workspace % 16) != 0 || ws_bytes < kWsHeader) {
        set_error("%s: the workspace must be 16-byte aligned and hold at least %zu bytes", fn, kWsHeader);
        return FNN_ERR_ARG;
    }
    const Call call(fn);
    note_kernel("clear_words_kernel");
    clear_words_kernel<<<dim3(kWsCounters / 256), dim3(256), 0, (hipStream_t)stream>>>((int*)workspace, kWsCounters);
    return call.done();
}

extern "C" int fnn_gemm_a8w8_ws(void* out, const void* a, const void* b, const void* alpha_row,
                                const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                                int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                                int alpha_col_dtype, void* workspace, size_t ws_bytes, void* stream) {
    return gemm_a8w8_entry("fnn_gemm_a8w8_ws", out, a, b, alpha_row, alpha_col, M, N, K, lda, ldb, ldc, out_dtype,
                           alpha_row_dtype, alpha_col_dtype, 0, 0, 0, stream, Workspace{workspace, ws_bytes, 0});
}

extern "C" int fnn_gemm_a8w8_ws_tiled(void* out, const void* a, const void* b, const void* alpha_row,
                                      const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                                      int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                                      int alpha_col_dtype, int tile_m, int tile_n, int kparts, void* workspace,
                                      size_t ws_bytes, void* stream) {
    return gemm_a8w8_entry("fnn_gemm_a8w8_ws_tiled", out, a, b, alpha_row, alpha_col, M, N, K, lda, ldb, ldc,
                           out_dtype, alpha_row_dtype, alpha_col_dtype, tile_m, tile_n, 0, stream,
                           Workspace{workspace, ws_bytes, kparts == 1 ? 0 : kparts});
}

// ---- the workspace held by the library itself, for callers that cannot allocate ----
// One array per GPU, part of the code object: every GPU the library runs on holds it from the moment the
// library's code is loaded there until the process ends.  In host code the array's name is only a handle
// for hipGetSymbolAddress - the device address differs per GPU and is looked up once per device.
constexpr size_t kStaticScratchBytes = 16u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static std::atomic<void*> g_scratch_of[64];     // device address of `scratch` on each device, once known

static int static_scratch(const char* fn, void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) {
        set_error("%s: no current device (%s)", fn, hipGetErrorString(e));
        return FNN_ERR_HIP;
    }
    void* ptr = g_scratch_of[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));     // the current device's copy of the array
        if (e != hipSuccess || !ptr) {
            set_error("%s: hipGetSymbolAddress failed on device %d: %s", fn, dev, hipGetErrorString(e));
            return FNN_ERR_HIP;
        }
        g_scratch_of[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return FNN_OK;
}

extern "C" int fnn_gemm_a8w8_static(void* out, const void* a, const void* b, const void* alpha_row,
                                    const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                                    int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                                    int alpha_col_dtype, int tile_m, int tile_n, int kparts, void* stream) {
    const char* fn = "fnn_gemm_a8w8_static";
    if (kparts > 1 && M > 0 && N > 0 && K > 0 && tile_m > 0 && tile_n > 0) {
        // a named split is the only way to ask for more than the array holds (the library's own plans fit)
        const SplitPlan s{tile_m, tile_n, kparts, 0, 0.0};
        const size_t need = split_ws_bytes(s, M, N);
        if (need > kStaticScratchBytes) {
            set_error("%s: this split needs %zu bytes of workspace, the library's own holds %zu; use "
                      "fnn_gemm_a8w8_ws_tiled with a workspace of that size, or fewer parts", fn, need,
                      kStaticScratchBytes);
            return FNN_ERR_UNSUPPORTED;
        }
    }
    void* ws = nullptr;
    const int rc = static_scratch(fn, &ws);
    if (rc != FNN_OK) return rc;
    // The counters at the start of the array are zero when the code is loaded and every call's kernel
    // returns the counters it used to zero before it ends (the unit that adds up a tile clears the tile's
    // counter), so this call finds them zero; the slots behind them need no clearing.
    return gemm_a8w8_entry(fn, out, a, b, alpha_row, alpha_col, M, N, K, lda, ldb, ldc, out_dtype, alpha_row_dtype,
                           alpha_col_dtype, tile_m, tile_n, 0, stream,
                           Workspace{ws, kStaticScratchBytes, kparts == 1 ? 0 : kparts});
}

extern "C" int fnn_gemm_a8w8_i32(int32_t* acc, const void* a, const void* b, int64_t M, int64_t N,
                                 int64_t K, int64_t lda, int64_t ldb, int64_t ldc, void* stream) {
    return gemm_a8w8_i32_entry("fnn_gemm_a8w8_i32", acc, a, b, M, N, K, lda, ldb, ldc, 0, 0, 0, stream);
}

extern "C" int fnn_gemm_a8w8_i32_tiled(int32_t* acc, const void* a, const void* b, int64_t M, int64_t N,
                                       int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int tile_m, int tile_n,
                                       int waves, void* stream) {
    return gemm_a8w8_i32_entry("fnn_gemm_a8w8_i32_tiled", acc, a, b, M, N, K, lda, ldb, ldc, tile_m, tile_n, waves,
                               stream);
}

extern "C" int fnn_fused_moe_a8w8(void* c, const void* a, const void* b, const void* alpha_row,
                                  const void* alpha_col, const void* topk_weights,
                                  const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                  const int32_t* num_tokens_post_padded, int64_t N, int64_t K, int64_t EM,
                                  int64_t num_valid_tokens, int64_t lda, int64_t stride_be, int64_t ldb,
                                  int64_t ldc, int64_t stride_scale_be, int mul_routed_weight, int top_k,
                                  int block_m, int out_dtype, int alpha_row_dtype, int alpha_col_dtype,
                                  int topk_weights_dtype, void* stream) {
    using namespace fnn;
    const char* fn = "fnn_fused_moe_a8w8";
    if (!c || !a || !b || !alpha_row || !alpha_col || !sorted_token_ids || !expert_ids || !num_tokens_post_padded ||
        (mul_routed_weight && !topk_weights)) {
        set_error("%s: null pointer argument", fn);
        return FNN_ERR_ARG;
    }
    if (N < 0 || K <= 0 || EM < 0 || num_valid_tokens < 0 || top_k <= 0 || block_m <= 0 || lda < K || ldb < K ||
        ldc < N || stride_be < 0 || stride_scale_be < 0) {
        set_error("%s: bad shape N=%lld K=%lld EM=%lld tokens=%lld top_k=%d block_m=%d", fn, (long long)N,
                  (long long)K, (long long)EM, (long long)num_valid_tokens, top_k, block_m);
        return FNN_ERR_ARG;
    }
    if (N > 0x7FFFFFFFLL || K > 0x7FFFFFFFLL || EM > 0x7FFFFFFFLL || num_valid_tokens > 0x7FFFFFFFLL) {
        set_error("%s: shape too large", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (!is16(out_dtype)) { set_error("%s: Output type must be float16 or bfloat16", fn); return FNN_ERR_UNSUPPORTED; }
    if (!isflt(alpha_row_dtype) || !isflt(alpha_col_dtype) || (mul_routed_weight && !isflt(topk_weights_dtype))) {
        set_error("%s: bad scale type", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (N == 0 || EM == 0 || num_valid_tokens == 0) return FNN_OK;
    A8W8Args p{};
    p.a = (const int8_t*)a; p.b = (const int8_t*)b; p.out = c; p.arow = alpha_row; p.acol = alpha_col;
    p.M = (int)EM; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.out_dtype = out_dtype; p.arow_dtype = alpha_row_dtype; p.acol_dtype = alpha_col_dtype;
    MoeArgs q{};
    q.sorted_ids = sorted_token_ids; q.expert_ids = expert_ids; q.ntpp = num_tokens_post_padded;
    q.topk_w = topk_weights; q.topk_w_dtype = topk_weights_dtype; q.mul_w = mul_routed_weight ? 1 : 0;
    q.top_k = top_k; q.block_m = block_m; q.num_valid = (int)num_valid_tokens; q.EM = (int)EM;
    q.stride_be = stride_be; q.stride_scale_be = stride_scale_be;
    const Call call(fn);
    const int mode = out_dtype == FNN_F16 ? OUT_F16 : OUT_BF16;
    if (!launch_a8w8_moe_tiled(p, q, mode, (hipStream_t)stream)) launch_a8w8_moe(p, q, mode, (hipStream_t)stream);
    return call.done();
}
