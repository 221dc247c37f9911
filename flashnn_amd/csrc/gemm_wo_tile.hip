// Weight-only GEMM for many activation rows (M > 64): a tiled MFMA kernel, gfx950.
//
// With hundreds of activation rows the job is no longer streaming the weights but multiplying: every
// weight has to be dequantised once per workgroup and used against as many rows as possible.  A
// 512-thread workgroup (8 waves, 2 along M x 4 along N, two on every SIMD) owns BM activation rows
// (256 or 128) x 128 output channels and walks K in slabs of 128 (one scale group):
//   * activations: the slab of the tile's rows (BM x 256 bytes) is copied L2 -> LDS with direct-to-LDS
//     16-byte loads into a ring of two stages, one slab ahead; 16-byte chunks XOR-swizzled with the row so
//     that the 16 lanes of a fragment read hit 16 different bank groups;
//   * weights: the slab of the tile's weight rows (64 packed int4 rows or 128 int8 rows x 128 bytes) goes
//     the same way into a ring of three stages, two slabs ahead; the slab's scales and zero points (group
//     size 128) one slab ahead into three stages of their own: nothing waits in registers for HBM, and one
//     s_waitcnt vmcnt(N) with a compile-time N plus a bare s_barrier publishes a slab (all copies of an
//     iteration are issued in a fixed order, the weights last: they have two slabs to land and may stay in
//     flight over the next barrier);
//   * a wave reads 16 bytes per lane of its weight rows from LDS (16 k of one row), turns them into MFMA
//     "A" operands with the exponent tricks of wo_common.h (values c + q, exact), reads the activation
//     fragments ("B" operands) and runs v_mfma_f32_16x16x32_{f16,bf16}: wave tile (BM/2) x 32, 16 or 8
//     accumulator fragments; an MFMA against ones per activation fragment gives the row sums that remove c
//     and the zero points;
//   * at the end of a slab (group size 128) the slab's accumulators are folded into the running output in
//     fp32: out += s * (acc - (c + zp) * sum_k a_k); with per-channel scales there is one fold at the end;
//   * bias, rounding, 16-byte (int4: 8 channels) or 8-byte stores.
// The weights are read from HBM once per 256 rows; tiles of the same channels and different rows follow
// each other on one XCD and share the weights through its L2.
//
// Reference semantics: flashnn/quant_gemm.py:148-206; the Triton kernels this replaces for large M:
// flashnn/triton_kernels/gemm_a16w4.py:209-333, gemm_a16w8.py:179-272.
#include <type_traits>

#include "wo_common.h"

namespace fnn {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// REFQ (1, or 2 with zero points; fp16 activations, fp16 scales and zero points, per channel or per group of
// 128 .. values): every weight is dequantised and rounded to fp16 as the reference's torch path does before the dot
// product, (q - zp) * s with both operations rounded (ref_dq_f16 in wo_common.h; flashnn/quant_gemm.py:14-36).
// The accumulators then run over all of K: no MFMAs against ones, no fold per slab, no second accumulator
// set, and the result differs from the reference's only by the order of the fp32 additions.  bf16
// activations reach this form through the conversion pass of gemm_weight_only.hip (rows scaled by a power
// of two, p.act_unscale undoes it).  bf16 activations with bf16 tables: the same with both roundings to bf16,
// worked in fp32 (ref_dq_bf16 in wo_common.h), the operands meeting in the bf16 MFMA.
// MOE (per-channel tables, no REFQ): the mixture-of-experts form for many routed rows per expert
// (flashnn/triton_kernels/fused_moe_a16w4.py:50-206).  The M dimension is the list of sorted routed rows,
// padded per expert to blocks of q.block_m rows, a multiple of BM: tile row r multiplies activation row
// sorted_ids[r] / top_k with the weights, scales and zero points of the expert its block belongs to, and the
// result goes to output row sorted_ids[r], times the routing weight on request.  Tiles beyond the rows in
// use return at once; padding rows read activation row 0 and store nothing.
template <int WBITS, int ADT, bool G128, int SDT, int BM, int REFQ = 0, bool MOE = false>
__global__ __launch_bounds__(512) void gemm_wo_tile_kernel(const WoArgs p, const int tiles_m, const int tiles,
                                                           const MoeArgs q) {
    // REFQ = 3: the same software pipeline over the slabs without the per-weight rounding, for per-channel
    // tables of any type: the operands are the converted integers, the activation sums come from MFMAs
    // against ones and scale and zero point are applied once at the end.
    constexpr bool ROUNDQ = REFQ == 1 || REFQ == 2;
    static_assert(!ROUNDQ || (ADT == SDT && (ADT == FNN_F16 || ADT == FNN_BF16)), "reference rounding: activations and tables of one 16-bit type");
    // bf16 activations with bf16 tables: the weights are rounded to bf16 as the reference's torch path rounds them
    // (in fp32 arithmetic, ref_dq_bf16 in wo_common.h) and meet the activations in the bf16 MFMA
    constexpr bool RQBF = ROUNDQ && ADT == FNN_BF16;
    constexpr float kWholeZpMax = RQBF ? 128.f : 512.f;    // whole zero points up to here take the one-step form
    static_assert(REFQ != 3 || !G128, "the pipeline without rounding: per-channel tables");
    // The gathered form takes per-channel tables (pipelined, REFQ = 3) or tables per group of 128 in the
    // layout of the reference's MoE launcher, [expert][channel][group] (fp32 scaling per slab, 128-row tiles):
    // the tile's slice of both tables is transposed into LDS once, in the format of a table stage per group.
    static_assert(!MOE || (WBITS == 4 && ((!G128 && REFQ == 3) || (G128 && REFQ == 0 && BM == 128))), "the gathered form");
    typedef MfmaT<ADT> MT;
    static_assert(WBITS == 4 || BM == 128, "three stages of 128 int8 weight rows leave room for 128 activation rows");
    constexpr int NH = WBITS == 4 ? 2 : 1;          // channels per weight row
    constexpr int BN = 128;                          // channels per workgroup
    constexpr int WROWS = BN / NH;                   // weight rows per workgroup
    constexpr int WGM = 2, WGN = 4;                  // waves along M and N
    constexpr int WTM = BM / WGM, WTN = BN / WGN;    // wave tile: 128 or 64 rows x 32 channels
    constexpr int FB = WTM / 16;                     // activation fragments per wave
    constexpr int NF = WTN / NH / 16;                // 16-row weight fragments per wave (int4: 1, int8: 2)
    constexpr int NA = NF * NH;                      // A operands per k-step (int4: even and odd channel of the fragment)
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    constexpr int ASTG = BM * 256;                   // bytes of an activation stage
    constexpr int WSTG = WROWS * 128;                // bytes of a weight stage
    constexpr int TSTG = 1024;                       // a table stage: scales of 128 channels, then zero points (16-bit)
    __shared__ __attribute__((aligned(1024))) char sa0[ASTG];
    __shared__ __attribute__((aligned(1024))) char sa1[ASTG];
    __shared__ __attribute__((aligned(1024))) char sw0[WSTG];
    __shared__ __attribute__((aligned(1024))) char sw1[WSTG];
    __shared__ __attribute__((aligned(1024))) char sw2[WSTG];
    __shared__ __attribute__((aligned(1024))) char st0[TSTG];
    __shared__ __attribute__((aligned(1024))) char st1[TSTG];
    __shared__ __attribute__((aligned(1024))) char st2[TSTG];
    constexpr int kMoeGroups = 64;                   // K / 128 at most, where the gathered form has group tables
    __shared__ __attribute__((aligned(1024))) char mtab[MOE && G128 ? kMoeGroups * TSTG / 2 : 16];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int row16 = lane & 15, g = lane >> 4;

    // workgroups id, id + 8, .. share an XCD and take consecutive tile numbers
    const int per_xcd = gridDim.x >> 3;
    const int t = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (t >= tiles) return;
    // tiles are numbered in groups of four channel tiles, the channel tile fastest within a group: the 32
    // workgroups an XCD runs at a time then cover 8 row tiles x 4 channel tiles, and the activation rows are
    // fetched into its L2 once per group instead of once per channel tile
    constexpr int GN = 4;
    const int tiles_n = tiles / tiles_m;
    const int grp = t / (GN * tiles_m), rem = t - grp * (GN * tiles_m);
    const int gcols = min(GN, tiles_n - grp * GN);
    const int tile_n = grp * GN + rem % gcols, tile_m = rem / gcols;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int KT = p.K / 128;
    int expert = 0;
    if constexpr (MOE) {
        if (m0 >= q.ntpp[0]) return;
        expert = q.expert_ids[m0 / q.block_m];
    }

    // ---- copies.  A wave instruction writes 1 KB of LDS, linear in the lane id; the swizzle is applied
    // on the global side.  Activations: instruction i of a wave covers rows (i * 8 + wave) * 4 .. + 3,
    // lane L row L >> 4, slot L & 15 holding chunk (L & 15) ^ (row & 15).
    // (row offsets are formed when the copy is issued: eight registers holding them are eight the
    // accumulators cannot have)
    constexpr int NCA = BM / 32;
    const int ar0 = wave * 4 + (lane >> 4);          // the lane's row in instruction 0; instruction i: + 32 i
    const int ar_max = p.M - 1 - m0;                 // rows beyond M read the last row (and are not stored)
    const uint32_t a_chunk = (((lane & 15) ^ (ar0 & 15)) << 4);
    const uint32_t lda2 = (uint32_t)(p.lda * 2);
    const char* const a_base = (const char*)p.act + (MOE ? 0 : (int64_t)m0 * p.lda * 2);
    // MOE: the activation row of every tile row, staged once in the first table stage (per-channel tables
    // leave the table stages unused); a copy reads its rows from there instead of keeping NCA offsets in registers
    int* const a_rows = (int*)st0;
    if constexpr (MOE) {
        static_assert(BM * 4 <= TSTG, "the tile's row numbers fit a table stage");
        for (int r = threadIdx.x; r < BM; r += 512) {
            const int tok = q.sorted_ids[m0 + r];
            a_rows[r] = tok < q.num_valid ? tok / q.top_k : 0;
        }
        if constexpr (G128) {
            // group g of the tile: 256 bytes of scales, then 256 of zero points, channel by channel
            const uint16_t* const sc = (const uint16_t*)p.scale + (int64_t)expert * q.stride_scale_be + (int64_t)n0 * KT;
            const uint16_t* const zp = p.zp ? (const uint16_t*)p.zp + (int64_t)expert * q.stride_zp_be + (int64_t)n0 * KT : nullptr;
            for (int e = threadIdx.x; e < BN * KT; e += 512) {
                const int ch = e / KT, g2 = e - ch * KT;
                *(uint16_t*)(mtab + g2 * 512 + ch * 2) = sc[e];
                *(uint16_t*)(mtab + g2 * 512 + 256 + ch * 2) = zp ? zp[e] : (uint16_t)0;
            }
        }
        __syncthreads();
    }
    auto copy_a = [&](char* stage, int j) {
        const char* src = a_base + (int64_t)min(j, KT - 1) * 256;        // scalar
#pragma unroll
        for (int i = 0; i < NCA; ++i) {
            const uint32_t off = (uint32_t)(MOE ? a_rows[ar0 + 32 * i] : min(ar0 + 32 * i, ar_max)) * lda2 + a_chunk;
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + off), (lds_ptr_t)(stage + (i * 8 + wave) * 1024), 16, 0, 0);
        }
        // (the compiler keeps these offsets in registers where it has them to spare)
    };
    // Weights: instruction i of a wave covers weight rows (i * 8 + wave) * 8 .. + 7, lane L row L >> 3, slot
    // L & 7 holding chunk (L & 7) ^ ((row >> 1) & 7).
    constexpr int NCW = WROWS / 64;
    uint32_t gw[NCW];
#pragma unroll
    for (int i = 0; i < NCW; ++i) {
        const int r = (i * 8 + wave) * 8 + (lane >> 3);
        gw[i] = (uint32_t)r * (uint32_t)p.ldw + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
    }
    const char* const w_base = (const char*)p.qw + (int64_t)(n0 / NH) * p.ldw + (MOE ? (int64_t)expert * q.stride_be : 0);
    auto copy_w = [&](char* stage, int j) {
        const char* src = w_base + (int64_t)min(j, KT - 1) * 128;
#pragma unroll
        for (int i = 0; i < NCW; ++i)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + gw[i]), (lds_ptr_t)(stage + (i * 8 + wave) * 1024), 16, 0, 0);
    };
    // Tables: 256 bytes of scales and 256 bytes of zero points per slab; every wave issues the same copy
    // (lanes 0..15 the scales, 16..31 the zero points, the rest a second time), so that all waves count
    // the same number of loads.
    constexpr int NCT = G128 ? 1 : 0;
    const bool has_zp = p.zp != nullptr;
    const char* const t_src = (lane & 16) && has_zp ? (const char*)p.zp : (const char*)p.scale;
    const uint32_t gt = (uint32_t)n0 * 2 + (lane & 15) * 16;
    auto copy_t = [&](char* stage, int j) {
        if constexpr (G128 && !MOE) {
            const int64_t off = (int64_t)(min(j, KT - 1) >> p.gshift) * p.N * 2;      // groups of 128 << gshift values
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(t_src + off + gt), (lds_ptr_t)stage, 16, 0, 0);
        }
    };
    auto wait_barrier = [&]() {   // everything but the newest weight copies has landed, for every wave
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070 | (NCW & 15));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- reads
    // weight fragment f of the wave: rows wn * (64 / NH) + f * 16 + row16; 16 bytes = k 64 h + 16 g .. + 15
    int w_rd[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) w_rd[h] = (wn * (WTN / NH) + row16) * 128 + (((4 * h + g) ^ ((row16 >> 1) & 7)) << 4);
    // activation fragment b: rows wm * WTM + b * 16 + row16; k-step (h, q): chunk 8 h + 2 g + q
    int a_rd[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int q = 0; q < 2; ++q) a_rd[h][q] = (wm * WTM + row16) * 256 + (((8 * h + 2 * g + q) ^ row16) << 4);

    // G128: outv is the running output and a slab's accumulators live only while one activation fragment is
    // worked on; per-channel scales: outv accumulates over all of K, asum the activation row sums
    v4f outv[NA][FB], asum[FB];
#pragma unroll
    for (int b = 0; b < FB; ++b) {
        asum[b] = v4f{0, 0, 0, 0};
#pragma unroll
        for (int a = 0; a < NA; ++a) outv[a][b] = v4f{0, 0, 0, 0};
    }
    const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
    const v4f zero4 = v4f{0, 0, 0, 0};
    const float zmul = has_zp ? 1.f : 0.f;
    typedef typename std::conditional<NH == 2, v4u, v2u>::type tab_t;

    // REFQ with per-channel tables: the scale and zero point of the channels this lane's operand rows hold
    const v2h rq_c = pair_of_f16_bits(WBITS == 4 ? 0x6408u : 0x6480u);   // 1032 / 1152: what the conversion adds
    const v2h rq_c_odd = pair_of_f16_bits(0x5480u);                      // 72: .. to the odd channel of an int4 row
    v2h rq_s[NA], rq_z[NA];
    float bq_s[NA], bq_z[NA];                                            // the same as fp32 numbers (bf16 tables)
    if constexpr (ROUNDQ && !G128) {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            const int n = n0 + wn * WTN + (a / NH) * 16 * NH + NH * row16 + (a % NH);
            const uint32_t sb = ((const uint16_t*)p.scale)[n], zb = p.zp ? ((const uint16_t*)p.zp)[n] : 0u;
            if constexpr (RQBF) {
                bq_s[a] = bf16_bits_to_f32(sb);
                bq_z[a] = bf16_bits_to_f32(zb);
            } else {
                rq_s[a] = pair_of_f16_bits(sb);
                rq_z[a] = pair_of_f16_bits(zb);
            }
        }
    }

    // One slab.  All of the slab's weights are converted first (A operand a of k-step ks; int4: operand
    // 2 f + (0 even, 1 odd channel) of fragment f, int8: operand = fragment).  Then one activation fragment
    // at a time: its four k-steps against all operands (five independent MFMA chains, the fifth against
    // ones for the row sums) and, with group scales, the fold of those accumulators into the running
    // output, out += s * (acc - (c + zp) * sum a) - vector-ALU work that has the MFMAs of the next
    // fragment to run under, and accumulators that are dead before the next fragment needs registers.
    auto slab = [&](const char* sa, const char* sw, const char* stg) {
        v4u A[4][NA];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const v4u w = *(const v4u*)(sw + w_rd[h] + f * 16 * 128);
                if constexpr (WBITS == 4)
                    convert_w4_nat<ADT>(w, A[2 * h][2 * f], A[2 * h + 1][2 * f], A[2 * h][2 * f + 1], A[2 * h + 1][2 * f + 1]);
                else
                    convert_w8<ADT>(w, A[2 * h][f], A[2 * h + 1][f]);
            }
        float sc[NA][4], zc[NA][4];
        if constexpr (G128) {
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const int ch = wn * WTN + f * 16 * NH + g * 4 * NH;   // this lane's 4 rows of fragment f: NH * 4 consecutive channels
                const tab_t sv = *(const tab_t*)(stg + ch * 2);
                const tab_t zv = *(const tab_t*)(stg + 256 + ch * 2);
#pragma unroll
                for (int o = 0; o < NH; ++o)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int c = NH * r + o;    // channel within the lane's NH * 4
                        sc[NH * f + o][r] = bits_to_f32<SDT>((sv[c >> 1] >> (16 * (c & 1))) & 0xFFFFu);
                        zc[NH * f + o][r] = c_off + zmul * bits_to_f32<SDT>((zv[c >> 1] >> (16 * (c & 1))) & 0xFFFFu);
                    }
            }
        }
        if constexpr (G128) {
            // software pipeline over the activation fragments: the MFMAs of fragment b are issued between
            // the fold instructions of fragment b - 1 (one MFMA, then a few vector instructions, and so on),
            // so that both units work at once within one wave
            constexpr int NM = 4 * (NA + 1);         // MFMAs per fragment
            constexpr int NV = NA * 4 * 2;           // fold instructions per fragment
            constexpr int VPM = (NV + NM - 1) / NM;
            v4f acc[2][NA], as[2];
#pragma unroll
            for (int b = 0; b <= FB; ++b) {
                if (b < FB) {
                    v4u B[4];
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) B[ks] = *(const v4u*)(sa + a_rd[ks >> 1][ks & 1] + b * 16 * 256);
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                        for (int a = 0; a < NA; ++a) acc[b & 1][a] = MT::mma(A[ks][a], B[ks], ks == 0 ? zero4 : acc[b & 1][a]);
                        as[b & 1] = MT::mma(ones, B[ks], ks == 0 ? zero4 : as[b & 1]);
                    }
                }
                if (b > 0) {
                    const int pb = b - 1;
#pragma unroll
                    for (int a = 0; a < NA; ++a)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            outv[a][pb][r] += sc[a][r] * (acc[pb & 1][a][r] - zc[a][r] * as[pb & 1][r]);
                }
                if (b > 0 && b < FB) {
#pragma unroll
                    for (int q = 0; q < NM; ++q) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int b = 0; b < FB; ++b) {
                v4u B[4];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) B[ks] = *(const v4u*)(sa + a_rd[ks >> 1][ks & 1] + b * 16 * 256);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                    for (int a = 0; a < NA; ++a) outv[a][b] = MT::mma(A[ks][a], B[ks], outv[a][b]);
                    asum[b] = MT::mma(ones, B[ks], asum[b]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    if constexpr (REFQ != 0) {
        // ---- per-weight rounding: a software pipeline over the slabs.  While the MFMAs of slab j run on
        // operands that are already dequantised in registers, the weights of slab j + 1 are read from LDS,
        // converted and dequantised into a second set - vector instructions placed between the MFMAs, two
        // per MFMA - so that the matrix cores and the vector unit of a SIMD work at the same time although
        // both waves of the SIMD cross the same barrier every slab.  The weight stage of slab j is free
        // from barrier j on (its operands were formed during slab j - 1), so the weights are copied three
        // slabs ahead into three stages, the tables two ahead.
        // Zero points that are whole numbers (the usual case) let the offset of the conversion and the zero point
        // go in one subtraction, x - (offset + zp): both forms are exact then, so the bits are the same and a
        // third of the rounding step's instructions is saved.  Whether all zero points of the tile's channels are
        // whole (and small enough for offset + zp to be exact in fp16) is found once per workgroup, before the
        // first copy is issued; if not, the two-step form runs.
        bool whole_zp = false;
        if constexpr (REFQ == 2) {
            int bad = 0;
            auto check = [&](uint32_t pair) {
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float z = bits_to_f32<SDT>((pair >> (16 * e)) & 0xFFFFu);
                    bad |= !(z == rintf(z) && fabsf(z) <= kWholeZpMax);
                }
            };
            if constexpr (G128) {
                const int pieces = (KT >> p.gshift) * 16;        // 16-byte pieces of the tile's 128 channels, row by row
                for (int e = threadIdx.x; e < pieces; e += 512) {
                    const v4u v = *(const v4u*)((const char*)p.zp + ((int64_t)(e >> 4) * p.N + n0) * 2 + (e & 15) * 16);
                    check(v[0]); check(v[1]); check(v[2]); check(v[3]);
                }
            } else {
                const uint16_t* const z16 = (const uint16_t*)p.zp + n0;
                if (threadIdx.x < BN / 2) check((uint32_t)z16[2 * threadIdx.x] | ((uint32_t)z16[2 * threadIdx.x + 1] << 16));
            }
            whole_zp = !__syncthreads_or(bad);
        }
        auto run = [&](auto merged_tag) {
        constexpr bool MERGED = decltype(merged_tag)::value;
        v4u A0[4][NA], A1[4][NA];
        auto dequant_slab = [&](v4u(&A)[4][NA], const char* sw, const char* stg) {
            if constexpr (RQBF) {
                constexpr float off = WBITS == 4 ? 8.f : 128.f;
                constexpr bool ONE_STEP = REFQ == 1 || MERGED;          // (no zero points: zeros)
                float s_[NA], z_[NA], c_[NA];
#pragma unroll
                for (int a = 0; a < NA; ++a) {
                    if constexpr (G128) {
                        const int ch = wn * WTN + (a / NH) * 16 * NH + NH * row16 + (a % NH);
                        s_[a] = bf16_bits_to_f32(*(const uint16_t*)(stg + ch * 2));
                        z_[a] = REFQ == 2 ? bf16_bits_to_f32(*(const uint16_t*)(stg + 256 + ch * 2)) : 0.f;
                    } else {
                        s_[a] = bq_s[a];
                        z_[a] = bq_z[a];
                    }
                    c_[a] = -(off + z_[a]) * s_[a];
                }
                auto dq = [&](float u0, float u1, int a) {
                    if constexpr (ONE_STEP) return ref_dq_bf16_merged(u0, u1, s_[a], c_[a]);
                    else return ref_dq_bf16(u0, u1, off, z_[a], s_[a]);
                };
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int f = 0; f < NF; ++f) {
                        const v4u w = *(const v4u*)(sw + w_rd[h] + f * 16 * 128);
#pragma unroll
                        for (int q = 0; q < 4; ++q) {      // 4 k of the row: operand 2 h + (q >> 1), registers 2 (q & 1), + 1
                            if constexpr (WBITS == 4) {
                                const uint32_t x = w[q] ^ 0x88888888u;      // two's complement -> offset by 8
                                float fe[4], fo[4];
                                bytes_to_f32(x & 0x0F0F0F0Fu, fe);
                                bytes_to_f32((x >> 4) & 0x0F0F0F0Fu, fo);
#pragma unroll
                                for (int i = 0; i < 2; ++i) {
                                    A[2 * h + (q >> 1)][2 * f][2 * (q & 1) + i] = dq(fe[2 * i], fe[2 * i + 1], 2 * f);
                                    A[2 * h + (q >> 1)][2 * f + 1][2 * (q & 1) + i] = dq(fo[2 * i], fo[2 * i + 1], 2 * f + 1);
                                }
                            } else {
                                float fb[4];
                                bytes_to_f32(w[q] ^ 0x80808080u, fb);
#pragma unroll
                                for (int i = 0; i < 2; ++i) A[2 * h + (q >> 1)][f][2 * (q & 1) + i] = dq(fb[2 * i], fb[2 * i + 1], f);
                            }
                        }
                    }
                return;
            }
            if constexpr (G128) {
#pragma unroll
                for (int a = 0; a < NA; ++a) {
                    const int ch = wn * WTN + (a / NH) * 16 * NH + NH * row16 + (a % NH);
                    rq_s[a] = pair_of_f16_bits(*(const uint16_t*)(stg + ch * 2));
                    rq_z[a] = pair_of_f16_bits(REFQ == 2 ? *(const uint16_t*)(stg + 256 + ch * 2) : 0u);
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int f = 0; f < NF; ++f) {
                    const v4u w = *(const v4u*)(sw + w_rd[h] + f * 16 * 128);
                    if constexpr (WBITS == 4 && ROUNDQ)
                        convert_w4_nat_f16_2off(w, A[2 * h][2 * f], A[2 * h + 1][2 * f], A[2 * h][2 * f + 1], A[2 * h + 1][2 * f + 1]);
                    else if constexpr (WBITS == 4)
                        convert_w4_nat<ADT>(w, A[2 * h][2 * f], A[2 * h + 1][2 * f], A[2 * h][2 * f + 1], A[2 * h + 1][2 * f + 1]);
                    else
                        convert_w8<ADT>(w, A[2 * h][f], A[2 * h + 1][f]);
                }
            if constexpr (ROUNDQ) {
                v2h sub[NA];
#pragma unroll
                for (int a = 0; a < NA; ++a) {
                    sub[a] = WBITS == 4 && (a % NH) == 1 ? rq_c_odd : rq_c;
                    if constexpr (MERGED) sub[a] = sub[a] + rq_z[a];
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int a = 0; a < NA; ++a)
                        A[ks][a] = ref_dq_f16<REFQ == 2 && !MERGED>(A[ks][a], sub[a], rq_z[a], rq_s[a]);
            }
        };
        auto mfma_slab = [&](const v4u(&A)[4][NA], const char* sa) {
#pragma unroll
            for (int b = 0; b < FB; ++b) {
                v4u B[4];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) B[ks] = *(const v4u*)(sa + a_rd[ks >> 1][ks & 1] + b * 16 * 256);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                    for (int a = 0; a < NA; ++a) outv[a][b] = MT::mma(A[ks][a], B[ks], outv[a][b]);
                    if constexpr (!ROUNDQ) asum[b] = MT::mma(ones, B[ks], asum[b]);
                }
            }
        };
        // the order asked of the scheduler: per activation fragment its four LDS reads, then each of its MFMAs
        // followed by two vector instructions of the dequantisation (what is left of those comes last)
        auto interleave = [&]() {
            // (first the LDS reads of the dequantisation: 2 NF weight pieces and, with group tables, 2 NA entries)
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * NF + (G128 ? 2 * NA : 0), 0);
#pragma unroll
            for (int b = 0; b < FB; ++b) {
                __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
                for (int q = 0; q < 4 * (NA + (ROUNDQ ? 0 : 1)); ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, RQBF ? (BM == 256 ? 3 : 6) : ROUNDQ ? 2 : 1, 0);
                }
            }
        };
#define FNN_RQ_ITER(CUR, NXT, CA, CWN, CTN, FA, FW, FT, J)                \
    do {                                                                  \
        wait_barrier();                                                   \
        copy_a(FA, (J) + 1);                                              \
        copy_t(FT, (J) + 2);                                              \
        copy_w(FW, (J) + 3);                                              \
        __builtin_amdgcn_sched_barrier(0);                                \
        dequant_slab(NXT, CWN, CTN);                                      \
        mfma_slab(CUR, CA);                                               \
        interleave();                                                     \
        __builtin_amdgcn_sched_barrier(0);                                \
    } while (0)
        // prologue: the weights and tables of slab 0 first (they are waited for at once), then what the loop
        // would have issued before its first barrier
        copy_w(sw0, 0);
        copy_t(st0, 0);
        copy_a(sa0, 0);
        copy_t(st1, 1);
        copy_w(sw1, 1);
        copy_w(sw2, 2);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070 | ((NCA + NCT + 2 * NCW) & 15) | (((NCA + NCT + 2 * NCW) >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        dequant_slab(A0, sw0, st0);
        __builtin_amdgcn_sched_barrier(0);
        int j = 0;
        for (; j + 6 <= KT; j += 6) {
            FNN_RQ_ITER(A0, A1, sa0, sw1, st1, sa1, sw0, st2, j);
            FNN_RQ_ITER(A1, A0, sa1, sw2, st2, sa0, sw1, st0, j + 1);
            FNN_RQ_ITER(A0, A1, sa0, sw0, st0, sa1, sw2, st1, j + 2);
            FNN_RQ_ITER(A1, A0, sa1, sw1, st1, sa0, sw0, st2, j + 3);
            FNN_RQ_ITER(A0, A1, sa0, sw2, st2, sa1, sw1, st0, j + 4);
            FNN_RQ_ITER(A1, A0, sa1, sw0, st0, sa0, sw2, st1, j + 5);
        }
        // (KT is a multiple of 2: the remaining slabs come in pairs and the operand sets line up)
        if (j < KT) {
            FNN_RQ_ITER(A0, A1, sa0, sw1, st1, sa1, sw0, st2, j);
            FNN_RQ_ITER(A1, A0, sa1, sw2, st2, sa0, sw1, st0, j + 1);
        }
        if (j + 2 < KT) {
            FNN_RQ_ITER(A0, A1, sa0, sw0, st0, sa1, sw2, st1, j + 2);
            FNN_RQ_ITER(A1, A0, sa1, sw1, st1, sa0, sw0, st2, j + 3);
        }
#undef FNN_RQ_ITER
        };
        if constexpr (REFQ == 2) {
            if (whole_zp) run(std::true_type{});
            else run(std::false_type{});
        } else {
            run(std::false_type{});
        }
    } else {
#define FNN_TILE_ITER(CA, CW, CT, FA, FW, FT, J)                          \
    do {                                                                  \
        wait_barrier();                                                   \
        copy_a(FA, (J) + 1);                                              \
        copy_t(FT, (J) + 1);                                              \
        copy_w(FW, (J) + 2);                                              \
        __builtin_amdgcn_sched_barrier(0);                                \
        slab(CA, CW, MOE && G128 ? mtab + (J) * 512 : CT);                \
        __builtin_amdgcn_sched_barrier(0);                                \
    } while (0)

    // prologue, in the order the loop issues them: slab 0 whole, then the weights of slab 1
    copy_a(sa0, 0);
    copy_t(st0, 0);
    copy_w(sw0, 0);
    copy_w(sw1, 1);
    __builtin_amdgcn_sched_barrier(0);
    // the stages rotate with periods 2 and 3: six iterations per round
    int j = 0;
    for (; j + 6 <= KT; j += 6) {
        FNN_TILE_ITER(sa0, sw0, st0, sa1, sw2, st1, j);
        FNN_TILE_ITER(sa1, sw1, st1, sa0, sw0, st2, j + 1);
        FNN_TILE_ITER(sa0, sw2, st2, sa1, sw1, st0, j + 2);
        FNN_TILE_ITER(sa1, sw0, st0, sa0, sw2, st1, j + 3);
        FNN_TILE_ITER(sa0, sw1, st1, sa1, sw0, st2, j + 4);
        FNN_TILE_ITER(sa1, sw2, st2, sa0, sw1, st0, j + 5);
    }
    // the remaining slabs (KT is a multiple of 2: checked on the host, so the activation stages line up)
    if (j < KT) { FNN_TILE_ITER(sa0, sw0, st0, sa1, sw2, st1, j); }
    if (j + 1 < KT) { FNN_TILE_ITER(sa1, sw1, st1, sa0, sw0, st2, j + 1); }
    if (j + 2 < KT) { FNN_TILE_ITER(sa0, sw2, st2, sa1, sw1, st0, j + 2); }
    if (j + 3 < KT) { FNN_TILE_ITER(sa1, sw0, st0, sa0, sw2, st1, j + 3); }
#undef FNN_TILE_ITER
    }
    // ---- per-channel scales: one fold at the end
    if constexpr (!G128 && !ROUNDQ) {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            float sc[4], zc[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = n0 + wn * WTN + (NH == 2 ? (a >> 1) * 32 + 2 * (4 * g + r) + (a & 1) : a * 16 + 4 * g + r);
                sc[r] = load_as_f32(p.scale, (MOE ? (int64_t)expert * q.stride_scale_be : 0) + n, p.scale_dtype);
                zc[r] = c_off + (has_zp ? load_as_f32(p.zp, (MOE ? (int64_t)expert * q.stride_zp_be : 0) + n, p.zp_dtype) : 0.f);
            }
#pragma unroll
            for (int b = 0; b < FB; ++b)
#pragma unroll
                for (int r = 0; r < 4; ++r) outv[a][b][r] = sc[r] * (outv[a][b][r] - zc[r] * asum[b][r]);
        }
    }

    // ---- bias, rounding, store: lane (row16, g) holds, for row m = .. + row16 of fragment b, the channels
    // int4: n0 + wn * 64 + f * 32 + 8 g .. + 7 (even and odd operands interleaved); int8: .. + f * 16 + 4 g .. + 3
    const bool out_f16 = p.out_dtype == FNN_F16;
    const bool vec_out = (p.ldc % 8) == 0 && ((uintptr_t)p.out % 16) == 0;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        const int nb = n0 + wn * WTN + f * 16 * NH + g * 4 * NH;
        float bias[4 * NH];
#pragma unroll
        for (int c = 0; c < 4 * NH; ++c) bias[c] = p.bias ? load_as_f32(p.bias, nb + c, p.bias_dtype) : 0.f;
#pragma unroll
        for (int b = 0; b < FB; ++b) {
            int m = m0 + wm * WTM + b * 16 + row16;
            if (!MOE && m >= p.M) continue;
            // (rows converted from bf16 were scaled by a power of two: the exact inverse)
            float un = 1.f;
            if constexpr (ROUNDQ) un = p.act_unscale ? p.act_unscale[m] : 1.f;
            if constexpr (MOE) {       // the output row is the routed row; `un` carries the routing weight
                m = q.sorted_ids[m];
                if (m >= q.num_valid) continue;
                if (q.mul_w) un = load_as_f32(q.topk_w, m, q.topk_w_dtype);
            }
            uint32_t pk[2 * NH];
#pragma unroll
            for (int c = 0; c < 4 * NH; c += 2) {
                // channel c of the lane: int4: register c >> 1 of operand 2 f + (c & 1); int8: register c of operand f
                float v0 = (NH == 2 ? outv[2 * f][b][c >> 1] : outv[f][b][c]) * un;
                float v1 = (NH == 2 ? outv[2 * f + 1][b][c >> 1] : outv[f][b][c + 1]) * un;
                if (p.bias) {
                    v0 = add_bias<WBITS>(v0, bias[c], p.out_dtype);
                    v1 = add_bias<WBITS>(v1, bias[c + 1], p.out_dtype);
                }
                const uint32_t b0 = out_f16 ? f32_to_f16_bits(v0) : f32_to_bf16_bits(v0);
                const uint32_t b1 = out_f16 ? f32_to_f16_bits(v1) : f32_to_bf16_bits(v1);
                pk[c >> 1] = (b0 & 0xFFFFu) | (b1 << 16);
            }
            uint16_t* dst = (uint16_t*)p.out + (int64_t)m * p.ldc + nb;
            if (vec_out) {
                if constexpr (NH == 2) *(v4u*)dst = v4u{pk[0], pk[1], pk[2], pk[3]};
                else *(v2u*)dst = v2u{pk[0], pk[1]};
            } else {
#pragma unroll
                for (int c = 0; c < 4 * NH; ++c) dst[c] = (uint16_t)(pk[c >> 1] >> (16 * (c & 1)));
            }
        }
    }
}

// Rows per tile: 256 for int4 from 129 rows on - unless the 256-row tiles would leave half the CUs idle: then
// twice as many workgroups of 128 rows, each with half the work, finish sooner.
static int tile_rows(const WoArgs& p, int wbits) {
    const int64_t tiles256 = (int64_t)((p.M + 255) / 256) * (p.N / 128);
    return (p.M <= 128 || wbits == 8 || tiles256 <= 128) ? 128 : 256;
}

int wo_tile_count(const WoArgs& p, int wbits) {
    const int bm = tile_rows(p, wbits);
    return (int)((p.M + bm - 1) / bm) * (p.N / 128);
}

// Launches the tiled kernel if the shape suits it; returns false otherwise.
template <int WBITS, int ADT>
static bool launch_tile_t(WoArgs& p, hipStream_t st) {
    constexpr int NH = WBITS == 4 ? 2 : 1;
    if (p.M <= 64 || p.N % 128 != 0 || p.K % 256 != 0 || p.K < 512) return false;
    // tables per channel, or per group of 128, 256, 512 .. values
    const int gs = p.group == 0 ? 0 : group_shift(p.group);
    if (gs < 0 || (p.group != 0 && p.K % p.group != 0)) return false;
    p.gshift = gs;
    if (p.lda % 8 != 0 || p.ldw % 16 != 0 || ((uintptr_t)p.qw % 16) != 0 || ((uintptr_t)p.act % 16) != 0) return false;
    // the copies address rows with 32-bit offsets from the tile's first row
    if ((int64_t)256 * p.lda * 2 >= (1LL << 31) || (int64_t)(128 / NH) * p.ldw >= (1LL << 31)) return false;
    if (p.group != 0) {
        const bool tables16 = is16(p.scale_dtype) && (!p.zp || p.zp_dtype == p.scale_dtype) &&
                              ((uintptr_t)p.scale % 16) == 0 && (!p.zp || ((uintptr_t)p.zp % 16) == 0);
        if (!tables16) return false;
    }
    if constexpr (ADT == FNN_BF16) {
        // bf16 rows become fp16 rows where scratch was given: the weights are then rounded as the reference does
        WoArgs q;
        if (convert_act_to_f16(p, q, st) && launch_tile_t<WBITS, FNN_F16>(q, st)) return true;
    }
    const int bm = tile_rows(p, WBITS);
    const int tiles_m = (p.M + bm - 1) / bm;
    const int tiles = tiles_m * (p.N / 128);
    const dim3 grid(((tiles + 7) / 8) * 8);   // (workgroups beyond the last tile return at once)
    // fp16 activations with fp16 tables: every weight rounded as the reference rounds it
    // .. and bf16 activations with bf16 tables
    const bool refq = p.scale_dtype == ADT && (!p.zp || p.zp_dtype == ADT) &&
                      (p.group != 0 || (((uintptr_t)p.scale % 2) == 0 && (!p.zp || ((uintptr_t)p.zp % 2) == 0)));
    note_kernel(refq ? "gemm_wo_tile_kernel(per-weight rounding)" : "gemm_wo_tile_kernel", WBITS, bm, 128);
#define FNN_TILE(G, SDTV, RQ)                                                                            \
    do {                                                                                                 \
        if constexpr (WBITS == 4) {                                                                      \
            if (bm == 256) {                                                                             \
                gemm_wo_tile_kernel<WBITS, ADT, G, SDTV, 256, RQ><<<grid, dim3(512), 0, st>>>(p, tiles_m, tiles, MoeArgs{}); \
                break;                                                                                   \
            }                                                                                            \
        }                                                                                                \
        gemm_wo_tile_kernel<WBITS, ADT, G, SDTV, 128, RQ><<<grid, dim3(512), 0, st>>>(p, tiles_m, tiles, MoeArgs{}); \
    } while (0)
    if (refq) {
        if (p.group != 0) { if (p.zp) FNN_TILE(true, ADT, 2); else FNN_TILE(true, ADT, 1); }
        else { if (p.zp) FNN_TILE(false, ADT, 2); else FNN_TILE(false, ADT, 1); }
        return true;
    }
    if (p.group != 0) {
        if (p.scale_dtype == FNN_F16) FNN_TILE(true, FNN_F16, 0);
        else FNN_TILE(true, FNN_BF16, 0);
    } else {
        FNN_TILE(false, FNN_F16, 3);
    }
#undef FNN_TILE
    return true;
}

// Mixture of experts, int4 weights with per-channel tables, many routed rows per expert; false where this
// form does not apply.
template <int ADT>
static bool launch_tile_moe_t(WoArgs& p, const MoeArgs& q, hipStream_t st) {
    if (p.group == 128) {
        const int tiles_m = p.M / 128;
        const int tiles = tiles_m * (p.N / 128);
        const dim3 grid(((tiles + 7) / 8) * 8);
        note_kernel("gemm_wo_tile_kernel(moe, group tables)", 4, 128, 128);
        if (p.scale_dtype == FNN_F16)
            gemm_wo_tile_kernel<4, ADT, true, FNN_F16, 128, 0, true><<<grid, dim3(512), 0, st>>>(p, tiles_m, tiles, q);
        else
            gemm_wo_tile_kernel<4, ADT, true, FNN_BF16, 128, 0, true><<<grid, dim3(512), 0, st>>>(p, tiles_m, tiles, q);
        return true;
    }
    const int bm = q.block_m % 256 == 0 ? 256 : 128;
    const int tiles_m = p.M / bm;
    const int tiles = tiles_m * (p.N / 128);
    const dim3 grid(((tiles + 7) / 8) * 8);
    note_kernel("gemm_wo_tile_kernel(moe)", 4, bm, 128);
    if (bm == 256) gemm_wo_tile_kernel<4, ADT, false, FNN_F16, 256, 3, true><<<grid, dim3(512), 0, st>>>(p, tiles_m, tiles, q);
    else gemm_wo_tile_kernel<4, ADT, false, FNN_F16, 128, 3, true><<<grid, dim3(512), 0, st>>>(p, tiles_m, tiles, q);
    return true;
}

bool launch_wo_tile_moe(WoArgs& p, const MoeArgs& q, int act_dtype, hipStream_t st) {
    const int64_t rows = (q.num_valid + q.top_k - 1) / q.top_k;          // activation rows
    const int G = p.K / 128;
    // group tables: contiguous [expert][channel][group] of one 16-bit type, at most 64 groups
    const bool tables_ok = p.group == 0 ? q.stride_scale_n == 1 && (!p.zp || (q.stride_zp_n == 1 && p.zp_dtype != FNN_I8))
                                        : p.group == 128 && G <= 64 && is16(p.scale_dtype) && q.stride_scale_k == 1 &&
                                              q.stride_scale_n == G &&
                                              (!p.zp || (p.zp_dtype == p.scale_dtype && q.stride_zp_k == 1 && q.stride_zp_n == G));
    const bool ok = tables_ok && q.block_m % 128 == 0 && q.EM % q.block_m == 0 && p.N % 128 == 0 &&
                    p.K % 256 == 0 && p.K >= 512 && p.lda % 8 == 0 && p.ldw % 16 == 0 &&
                    q.stride_be % 16 == 0 && ((uintptr_t)p.qw % 16) == 0 && ((uintptr_t)p.act % 16) == 0 &&
                    rows * p.lda * 2 < (1LL << 32) && (int64_t)64 * p.ldw < (1LL << 31) &&
                    (int64_t)(p.M / 128) * (p.N / 128) < (1LL << 31);
    if (!ok) return false;
    return act_dtype == FNN_F16 ? launch_tile_moe_t<FNN_F16>(p, q, st) : launch_tile_moe_t<FNN_BF16>(p, q, st);
}

bool launch_wo_tile(WoArgs& p, int wbits, int act_dtype, hipStream_t st) {
    if (wbits == 4) return act_dtype == FNN_F16 ? launch_tile_t<4, FNN_F16>(p, st) : launch_tile_t<4, FNN_BF16>(p, st);
    return act_dtype == FNN_F16 ? launch_tile_t<8, FNN_F16>(p, st) : launch_tile_t<8, FNN_BF16>(p, st);
}

}  // namespace fnn
