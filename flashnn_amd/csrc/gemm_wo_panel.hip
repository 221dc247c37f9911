// Weight-only GEMM for 9 .. a few hundred activation rows ("panel" kernel, gfx950).
//
// The weights are still read exactly once per pass and go straight from global memory into the
// MFMA "A" operand; what changes against the decode kernels is the activation side.  With 16..64
// activation rows every weight tile needs M*K*2 bytes of activations, too much to pull through
// the vector memory path once per 16 weight rows.  Here a workgroup owns 64 weight rows (four
// waves, 16 rows each) and the four waves share each 128-k slab of the activation panel through
// LDS:
//   * 4*KS waves; wave (rt, ks) owns weight rows 16*rt .. +15 of the tile and the ks-th part of K;
//   * activations: slabs of (16*MB rows) x 128 k are copied global -> LDS with 16-byte
//     direct-to-LDS loads into a ring of 4 stages (3 slabs ahead).  The 16-byte chunks of a row
//     are stored at slot (chunk ^ (row & 15)) so that the 16 lanes that read the same chunk of 16
//     different rows hit 16 different bank groups;
//   * weights: two 16-byte loads per lane and slab, kept 4 slabs ahead in registers and fetched
//     as full 128-byte lines (8 rows per load); a wave-private LDS staging area reshapes them into
//     the MFMA operand layout; the refill of a register is issued right after its last use;
//   * group scales and zero points (group == 128): one 16-byte load each per lane and slab,
//     4 slabs ahead, folded into the running output at the end of each slab:
//         out += s * (acc - (c + zp) * sum_k a_k),
//     c being the constant the exponent-trick conversion adds, sum_k a_k coming from an MFMA
//     against ones;
//   * all loads of an iteration are issued in a fixed order, so "slab j has landed" is one
//     s_waitcnt vmcnt(X) with a compile-time X, followed by a bare s_barrier;
//   * the K parts are added through LDS in a fixed order, then bias, rounding, 16-byte stores.
//
// Reference semantics: flashnn/quant_gemm.py:148-206.
#include <type_traits>

#include "wo_common.h"

namespace fnn {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// G128: per-group tables with group size 128, entries of type SDT (fp16 or bf16), zero points in
// the same type; otherwise per-channel scales of any type, applied once at the end.
// RT: 16-row weight tiles per workgroup (4, 2 or 1); the 8 waves are RT tiles x KS = 8 / RT parts of K.
// Fewer rows per workgroup make more workgroups for matrices with few rows, at the price of each
// activation slab being shared by fewer waves.  K parts may differ by one slab; all waves run the
// same number of iterations (the barriers are shared) and skip the work of slabs they do not have.
// D: slabs of weights in flight per wave (8 loads per lane in flight stream faster than 16: measured
// 19.8 against 21.7 us for 117 MB in a load-only model).  NTL: non-temporal weight loads, for a
// single pass over the weights.
// REFQ (1, or 2 with zero points; fp16 activations, per-channel fp16 scales and zero points): every weight is dequantised and rounded to
// fp16 as the reference's torch path does before the dot product (ref_dq_f16 in wo_common.h); the MFMAs
// against ones and the fold at the end are then not needed.  With bf16 activations and per-channel bf16 tables
// the same with both roundings to bf16 (ref_dq_bf16: fp32 arithmetic; the short form where every zero point of
// the wave's rows is whole, the two-step form otherwise, chosen per wave).  (The same with tables per group of 128 - a
// lane fetching its row's scale and zero point slab by slab, bf16 rows converted to fp16 by a pass of their
// own - was built and measured on A16W4, K = 8192, N = 28672: 16 rows 28.0 -> 38.5 us, 64 rows 52.5 -> 56.5 us.
// Three more instructions per pair of weights where the fold costs two per output and slab: at these row
// counts the kernel streams weights, and the vector unit has no room for it.  Not kept; the tiled kernel for
// more than 64 rows has it.)
// GSUB = 2: tables per group of 64 values - two groups per slab, each half of the slab's MFMAs folded with its own
// table row (G128 is set as well: the table path is the same, with twice the rows).
template <int WBITS, int ADT, bool G128, int SDT, int MB, int RT, int D, bool NTL, bool MOE = false, int REFQ = 0, int GSUB = 1>
__global__ __launch_bounds__(512) void gemm_wo_panel_kernel(const WoArgs p, const int passes, const MoeArgs q) {
    static_assert(!REFQ || (!G128 && !MOE), "reference rounding: per-channel tables of the activations' type");
    // bf16 activations with bf16 tables: both roundings to bf16, worked in fp32 (ref_dq_bf16 in wo_common.h)
    constexpr bool RQBF = REFQ != 0 && ADT == FNN_BF16;
    static_assert(GSUB == 1 || (GSUB == 2 && G128 && !MOE), "groups of 64: plain calls with group tables");
    // Gathered form with group tables: the reference's mixture-of-experts launcher lays them out
    // [expert][channel][group] (flashnn/triton_kernels/fused_moe_a16w4.py:336-344), the transpose of the
    // [group][channel] tables above, so 16-byte loads of 8 neighbouring channels do not exist.  The
    // workgroup's slice of both tables (its channels x all groups, at most 32 KB) is transposed into LDS
    // once, and the per-slab table reads come from there instead of from memory.
    constexpr bool TABLDS = MOE && G128;
    constexpr bool TABG = G128 && !TABLDS;      // tables fetched from memory, slab by slab
    constexpr int KS = 8 / RT;
    typedef MfmaT<ADT> MT;
    constexpr int NH = WBITS == 4 ? 2 : 1;      // channels per weight row
    constexpr int NCL = 4 * NH;                 // consecutive channels per lane
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    constexpr int SLAB = MB * 16 * 256;         // bytes of one activation slab: 16*MB rows x 128 k
    constexpr int STG = KS * SLAB;
    constexpr int RED = (KS - 1) * RT * MB * NH * 4 * 64 * 4;
    constexpr int STG0 = STG > RED ? STG : RED;
    // one array per stage: the compiler then knows that reads of one stage cannot alias the
    // copies in flight into another
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

    // workgroups id, id+8, id+16 .. run on the same XCD: give them the same weight tile and
    // consecutive passes so that the tile is fetched from HBM once and re-read from that L2
    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = wrows / (16 * RT);
    const int y = blockIdx.x >> 3;
    const int pass = y % passes;
    const int tile = (y / passes) * 8 + (blockIdx.x & 7);
    if (tile >= tiles) return;
    const int m_base = p.m_base + pass * (MB * 16);
    const int row0 = (tile * RT + rt) * 16;
    // mixture of experts: the pass covers sorted rows m_base .. of one expert; passes beyond the rows
    // in use have nothing to do
    int expert = 0;
    if constexpr (MOE) {
        if (m_base >= q.ntpp[0]) return;
        expert = q.expert_ids[m_base / q.block_m];
    }
    auto token_of = [&](int r) -> int {
        const int sidx = m_base + r;
        return sidx < q.EM ? q.sorted_ids[sidx] : q.num_valid;
    };

    // K = 128 * (KT - 1) + tail_k.  With per-channel scales the last slab may be partial (tail_k = 32, 64
    // or 96): lanes whose 16-byte chunk lies beyond K fetch the first chunk of their row piece instead
    // (bytes that exist), and the activation fragments of those k are replaced by zeros before the MFMAs,
    // which removes them from the products and from the activation sums alike.
    const int KT = (p.K + 127) / 128;
    const int tail_k = p.K - (KT - 1) * 128;
    const bool part_tail = tail_k < 128 && ks == KS - 1;   // wave-uniform
    const int sl0 = KT * ks / KS;               // this wave's slabs: sl0 .. sl0 + nsl - 1
    const int nsl = KT * (ks + 1) / KS - sl0;
    const int n_iter = ((KT + KS - 1) / KS + D - 1) / D * D;   // iterations of every wave

    // ---- weights: load h of a slab fetches rows 8h .. 8h+7 of the wave's tile, 8 lanes per row, one
    // full 128-byte line per row (16 rows x 64 bytes per load, the MFMA operand's own shape, streams
    // a quarter slower from HBM).  A wave-private 2 KB staging area in LDS turns the two loads
    // into the operand layout: row i at i*128, its 16-byte chunk c at slot c ^ ((i >> 1) & 7).
    // An address is a wave-uniform 64-bit base (matrix, tile, slab: scalar arithmetic) plus the lane's 32-bit
    // offset, the form the load instruction takes directly: no 64-bit vector adds per load.
    const int wr8 = lane >> 3, wc8 = lane & 7;
    const char* const wbase = (const char*)p.qw + (MOE ? (int64_t)expert * q.stride_be : 0) + (int64_t)row0 * p.ldw +
                              (int64_t)sl0 * 128;
    const int64_t w_half = 8 * p.ldw;
    const uint32_t woff = (uint32_t)wr8 * (uint32_t)p.ldw + wc8 * 16;
    const uint32_t woff_tail = wc8 * 16 >= tail_k ? woff - wc8 * 16 : woff;
    auto load_w = [&](int jj, int half) -> v4u {
        const int j = min(jj, nsl - 1);
        const char* base = wbase + (int64_t)j * 128 + half * w_half;               // scalar
        const uint32_t off = part_tail && j == nsl - 1 ? woff_tail : woff;          // uniform choice
        const v4u* src = (const v4u*)(base + off);
        return NTL ? __builtin_nontemporal_load(src) : *src;
    };
    char* const wmine = wst + wave * 2048;
    int wwr[2], wrd[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        wwr[h] = (8 * h + wr8) * 128 + ((wc8 ^ ((4 * h + (wr8 >> 1)) & 7)) << 4);
        wrd[h] = li * 128 + (((4 * h + lg) ^ ((li >> 1) & 7)) << 4);
    }

    // ---- activation copies: thread t of the K part copies chunk (t & 15) ^ (t >> 4) of rows
    // (t >> 4) + 16 i into slot (t & 15) of those rows
    // (the RT waves of a K part make 64 RT lanes; copy i of a wave covers rows 4 RT i + (t >> 4))
    constexpr int NCP = MB * 4 / RT;            // copies per wave and slab
    const int t = rt * 64 + lane;
    const int tokq = t >> 4;
    // (rows of a pass lie within 64 rows of its first one, so their offsets fit 32 bits; gathered rows do not)
    typedef typename std::conditional<MOE, int64_t, uint32_t>::type aoff_t;
    const char* act_part = (const char*)p.act + (int64_t)sl0 * 256 + (MOE ? 0 : (int64_t)m_base * p.lda * 2);
    aoff_t goff[NCP], goff_tail[NCP];
#pragma unroll
    for (int i = 0; i < NCP; ++i) {
        const int tok = i * (4 * RT) + tokq;
        const int chunk = (t & 15) ^ (tok & 15);
        if constexpr (MOE) {
            const int id = token_of(tok);
            goff[i] = (int64_t)(id < q.num_valid ? id / q.top_k : 0) * p.lda * 2 + chunk * 16;
        } else {
            goff[i] = (uint32_t)min(tok, p.M - 1 - m_base) * (uint32_t)(p.lda * 2) + chunk * 16;
        }
        goff_tail[i] = chunk * 8 >= tail_k ? goff[i] - chunk * 16 : goff[i];
    }
    auto copy_act = [&](char* stage, int jj) {
        const int j = min(jj, nsl - 1);
        const char* src = act_part + (int64_t)j * 256;
        const bool last = part_tail && j == nsl - 1;
#pragma unroll
        for (int i = 0; i < NCP; ++i)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + (last ? goff_tail[i] : goff[i])),
                                             (lds_ptr_t)(stage + ks * SLAB + (i * RT * 64 + rt * 64) * 16), 16, 0, 0);
    };
    // ---- activation fragment reads: lane (li, lg) reads chunks 8 s + 2 lg + h of row 16 mb + li
    int rd[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int h = 0; h < 2; ++h) rd[s][h] = ks * SLAB + li * 256 + (((s * 8 + lg * 2 + h) ^ li) << 4);

    // ---- group tables: NCL consecutive channels per lane
    typedef typename std::conditional<NH == 2, v4u, v2u>::type tab_t;
    const int n0 = NH * (row0 + 4 * lg);
    const uint16_t* sptr = (const uint16_t*)p.scale + NH * row0;             // scalar
    const uint16_t* zptr = (p.zp ? (const uint16_t*)p.zp : (const uint16_t*)p.scale) + NH * row0;
    const uint32_t tab_off = NH * 4 * lg * 2;                                                        // bytes
    const bool has_zp = p.zp != nullptr;
    // without zero points the second table load reads the scales again and is multiplied away
    const float zmul = has_zp ? 1.f : 0.f;
    // (groups of 128 << gshift values: the slab's table row is its number >> gshift; groups of 64: rows 2 j and 2 j + 1)
    auto load_tab = [&](const uint16_t* base, int jj, int sub) -> tab_t {
        const int slab = sl0 + min(jj, nsl - 1);
        const int j = GSUB == 2 ? 2 * slab + sub : slab >> p.gshift;
        return *(const tab_t*)((const char*)(base + (int64_t)j * p.N) + tab_off);
    };

    // REFQ: the scale and zero point of the weight row this lane feeds to the MFMAs (row li of the tile)
    v2h rq_s[NH], rq_z[NH];
    const v2h rq_c = pair_of_f16_bits(WBITS == 4 ? 0x6408u : 0x6480u);   // 1032 / 1152: what the conversion adds
    float bq_s[2], bq_z[2], bq_c[2];                                     // the same as fp32 numbers (bf16 tables)
    bool whole_zp = true;    // wave-uniform: every zero point of the wave's rows is whole and at most 128 (one-step form)
    if constexpr (REFQ) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const int n = NH * (row0 + li) + h;
            const uint32_t sb = ((const uint16_t*)p.scale)[n], zb = p.zp ? ((const uint16_t*)p.zp)[n] : 0u;
            if constexpr (RQBF) {
                bq_s[h] = bf16_bits_to_f32(sb);
                bq_z[h] = bf16_bits_to_f32(zb);
                bq_c[h] = -((WBITS == 4 ? 8.f : 128.f) + bq_z[h]) * bq_s[h];
                whole_zp = whole_zp && bf16_zp_is_whole(bq_z[h]);
            } else {
                rq_s[h] = pair_of_f16_bits(sb);
                rq_z[h] = pair_of_f16_bits(zb);
            }
        }
        if constexpr (RQBF && REFQ == 2) whole_zp = __builtin_amdgcn_ballot_w64(!whole_zp) == 0;
    }

    v4f outv[MB][NH], accg[MB][NH], asum[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        asum[mb] = v4f{0, 0, 0, 0};
#pragma unroll
        for (int h = 0; h < NH; ++h) { outv[mb][h] = v4f{0, 0, 0, 0}; accg[mb][h] = v4f{0, 0, 0, 0}; }
    }
    const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};

    // loads issued per iteration, in this order: NCP copies, 2 weight loads, 2 table loads
    constexpr int C = NCP + 2 + (TABG ? 2 * GSUB : 0);
    // the newest load slab j depends on is its last copy, issued three iterations earlier; after
    // it came the rest of that iteration and two whole ones
    constexpr int X = (C - NCP) + 2 * C;
    static_assert(X < 64, "vmcnt range");
    auto wait_barrier = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070 | (X & 15) | ((X >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);   // nothing of the slab's work moves above the wait
    };

    v4u wq[D][2];
    tab_t sq[4][GSUB], zq[4][GSUB];
    constexpr int CHW = RT * 16 * NH;           // channels of the workgroup
    constexpr int TABG_MAX = 64;                // groups the LDS tables hold (K <= 8192)
    __shared__ __attribute__((aligned(16))) uint16_t tabs[TABLDS ? 2 * TABG_MAX * CHW : 8];
    const int chl = NH * (rt * 16 + 4 * lg);    // the lane's first channel within the workgroup
    auto lds_tab = [&](int which, int jj) -> tab_t {
        const int kg = sl0 + min(jj, nsl - 1);
        return *(const tab_t*)(tabs + (which * TABG_MAX + kg) * CHW + chl);
    };

    auto fold = [&](const tab_t sv, const tab_t zv) {
        float sc[NCL], zc[NCL];
#pragma unroll
        for (int c = 0; c < NCL; ++c) {
            const uint32_t sb = (sv[c >> 1] >> (16 * (c & 1))) & 0xFFFFu;
            const uint32_t zb = (zv[c >> 1] >> (16 * (c & 1))) & 0xFFFFu;
            sc[c] = bits_to_f32<SDT>(sb);
            zc[c] = c_off + zmul * bits_to_f32<SDT>(zb);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int c = NH == 2 ? 2 * r + h : r;
                    outv[mb][h][r] += sc[c] * (accg[mb][h][r] - zc[c] * asum[mb][r]);
                    accg[mb][h][r] = 0.f;
                }
            asum[mb] = v4f{0, 0, 0, 0};
        }
    };

    // All activation fragments of the slab are requested first, the weights are converted while
    // those reads are in flight, and the MFMAs then run back to back behind a single wait.
    auto compute = [&](auto one_step_tag, const char* stage, const v4u w0, const v4u w1, const bool last, const tab_t s_first,
                       const tab_t z_first) {
        constexpr bool ONE_STEP = decltype(one_step_tag)::value;
        v4u bf[2][MB][2];
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                bf[s][mb][0] = *(const v4u*)(stage + rd[s][0] + mb * 4096);
                bf[s][mb][1] = *(const v4u*)(stage + rd[s][1] + mb * 4096);
            }
        if (last) {   // partial slab: fragment (s, h) of this lane holds k = 8 * (8 s + 2 lg + h) .. + 7
            asm volatile("" ::: "memory");   // a branch, taken once per wave, not sixteen selects in every slab
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const bool beyond = (8 * s + 2 * lg + h) * 8 >= tail_k;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) bf[s][mb][h] = beyond ? v4u{0, 0, 0, 0} : bf[s][mb][h];
                }
        }
        if constexpr (WBITS == 4) {
            v4u e[2][2], o[2][2];
            if constexpr (RQBF) {
                dq_w4_bf16<true, ONE_STEP>(w0, bq_s, bq_z, bq_c, e[0][0], e[0][1], o[0][0], o[0][1]);
                dq_w4_bf16<true, ONE_STEP>(w1, bq_s, bq_z, bq_c, e[1][0], e[1][1], o[1][0], o[1][1]);
            } else {
                convert_w4_nat<ADT>(w0, e[0][0], e[0][1], o[0][0], o[0][1]);
                convert_w4_nat<ADT>(w1, e[1][0], e[1][1], o[1][0], o[1][1]);
            }
            if constexpr (REFQ != 0 && !RQBF) {
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        e[s][h] = ref_dq_f16<REFQ == 2>(e[s][h], rq_c, rq_z[0], rq_s[0]);
                        o[s][h] = ref_dq_f16<REFQ == 2>(o[s][h], rq_c, rq_z[NH - 1], rq_s[NH - 1]);
                    }
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    accg[mb][0] = MT::mma(e[s][0], bf[s][mb][0], accg[mb][0]);
                    accg[mb][1] = MT::mma(o[s][0], bf[s][mb][0], accg[mb][1]);
                    if constexpr (!REFQ) asum[mb] = MT::mma(ones, bf[s][mb][0], asum[mb]);
                    accg[mb][0] = MT::mma(e[s][1], bf[s][mb][1], accg[mb][0]);
                    accg[mb][1] = MT::mma(o[s][1], bf[s][mb][1], accg[mb][1]);
                    if constexpr (!REFQ) asum[mb] = MT::mma(ones, bf[s][mb][1], asum[mb]);
                }
                if constexpr (GSUB == 2) { if (s == 0) fold(s_first, z_first); }     // values 0 .. 63 of the slab: a group of their own
            }
        } else {
            v4u c[2][2];
            if constexpr (RQBF) {
                dq_w8_bf16<ONE_STEP>(w0, bq_s[0], bq_z[0], bq_c[0], c[0][0], c[0][1]);
                dq_w8_bf16<ONE_STEP>(w1, bq_s[0], bq_z[0], bq_c[0], c[1][0], c[1][1]);
            } else {
                convert_w8<ADT>(w0, c[0][0], c[0][1]);
                convert_w8<ADT>(w1, c[1][0], c[1][1]);
            }
            if constexpr (REFQ != 0 && !RQBF) {
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int h = 0; h < 2; ++h) c[s][h] = ref_dq_f16<REFQ == 2>(c[s][h], rq_c, rq_z[0], rq_s[0]);
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    accg[mb][0] = MT::mma(c[s][0], bf[s][mb][0], accg[mb][0]);
                    if constexpr (!REFQ) asum[mb] = MT::mma(ones, bf[s][mb][0], asum[mb]);
                    accg[mb][0] = MT::mma(c[s][1], bf[s][mb][1], accg[mb][0]);
                    if constexpr (!REFQ) asum[mb] = MT::mma(ones, bf[s][mb][1], asum[mb]);
                }
                if constexpr (GSUB == 2) { if (s == 0) fold(s_first, z_first); }
            }
        }
    };

#define FNN_PANEL_ITER(Q, W, CUR, FREE, JJ)                                \
    do {                                                                   \
        wait_barrier();                                                    \
        copy_act(FREE, (JJ) + 3);                                          \
        const bool mine_ = (JJ) < nsl;   /* wave-uniform */                \
        if (mine_) {                                                       \
            *(v4u*)(wmine + wwr[0]) = wq[W][0];                            \
            *(v4u*)(wmine + wwr[1]) = wq[W][1];                            \
        }                                                                  \
        wq[W][0] = load_w((JJ) + D, 0);                                    \
        wq[W][1] = load_w((JJ) + D, 1);                                    \
        __builtin_amdgcn_sched_barrier(0);                                 \
        if (mine_) {                                                       \
            bool two_step_ = false;                                        \
            if constexpr (RQBF && REFQ == 2) two_step_ = !whole_zp;        \
            if (two_step_)                                                 \
                compute(std::integral_constant<bool, !(RQBF && REFQ == 2)>{}, CUR, *(const v4u*)(wmine + wrd[0]), \
                        *(const v4u*)(wmine + wrd[1]), !G128 && part_tail && (JJ) == nsl - 1, sq[Q][0], zq[Q][0]); \
            else                                                           \
                compute(std::true_type{}, CUR, *(const v4u*)(wmine + wrd[0]), *(const v4u*)(wmine + wrd[1]), \
                        !G128 && part_tail && (JJ) == nsl - 1, sq[Q][0], zq[Q][0]); \
            if constexpr (TABLDS) fold(lds_tab(0, (JJ)), lds_tab(1, (JJ))); \
            else if constexpr (G128) fold(sq[Q][GSUB - 1], zq[Q][GSUB - 1]); \
        }                                                                  \
        if constexpr (TABG) {                                              \
            _Pragma("unroll") for (int sub_ = 0; sub_ < GSUB; ++sub_) {    \
                sq[Q][sub_] = load_tab(sptr, (JJ) + 4, sub_);              \
                zq[Q][sub_] = load_tab(zptr, (JJ) + 4, sub_);              \
            }                                                              \
        }                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                 \
    } while (0)

    // ---- prologue: the older weight slabs first, then the same issue order as the three
    // iterations before the first one
#pragma unroll
    for (int d = 0; d <= D - 4; ++d) {
        wq[d][0] = load_w(d, 0);
        wq[d][1] = load_w(d, 1);
    }
    if constexpr (TABG) { for (int sub = 0; sub < GSUB; ++sub) { sq[0][sub] = load_tab(sptr, 0, sub); zq[0][sub] = load_tab(zptr, 0, sub); } }
    __builtin_amdgcn_sched_barrier(0);
    copy_act(st0, 0);
    wq[D - 3][0] = load_w(D - 3, 0);
    wq[D - 3][1] = load_w(D - 3, 1);
    if constexpr (TABG) { for (int sub = 0; sub < GSUB; ++sub) { sq[1][sub] = load_tab(sptr, 1, sub); zq[1][sub] = load_tab(zptr, 1, sub); } }
    __builtin_amdgcn_sched_barrier(0);
    copy_act(st1, 1);
    wq[D - 2][0] = load_w(D - 2, 0);
    wq[D - 2][1] = load_w(D - 2, 1);
    if constexpr (TABG) { for (int sub = 0; sub < GSUB; ++sub) { sq[2][sub] = load_tab(sptr, 2, sub); zq[2][sub] = load_tab(zptr, 2, sub); } }
    __builtin_amdgcn_sched_barrier(0);
    copy_act(st2, 2);
    wq[D - 1][0] = load_w(D - 1, 0);
    wq[D - 1][1] = load_w(D - 1, 1);
    if constexpr (TABG) { for (int sub = 0; sub < GSUB; ++sub) { sq[3][sub] = load_tab(sptr, 3, sub); zq[3][sub] = load_tab(zptr, 3, sub); } }
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (TABLDS) {
        // every channel's groups are contiguous in memory: 16-byte loads of 8 groups, written to
        // [group][channel]; behind the barrier everything the prologue asked for has landed as well
        const int G = p.K / 128;
        const int ch0 = NH * tile * RT * 16;
        const uint16_t* sg = (const uint16_t*)p.scale + (int64_t)expert * q.stride_scale_be + (int64_t)ch0 * G;
        const uint16_t* zg = p.zp ? (const uint16_t*)p.zp + (int64_t)expert * q.stride_zp_be + (int64_t)ch0 * G : sg;
        const int per_ch = G / 8;
        // int8 zero points (one byte per group) are widened to the scales' type on their way into the table
        const bool zp_i8 = p.zp && p.zp_dtype == FNN_I8;
        const int8_t* zg8 = zp_i8 ? (const int8_t*)p.zp + (int64_t)expert * q.stride_zp_be + (int64_t)ch0 * G : nullptr;
        for (int v = threadIdx.x; v < CHW * per_ch; v += 512) {
            const int ch = v / per_ch, g8 = v % per_ch;
            const v4u a = *(const v4u*)(sg + (int64_t)ch * G + g8 * 8);
            v4u b;
            if (zp_i8) {
                const v2u raw = *(const v2u*)(zg8 + (int64_t)ch * G + g8 * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lo = (float)(int8_t)(raw[i >> 1] >> (16 * (i & 1)));
                    const float hi = (float)(int8_t)(raw[i >> 1] >> (16 * (i & 1) + 8));
                    b[i] = SDT == FNN_F16 ? (f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16))
                                          : (f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16));
                }
            } else {
                b = *(const v4u*)(zg + (int64_t)ch * G + g8 * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                tabs[(g8 * 8 + i) * CHW + ch] = (uint16_t)(a[i >> 1] >> (16 * (i & 1)));
                tabs[(TABG_MAX + g8 * 8 + i) * CHW + ch] = (uint16_t)(b[i >> 1] >> (16 * (i & 1)));
            }
        }
        __syncthreads();
    }
    static_assert(D == 4, "the unrolled loop below walks four weight slots");
    for (int jj = 0; jj < n_iter; jj += D) {
        FNN_PANEL_ITER(0, 0, st0, st3, jj);
        FNN_PANEL_ITER(1, 1, st1, st0, jj + 1);
        FNN_PANEL_ITER(2, 2, st2, st1, jj + 2);
        FNN_PANEL_ITER(3, 3, st3, st2, jj + 3);
    }
#undef FNN_PANEL_ITER

    // ---- per-channel scales: one fold at the end
    if constexpr (REFQ) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < NH; ++h) outv[mb][h] = accg[mb][h];
    } else if constexpr (!G128) {
        float sc[NCL], zc[NCL];
#pragma unroll
        for (int c = 0; c < NCL; ++c) {
            sc[c] = load_as_f32(p.scale, (MOE ? (int64_t)expert * q.stride_scale_be : 0) + n0 + c, p.scale_dtype);
            zc[c] = c_off + (has_zp ? load_zp_f32(p.zp, (MOE ? (int64_t)expert * q.stride_zp_be : 0) + n0 + c, p.zp_dtype)
                                    : 0.f);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int c = NH == 2 ? 2 * r + h : r;
                    outv[mb][h][r] = sc[c] * (accg[mb][h][r] - zc[c] * asum[mb][r]);
                }
    }

    // ---- add the K parts in order (the stages are idle once every copy has landed)
    if constexpr (KS > 1) {
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        float* red = (float*)st0;
        if (ks > 0) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int h = 0; h < NH; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        red[(((((ks - 1) * RT + rt) * MB + mb) * NH + h) * 4 + r) * 64 + lane] = outv[mb][h][r];
        }
        __syncthreads();
        if (ks > 0) return;
#pragma unroll
        for (int k2 = 1; k2 < KS; ++k2)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int h = 0; h < NH; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        outv[mb][h][r] += red[(((((k2 - 1) * RT + rt) * MB + mb) * NH + h) * 4 + r) * 64 + lane];
    }

    // ---- bias, rounding, store: lane (li, lg) holds channels n0 .. n0+NCL-1 of row 16 mb + li
    float bias[NCL];
#pragma unroll
    for (int c = 0; c < NCL; ++c) bias[c] = p.bias ? load_as_f32(p.bias, n0 + c, p.bias_dtype) : 0.f;
    const bool vec_out = (p.ldc * 2) % (NCL * 2) == 0 && ((uintptr_t)p.out % (NCL * 2)) == 0;
    const bool out_f16 = p.out_dtype == FNN_F16;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        int m = m_base + mb * 16 + li;      // output row; for gathered rows the routed-row id
        float wroute = 1.f;
        if constexpr (MOE) {
            m = token_of(mb * 16 + li);
            if (m >= q.num_valid) continue;
            if (q.mul_w) wroute = load_as_f32(q.topk_w, m, q.topk_w_dtype);
        } else {
            if (m >= p.M) continue;
        }
        uint32_t pk[NCL / 2];
#pragma unroll
        for (int c = 0; c < NCL; c += 2) {
            float v0 = NH == 2 ? outv[mb][0][c >> 1] : outv[mb][0][c];
            float v1 = NH == 2 ? outv[mb][1][c >> 1] : outv[mb][0][c + 1];
            if (p.bias) {
                v0 = add_bias<WBITS>(v0, bias[c], p.out_dtype);
                v1 = add_bias<WBITS>(v1, bias[c + 1], p.out_dtype);
            }
            v0 *= wroute;
            v1 *= wroute;
            const uint32_t b0 = out_f16 ? f32_to_f16_bits(v0) : f32_to_bf16_bits(v0);
            const uint32_t b1 = out_f16 ? f32_to_f16_bits(v1) : f32_to_bf16_bits(v1);
            pk[c >> 1] = (b0 & 0xFFFFu) | (b1 << 16);
        }
        uint16_t* dst = (uint16_t*)p.out + (int64_t)m * p.ldc + n0;
        if (vec_out) {
            if constexpr (NH == 2) *(v4u*)dst = v4u{pk[0], pk[1], pk[2], pk[3]};
            else *(v2u*)dst = v2u{pk[0], pk[1]};
        } else {
#pragma unroll
            for (int c = 0; c < NCL; ++c) dst[c] = (uint16_t)(pk[c >> 1] >> (16 * (c & 1)));
        }
    }
}

// Rows per workgroup (64, 32 or 16, as rt = 4, 2, 1) and 16-row activation blocks per pass for M rows: the
// cheapest under a coarse model of the kernel.  A workgroup pays a start-up and wind-down worth about eight
// loop iterations, then ceil(KT * rt / 8) iterations whose cost grows with the row blocks per pass (MFMAs,
// fragment reads, folds: measured 1 : 1.2 : 1.8 for 1, 2, 4 blocks), and the grid runs in rounds of 256
// workgroups, one per CU.  Fewer rows per workgroup make more and shorter workgroups but allow fewer
// activation rows per pass (mb <= rt, the LDS ring's limit), hence more passes over the weights; fewer
// row blocks than the rows would allow make more, cheaper passes (the passes of a tile run on one XCD and
// share the weights through its L2).
// Measured on A16W8, N=4096: M=64 takes 12.6 us with 32 rows per workgroup and two passes, 27.5 us with 16
// rows and four passes, 22.1 us with 64 rows and one pass of 64 workgroups.
// What the model does not see: int8 weights, more than 16 activation rows, and a little more than one or two rounds
// of 64-row workgroups (257 .. 384 or 513 .. 640 of them).  Passes of 32 activation rows with 64-row workgroups, whose
// LDS lets two share a CU, are then faster than one pass of 64 rows with one workgroup per CU, and than 32-row
// workgroups (under a captured graph, rotating weights, bf16 rows, model's choice / 64-row workgroups with 32
// activation rows a pass: N=17792 K=4096 M=64 45.3 / 35.1 us, M=32 36.0 / 27.7; N=22016 K=4096 46.0 / 37.3 and
// 37.2 / 28.2; N=20480 K=8192 80.8 / 70.0 and 58.0 / 51.6; N=37888 K=3584 M=64 65.5 / 58.6; at 432 and 448
// workgroups, N=27648 and 28672, the single pass is ahead by 4 to 8 %, and so it is everywhere with int4 weights, whose
// conversion a second pass repeats).
static int choose_rows(int wrows, int64_t M, int KT, int* mb_out, int wbits) {
    const int need = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    if (wbits == 8 && M > 16 && wrows % 64 == 0) {
        const int wg4 = wrows / 64;
        if ((wg4 > 256 && wg4 <= 384) || (wg4 > 512 && wg4 <= 640)) { *mb_out = 2; return 4; }
    }
    static const double per_iter[5] = {0, 1.0, 1.2, 0, 1.8};
    int rt = 0;
    double best = 0.0;
    for (int cand = 4; cand >= 1; cand >>= 1) {
        if (wrows % (16 * cand) != 0) continue;
        for (int mb = cand < need ? cand : need; mb >= 1; mb >>= 1) {
            const int64_t passes = (M + 16 * mb - 1) / (16 * mb);
            const int64_t wgs = (int64_t)(wrows / (16 * cand)) * passes;
            const int64_t rounds = (wgs + 255) / 256;
            const double cost = (double)rounds * (8.0 + (double)((KT * cand + 7) / 8) * per_iter[mb]);
            if (rt == 0 || cost < best) { best = cost; rt = cand; *mb_out = mb; }
        }
    }
    return rt;
}

// Launches the panel kernel if the shape suits it; returns false otherwise.
template <int WBITS, int ADT>
static bool launch_panel_t(WoArgs& p, hipStream_t st) {
    constexpr int NH = WBITS == 4 ? 2 : 1;
    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    if (wrows % 16 != 0 || p.K % 32 != 0 || p.K < 8 * 128) return false;
    // tables per channel, or per group of 128, 256, 512 .. values
    // (or per group of 64: two groups per slab, K a multiple of 128)
    const bool g64 = p.group == 64 && p.K % 128 == 0;
    const int gs = p.group == 0 || g64 ? 0 : group_shift(p.group);
    if (gs < 0 || (p.group != 0 && p.K % p.group != 0)) return false;
    p.gshift = gs;
    if (p.lda % 8 != 0 || p.ldw % 16 != 0 || ((uintptr_t)p.qw % 16) != 0 || ((uintptr_t)p.act % 16) != 0) return false;
    if (p.group != 0) {
        const bool tables16 = is16(p.scale_dtype) && (!p.zp || p.zp_dtype == p.scale_dtype) &&
                              p.N % (4 * NH) == 0 && ((uintptr_t)p.scale % (8 * NH)) == 0 &&
                              (!p.zp || ((uintptr_t)p.zp % (8 * NH)) == 0);
        if (!tables16) return false;
    }
    int mb = 1;
    int rt = choose_rows(wrows, p.M, (int)((p.K + 127) / 128), &mb, WBITS);
    if (p.force_rt != 0 || p.force_mb != 0) {
        // blocks named by the caller: one of the built pairs, and weight rows that divide into such tiles
        rt = p.force_rt;
        mb = p.force_mb;
        const bool built = (rt == 4 && (mb == 1 || mb == 2 || mb == 4)) || (rt == 2 && (mb == 1 || mb == 2)) || (rt == 1 && mb == 1);
        if (!built || wrows % (16 * rt) != 0) return false;
    }
    const int tiles = wrows / (16 * rt);
    const int passes = (p.M + mb * 16 - 1) / (mb * 16);
    const dim3 grid(((tiles + 7) / 8) * 8 * passes);
    p.m_base = 0;
    // per-channel scales (and zero points) of the activations' 16-bit type: the reference's own per-weight rounding.
    // Not int4 weights under bf16: rounding to bf16 takes about three vector instructions per weight where the plain
    // conversion of a nibble takes 0.75, which cost 13 to 34 % at 1 to 64 rows, for weights of at most 8 scale steps
    // whose rounding moves an output 16 times less than an int8 weight's (int8 under bf16: -8 to +9 %).
    constexpr bool CAN_REFQ = ADT == FNN_F16 || WBITS == 8;
    const bool refq = CAN_REFQ && p.group == 0 && p.scale_dtype == ADT && (!p.zp || p.zp_dtype == ADT);
    note_kernel(refq ? "gemm_wo_panel_kernel(per-weight rounding)" : "gemm_wo_panel_kernel", WBITS, mb, rt);
#define FNN_PANEL3(G, SDTV, MBV, RTV, NTLV)                                                              \
    do {                                                                                                 \
        if constexpr (CAN_REFQ && !G) {                                                                  \
            if (refq) {                                                                                  \
                if (p.zp) gemm_wo_panel_kernel<WBITS, ADT, G, SDTV, MBV, RTV, 4, NTLV, false, 2><<<grid, dim3(512), 0, st>>>(p, passes, MoeArgs{}); \
                else gemm_wo_panel_kernel<WBITS, ADT, G, SDTV, MBV, RTV, 4, NTLV, false, 1><<<grid, dim3(512), 0, st>>>(p, passes, MoeArgs{}); \
                break;                                                                                   \
            }                                                                                            \
        }                                                                                                \
        if constexpr (G) {                                                                               \
            if (g64) {                                                                                   \
                gemm_wo_panel_kernel<WBITS, ADT, G, SDTV, MBV, RTV, 4, NTLV, false, 0, 2><<<grid, dim3(512), 0, st>>>(p, passes, MoeArgs{}); \
                break;                                                                                   \
            }                                                                                            \
        }                                                                                                \
        gemm_wo_panel_kernel<WBITS, ADT, G, SDTV, MBV, RTV, 4, NTLV><<<grid, dim3(512), 0, st>>>(p, passes, MoeArgs{}); \
    } while (0)
#define FNN_PANEL2(G, SDTV, MBV, RTV)                                                                    \
    do {                                                                                                 \
        if (passes == 1) FNN_PANEL3(G, SDTV, MBV, RTV, true);                                            \
        else FNN_PANEL3(G, SDTV, MBV, RTV, false);                                                       \
    } while (0)
#define FNN_PANEL(G, SDTV)                                   \
    do {                                                     \
        if (rt == 4) {                                       \
            if (mb == 1) FNN_PANEL2(G, SDTV, 1, 4);          \
            else if (mb == 2) FNN_PANEL2(G, SDTV, 2, 4);     \
            else FNN_PANEL2(G, SDTV, 4, 4);                  \
        } else if (rt == 2) {                                \
            if (mb == 1) FNN_PANEL2(G, SDTV, 1, 2);          \
            else FNN_PANEL2(G, SDTV, 2, 2);                  \
        } else {                                             \
            FNN_PANEL2(G, SDTV, 1, 1);                       \
        }                                                    \
    } while (0)
    if (p.group != 0) {
        if (p.scale_dtype == FNN_F16) FNN_PANEL(true, FNN_F16);
        else FNN_PANEL(true, FNN_BF16);
    } else {
        FNN_PANEL(false, FNN_F16);
    }
#undef FNN_PANEL
#undef FNN_PANEL2
#undef FNN_PANEL3
    return true;
}

template <int ADT>
static bool launch_panel_moe_t(WoArgs& p, const MoeArgs& q, hipStream_t st) {
    const int wrows = p.N / 2;
    if (p.N % 32 != 0 || p.K % 32 != 0 || p.K < 8 * 128 || (p.group != 0 && p.group != 128) || q.block_m % 16 != 0 ||
        q.EM % q.block_m != 0 || p.lda % 8 != 0 || p.ldw % 16 != 0 || q.stride_be % 16 != 0 ||
        ((uintptr_t)p.act % 16) != 0 || ((uintptr_t)p.qw % 16) != 0)
        return false;
    const int G = p.K / 128;
    if (p.group == 128) {
        // tables [expert][channel][group] of one 16-bit type, every channel's groups contiguous and 16-byte aligned
        const bool ok = p.K % 128 == 0 && G % 8 == 0 && G <= 64 && is16(p.scale_dtype) && q.stride_scale_k == 1 &&
                        q.stride_scale_n == G && q.stride_scale_be % 8 == 0 && ((uintptr_t)p.scale % 16) == 0 &&
                        (!p.zp || ((p.zp_dtype == p.scale_dtype || p.zp_dtype == FNN_I8) && q.stride_zp_k == 1 &&
                                   q.stride_zp_n == G && q.stride_zp_be % 8 == 0 && ((uintptr_t)p.zp % 16) == 0));
        if (!ok) return false;
    } else if (q.stride_scale_n != 1 || (p.zp && q.stride_zp_n != 1)) {
        return false;
    }
    int mb_max = q.block_m % 64 == 0 ? 4 : q.block_m % 32 == 0 ? 2 : 1;   // a pass stays within one expert's block
    int rt = 0;
    double best = 0.0;
    for (int cand = 4; cand >= 1; cand >>= 1) {
        if (wrows % (16 * cand) != 0) continue;
        const int t = wrows / (16 * cand);
        const double fill = (double)t / (((t + 255) / 256) * 256);
        const double score = fill * (cand == 4 ? 1.0 : cand == 2 ? 0.9 : 0.6);
        if (score > best) { best = score; rt = cand; }
    }
    // the transposed tables take LDS from the activation stages
    if (p.group == 128) mb_max = rt == 4 ? (mb_max < 2 ? mb_max : 2) : 1;
    const int mb = mb_max < rt ? mb_max : rt;
    const int tiles = wrows / (16 * rt);
    const int passes = q.EM / (mb * 16);
    const dim3 grid(((tiles + 7) / 8) * 8 * passes);
    p.m_base = 0;
    note_kernel("gemm_wo_panel_kernel(moe)", 4, mb, rt);
#define FNN_MOE2(G, SDTV, MBV, RTV) \
    gemm_wo_panel_kernel<4, ADT, G, SDTV, MBV, RTV, 4, false, true><<<grid, dim3(512), 0, st>>>(p, passes, q)
#define FNN_MOE(G, SDTV)                                   \
    do {                                                   \
        if (rt == 4) {                                     \
            if (mb == 1) FNN_MOE2(G, SDTV, 1, 4);          \
            else if (mb == 2) FNN_MOE2(G, SDTV, 2, 4);     \
            else if constexpr (!G) FNN_MOE2(G, SDTV, 4, 4); \
        } else if (rt == 2) {                              \
            if (mb == 1) FNN_MOE2(G, SDTV, 1, 2);          \
            else if constexpr (!G) FNN_MOE2(G, SDTV, 2, 2); \
        } else {                                           \
            FNN_MOE2(G, SDTV, 1, 1);                       \
        }                                                  \
    } while (0)
    if (p.group == 128) {
        if (p.scale_dtype == FNN_F16) FNN_MOE(true, FNN_F16);
        else FNN_MOE(true, FNN_BF16);
    } else {
        FNN_MOE(false, FNN_F16);
    }
#undef FNN_MOE
#undef FNN_MOE2
    return true;
}

bool launch_wo_panel_moe(WoArgs& p, const MoeArgs& q, int act_dtype, hipStream_t st) {
    return act_dtype == FNN_F16 ? launch_panel_moe_t<FNN_F16>(p, q, st) : launch_panel_moe_t<FNN_BF16>(p, q, st);
}

bool launch_wo_panel(WoArgs& p, int wbits, int act_dtype, hipStream_t st) {
    // the kernel addresses the up to 64 rows of a pass and the 8 weight rows of a load with 32-bit offsets
    // from a 64-bit base: strides that do not fit go to the other kernels
    if (64 * p.lda * 2 >= (1LL << 32) || 8 * p.ldw >= (1LL << 32)) return false;
    if (wbits == 4) return act_dtype == FNN_F16 ? launch_panel_t<4, FNN_F16>(p, st) : launch_panel_t<4, FNN_BF16>(p, st);
    return act_dtype == FNN_F16 ? launch_panel_t<8, FNN_F16>(p, st) : launch_panel_t<8, FNN_BF16>(p, st);
}

}  // namespace fnn
