// A16W4 decode (one activation row) on weights the caller has repacked once, with groups of 128.
//
// The reference layout ([N/2, K] bytes, channel 2j in the low nibble of row j; scales and zero points as
// [K/128, N] tables, flashnn/quant_gemm.py:174-204) makes a decode kernel fetch rows that lie K bytes apart
// and two side tables with a request pattern of their own.  The packed form is one stream: everything a wave
// needs for 16 channels x 1024 values of K - 8 KB of nibbles, then the 8 x 16 scales and the 8 x 16 zero points
// of those groups - is one contiguous unit of 8704 bytes, and a wave reads unit after unit with 16-byte loads.
//
// Packed layout (version 1; N % 16 == 0, K % 1024 == 0, group 128, fp16 tables):
//   unit (tile, kc) at byte ((tile * K/1024) + kc) * 8704, tile = channels 16 tile .. 16 tile + 15,
//   kc = values 1024 kc .. 1024 kc + 1023 of K.
//   bytes [1024 b, 1024 b + 1024), b = 0..7: the group of 128 values k0 = 1024 kc + 128 b.  The 16 bytes at
//     16 * (16 g + c) belong to channel c of the tile: four 32-bit words, word i = the eight values
//     k0 + 32 i + 8 g + (0..7), value j of them in bits 4 * pos(j) .. + 3 with pos(j) = (j >> 1) + 4 * (j & 1).
//     A nibble holds the weight as an unsigned number, reference nibble ^ 8 (the reference's signed value + 8).
//   bytes [8192, 8448): scales as fp16, entry [c][b] (channel c, group b of the unit) at 8192 + 2 * (8 c + b).
//   bytes [8448, 8704): zero points as fp16 in the same order, the caller's values unchanged (zeros if none).
// The byte count equals the reference layout's with fp16 tables: N K / 2 + 2 * (K / 128) * N * 2.
//
// Kernel: a workgroup of 8 waves owns `tpw` neighbouring tiles; wave w takes K range kc = w (mod 8) of each of
// them (fewer ranges than waves: the waves also split the tiles), so its activations - 1024 values - never
// change: they are converted once into a wave-private LDS area.  A word of eight nibbles becomes the eight
// fp16 numbers of one operand of v_mfma_f32_16x16x32_f16 with a shift and four bit-field inserts: a pair of
// nibbles is 1024 + u (bits 0..3) or 1024 + 16 u (bits 4..7) once the exponent bits are set around it, no
// unpacking.  The weights are the operand whose 16 columns are the tile's channels (lane 16 g + c supplies
// channel c, values 8 g .. 8 g + 7 of the instruction's 32); the other operand holds the activations, the
// same in all of its 16 rows, so every row of the result - and every one of a lane's four registers - is
// the channel's sum.  The activations of the pairs that come out as 1024 + 16 u are stored divided by 16.
// What the offset 1024 and the zero point contribute is removed per group from sums of the activations that
// are formed once and kept in scalar registers:
//   sum a u - z sum a  =  dot - 1024 S - (8 + zp) A,   S = sum of the stored activations, A = sum of a.
// Activations are scaled by a power of two per wave (largest magnitude to about 2^13) so that bf16 values
// become fp16 without loss and the division by 16 stays clear of the subnormal range; the partial result is
// scaled back (exactly) before the waves' parts are added in a fixed order.
// The group's scale is applied in fp32 to the group's sum; the reference rounds each dequantised weight to
// fp16 first (quant_gemm.py:20-36).  The difference is far inside rtol = atol = 1e-2.
#include <type_traits>

#include "wo_common.h"

namespace fnn {

constexpr int kPkUnitBytes = 8 * 1024 + 2 * 256;
constexpr int kPkWaves = 8;

typedef const __attribute__((address_space(1))) v4u* gv4u_t;     // a pointer known to be global memory

// the weights are read once: non-temporal loads (plain loads: 24.4 instead of 22.3 us at K = 8192, N = 28672)
#define FNN_PK_LOAD(p) __builtin_nontemporal_load(p)
// units of weights a wave keeps requested ahead of the one it works on (two and three were slower: 23.1, 23.9 us)
constexpr int DEPTH = 1;

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

struct PkArgs {
    const void* act;
    const char* packed;
    const void* bias;
    void* out;
    int M, N, K;
    int64_t lda, ldc;
    int tiles, tpw;
    int out_dtype, bias_dtype;
};

template <int ADT>
__global__ __launch_bounds__(kPkWaves * 64) void gemv_w4_prepacked_kernel(const PkArgs p) {
    constexpr int NW = kPkWaves;
    constexpr int WAVE_BYTES = 2048;                          // 1024 activations as fp16
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int KC = p.K >> 10;
    const int KCW = KC < NW ? KC : NW;      // waves that share a tile (KC is 1, 2, 4 or at least 8: host-checked)
    const int TS = NW / KCW;                // sets of tiles the waves split
    const int sub = wave / KCW;
    const int tile0 = blockIdx.x * p.tpw;
    const int ntile = min(p.tpw, p.tiles - tile0);
    const int nu = sub < ntile ? (ntile - sub + TS - 1) / TS : 0;     // tiles (units per K range) of this wave

    char* const my_act = smem + wave * WAVE_BYTES;
    float* const parts = (float*)(smem + NW * WAVE_BYTES);            // [tile][wave][16]

    bool first_range = true;
    for (int kc = wave % KCW; kc < KC; kc += KCW) {
        // ---- this K range of the activation row, once: lane l holds values 16 l .. 16 l + 15
        const char* const src = (const char*)p.act + (int64_t)kc * 2048 + lane * 32;
        const v4u a_lo = *(gv4u_t)src;
        const v4u a_hi = *(gv4u_t)(src + 16);
        // unit j of this wave: a scalar address (the lanes add 16 bytes each)
        const char* const units = p.packed + (((int64_t)tile0 + sub) * KC + kc) * kPkUnitBytes;
        const int64_t unit_step = (int64_t)KC * kPkUnitBytes * TS;
        auto unit_ptr = [&](int j) -> const char* {
            const uint64_t v = (uint64_t)units + (uint64_t)(j * unit_step);
            const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
            const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
            return (const char*)(((uint64_t)hi << 32) | lo);
        };
        const uint32_t w_off = lane * 16, t_off = 8192 + c * 16;
        v4u wq[DEPTH][8], sr[DEPTH], zr[DEPTH];
        // (a unit that does not exist is replaced by 16 bytes of the wave's first unit: every wave then has
        // the same number of loads in flight at every point, and the waits the compiler places count only
        // the loads that have to be back)
        auto load_unit = [&](int j, auto bank) __attribute__((always_inline)) {
            constexpr int B = decltype(bank)::value;
            const bool have = j < nu;
            const char* const u = have ? unit_ptr(j) : unit_ptr(0);
            const uint32_t stride = have ? 1024u : 0u, w_at = have ? w_off : 0u, t_at = have ? t_off : 0u;
#pragma unroll
            for (int b = 0; b < 8; ++b) wq[B][b] = FNN_PK_LOAD((gv4u_t)(u + b * stride + w_at));
            sr[B] = *(gv4u_t)(u + t_at);
            zr[B] = *(gv4u_t)(u + 256 + t_at);
        };
        // the activations are asked for first (loads return in order, and they are needed first), then DEPTH
        // units of weights: eight 16-byte loads per lane and unit, in flight from here to the end
        __builtin_amdgcn_sched_barrier(0);
        static_for<DEPTH>([&](auto d) __attribute__((always_inline)) { load_unit(decltype(d)::value, d); });
        __builtin_amdgcn_sched_barrier(0);

        float v[16];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[e] = bits_to_f32<ADT>((a_lo[e >> 1] >> (16 * (e & 1))) & 0xFFFFu);
            v[8 + e] = bits_to_f32<ADT>((a_hi[e >> 1] >> (16 * (e & 1))) & 0xFFFFu);
        }
        float mx = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, fabsf(v[e]));
        mx = wave_max(mx);
        // 2^sh brings the largest magnitude to [2^13, 2^14); nothing to scale in an all-zero or non-finite range
        const int ex = (int)((__float_as_uint(mx) >> 23) & 0xFF);
        const int sh = (ex == 0 || ex == 255) ? 0 : max(-100, min(100, 13 - (ex - 127)));
        const float up = __uint_as_float((uint32_t)(127 + sh) << 23);
        const float unscale = __uint_as_float((uint32_t)(127 - sh) << 23);
        // stored pairs: even pairs as they are, odd pairs divided by 16; S = sum of what is stored,
        // A = sum of what the stored values stand for (stored, or 16 x stored)
        uint32_t st[8];
        float S = 0.f, A = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float f = (j & 1) ? up * 0.0625f : up;
            const v2h h = __builtin_convertvector(v2f{v[2 * j] * f, v[2 * j + 1] * f}, v2h);
            st[j] = __builtin_bit_cast(uint32_t, h);
            const float s2 = (float)h[0] + (float)h[1];
            S += s2;
            A += (j & 1) ? 16.f * s2 : s2;
        }
        *(v4u*)(my_act + lane * 32) = v4u{st[0], st[1], st[2], st[3]};
        *(v4u*)(my_act + lane * 32 + 16) = v4u{st[4], st[5], st[6], st[7]};
        // a group of 128 values is eight neighbouring lanes; its two sums go to scalar registers
#pragma unroll
        for (int o = 1; o < 8; o <<= 1) {
            S += __shfl_xor(S, o, 64);
            A += __shfl_xor(A, o, 64);
        }
        float grp_c[8], grp_a[8];       // per group: -1024 S, and A
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            grp_c[b] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(-1024.f * S), 8 * b));
            grp_a[b] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(A), 8 * b));
        }
        // The 32 activation operands of this lane (8 groups x 4 instructions; they depend on g alone) are
        // read back once and stay in registers over all tiles: no LDS traffic inside the stream.  (LDS
        // operations of one wave complete in order: the reads see what was written above.)
        v4u areg[8][4];
#pragma unroll
        for (int b = 0; b < 8; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) areg[b][i] = *(const v4u*)(my_act + b * 256 + i * 64 + g * 16);

        // the fp16 pair (1024, 1024), kept in a register the compiler cannot see through: (w & m) | (k & ~m)
        // is then one bit-field insert instead of an and and an or with a literal each
        uint32_t k1024 = 0x64006400u;
        asm volatile("" : "+v"(k1024));
        // one unit.  As a block's registers become free they take the same block of the unit DEPTH further
        // on.  The last DEPTH units have no such successor: their loads all fetch, in every lane, the first 16
        // bytes of the unit itself (one cache hit per load where a real one moves a kilobyte; all waves
        // aiming at one address, or whole kilobytes of dummy traffic, cost 1 to 3 us) - one straight piece of
        // code for every unit, where a branch around the loads would let the compiler gather them at the top.
        auto process = [&](int j, auto bank) __attribute__((always_inline)) {
            constexpr int B = decltype(bank)::value;
            const bool more = j + DEPTH < nu;
            const char* const next = more ? unit_ptr(j + DEPTH) : unit_ptr(j);
            const uint32_t stride = more ? 1024u : 0u, w_at = more ? w_off : 0u, t_at = more ? t_off : 0u;
            const v4u sraw = sr[B], zraw = zr[B];
            float acc = 0.f;
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                const v4u w = wq[B][b];
                wq[B][b] = FNN_PK_LOAD((gv4u_t)(next + b * stride + w_at));
                v4f d = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t wi = w[i], w8 = wi >> 8;
                    const v4u x = v4u{(wi & 0x000F000Fu) | (k1024 & ~0x000F000Fu), (wi & 0x00F000F0u) | (k1024 & ~0x00F000F0u),
                                      (w8 & 0x000F000Fu) | (k1024 & ~0x000F000Fu), (w8 & 0x00F000F0u) | (k1024 & ~0x00F000F0u)};
                    d = MfmaT<FNN_F16>::mma(areg[b][i], x, d);
                }
                const float sb = f16_bits_to_f32((sraw[b >> 1] >> (16 * (b & 1))) & 0xFFFFu);
                const float z8 = 8.f + f16_bits_to_f32((zraw[b >> 1] >> (16 * (b & 1))) & 0xFFFFu);
                float t = d[0] + grp_c[b];
                t = __builtin_fmaf(-z8, grp_a[b], t);
                acc = __builtin_fmaf(sb, t, acc);
                __builtin_amdgcn_sched_barrier(0);      // keep each refill load inside its step
            }
            sr[B] = *(gv4u_t)(next + t_at);
            zr[B] = *(gv4u_t)(next + 256 + t_at);
            const int t_local = sub + j * TS;
            const float r = acc * unscale;
            if (lane < 16) {
                float* dst = parts + (t_local * NW + wave) * 16 + c;
                *dst = first_range ? r : *dst + r;
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        for (int j = 0; j < nu; j += DEPTH)
            static_for<DEPTH>([&](auto d) __attribute__((always_inline)) {
                if (j + decltype(d)::value < nu) process(j + decltype(d)::value, d);
            });
        first_range = false;
    }
    __syncthreads();
    // ---- the parts of a tile, in ascending wave order, plus the bias
    for (int idx = threadIdx.x; idx < ntile * 16; idx += NW * 64) {
        const int t = idx >> 4, ch = idx & 15;
        float v = 0.f;
        for (int w = (t % TS) * KCW; w < (t % TS + 1) * KCW; ++w) v += parts[(t * NW + w) * 16 + ch];
        const int n = (tile0 + t) * 16 + ch;
        if (p.bias) v += load_as_f32(p.bias, n, p.bias_dtype);
        store_from_f32(p.out, n, v, p.out_dtype);
    }
}

// ---- 2 .. 64 activation rows per pass on the packed form ---------------------------------------------------
// A workgroup of NW waves (8, or 4 for 64 rows) owns up to T neighbouring tiles and walks K in ranges of
// 128 NW values; in a range wave w takes the group of 128 values that is the kilobyte at 1024 (w + NW sub) of
// every tile's unit, so the waves read a unit's nibbles as one contiguous piece, and what a wave needs of the
// activations for a range - its 128 values of up to 64 rows, already in operand order - serves all tiles of
// the workgroup.  Those rows arrive by 16-byte direct-to-LDS copies, whole 128-byte lines per instruction, into
// a wave-private area one range ahead (fragment (mb, i) of lane (c, g): row 16 mb + c, values 32 i + 8 g .. + 7
// of the group); the weights and table entries of (tile, range + PD) are requested as those of
// (tile, range) are consumed, and the main loop has no barrier.  The integer weights go into the MFMAs as
// OFF + u (exponent trick, OFF = 1024 for fp16 and 128 for bf16 activations, u the nibble as an unsigned
// number); per group
//   out += s * (dot - (OFF + 8 + zp) * sum_k a_k),
// in fp32, the activation sums coming from MFMAs against ones once per range and wave.  The partial sums of
// the waves meet in LDS and are added in ascending wave order, then bias, rounding, store.
// 64 rows take four waves: 7 x 4 x 4 output registers per lane, the fragments of 64 rows and two ranges of
// weights in flight need more than the 256 registers a wave of an 8-wave workgroup can have.
constexpr int kPkRowTiles = 7;       // most tiles per workgroup

typedef __attribute__((address_space(3))) void* pk_lds_ptr_t;
typedef const __attribute__((address_space(1))) void* pk_gbl_ptr_t;

// A word of eight nibbles -> the eight numbers OFF + u of one MFMA operand: the nibble pair (j, j + 4) of the
// word, shifted to bits 0..3 and 16..19, set into the exponent pattern.  `k` holds that pattern in a register
// the compiler cannot see through, so that (w & m) | (k & ~m) is one bit-field insert (an and-or of a
// register with two constants takes two instructions on this ISA).
__device__ __forceinline__ v4u pk_operand(const uint32_t w, const uint32_t k) {
    constexpr uint32_t m = 0x000F000Fu;
    const uint32_t w1 = w >> 4, w2 = w >> 8, w3 = w >> 12;
    return v4u{(w & m) | (k & ~m), (w1 & m) | (k & ~m), (w2 & m) | (k & ~m), (w3 & m) | (k & ~m)};
}

constexpr int pk_rows_lds_bytes(int MB, int NW, int T) { return NW * MB * (T > 4 ? T : 4) * 1024; }

template <int ADT, int MB, int NW, int T, int PD, bool NT>
__global__ __launch_bounds__(NW * 64) void gemm_w4_prepacked_rows_kernel(const PkArgs p) {
    typedef MfmaT<ADT> MT;
    constexpr int SUB = 8 / NW;                 // ranges per unit
    constexpr int FR = 4 * MB;                  // activation fragments per range and wave
    constexpr int WAVE_LDS = FR * 1024;
    constexpr int LPS = 2 * T;                  // register loads per range and wave
    constexpr float OFF8 = (ADT == FNN_F16 ? 1024.f : 128.f) + 8.f;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int KC = p.K >> 10;
    const int NR = KC * SUB;                    // ranges
    const int tile0 = blockIdx.x * p.tpw;
    const int ntile = min(p.tpw, p.tiles - tile0);
    const int m0 = blockIdx.y * (MB * 16);

    // ---- activations: rows beyond M repeat the last row (their results are not stored)
    char* const mine = smem + wave * WAVE_LDS;
    const char* const abase = (const char*)p.act + (int64_t)m0 * p.lda * 2 + wave * 256;
    // Copy j of a range brings rows 4 j .. 4 j + 3, each row's 256 bytes of the wave's group as two whole
    // 128-byte lines: lane 16 q + ch asks for 16-byte chunk ch ^ (row & 15) of row 4 j + q, which lands in slot
    // ch of that row (the area is [row][slot], 256 bytes a row), so that the 16 lanes which later read the same
    // chunk of 16 different rows find it in 16 different slots.
    uint32_t aoff[FR];
#pragma unroll
    for (int j = 0; j < FR; ++j) {
        const int row = 4 * j + (lane >> 4);
        aoff[j] = (uint32_t)min(row, p.M - 1 - m0) * (uint32_t)(p.lda * 2) + (((lane & 15) ^ (row & 15)) << 4);
    }
    auto copy_act = [&](int r) __attribute__((always_inline)) {
        const char* const src = abase + (int64_t)r * (NW * 256);
#pragma unroll
        for (int j = 0; j < FR; ++j)
            __builtin_amdgcn_global_load_lds((pk_gbl_ptr_t)(src + aoff[j]), (pk_lds_ptr_t)(mine + j * 1024), 16, 0, 0);
    };

    // ---- weights and tables: tile t of the workgroup, range r.  A tile the workgroup does not have, and a
    // range behind the last one, are replaced by 16 bytes (4 for the tables) of a unit that exists, the same
    // for all lanes: every wave then has the same loads in flight at every point of the loop.  One table load
    // serves both tables: the lanes of even g ask for the scale of channel c, those of odd g for its zero point
    // (the aligned 32-bit word that holds the 16-bit entry; the half is taken where it is used).
    const char* const units = p.packed + (int64_t)tile0 * KC * kPkUnitBytes;
    const uint32_t w_lane = wave * 1024 + lane * 16, t_lane = 8192 + 256 * (g & 1) + 2 * (8 * c + (wave & ~1));
    const uint32_t t_shift = 16 * (wave & 1);
    v4u wq[PD][T];
    uint32_t tq[PD][T];
    auto unit_of = [&](int t, int r) -> const char* {
        const int rr = r < NR ? r : NR - 1;
        return units + ((int64_t)(t < ntile ? t : 0) * KC + rr / SUB) * kPkUnitBytes + (rr % SUB) * (NW * 1024);
    };
    auto load_w = [&](auto slot, int t, int r) __attribute__((always_inline)) {
        const v4u* const wp = (const v4u*)(unit_of(t, r) + (t < ntile && r < NR ? w_lane : 0u));
        wq[decltype(slot)::value][t] = NT ? __builtin_nontemporal_load(wp) : *wp;
    };
    auto load_t = [&](auto slot, int t, int r) __attribute__((always_inline)) {
        const bool have = t < ntile && r < NR;
        const int sub = (r < NR ? r : NR - 1) % SUB;
        // (the tables lie behind the unit's eight kilobytes of nibbles, not behind this range's)
        tq[decltype(slot)::value][t] =
            *(const uint32_t*)(unit_of(t, r) - sub * (NW * 1024) + (have ? t_lane + sub * NW * 2 : 8192u));
    };
    // Every wait for a load is written out.  (As long as direct-to-LDS copies are in flight the compiler
    // answers a register whose load it cannot place behind one of these waits with a wait for everything.)
    // A tile's weights and, one load later, the table entries of the tile before it were asked for PD ranges
    // ago; behind them came the rest of that range's loads, PD - 1 whole ranges, PD sets of copies and this
    // range's loads so far: 2 PD T - 2 + PD FR loads in all, whatever the tile.
    constexpr int NTILE_WAIT = (PD * T - 1) * 2 + PD * FR;
    static_assert(NTILE_WAIT < 64 && LPS < 64, "vmcnt range");
    auto wait_tile = [&]() __attribute__((always_inline)) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (NTILE_WAIT & 15) | ((NTILE_WAIT >> 4) << 14));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);       // nothing that reads the loaded registers moves above the wait
    };

    v4f out[T][MB];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) out[t][mb] = v4f{0.f, 0.f, 0.f, 0.f};
    const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
    uint32_t kexp = ADT == FNN_F16 ? 0x64006400u : 0x43004300u;       // OFF in both halves
    asm volatile("" : "+v"(kexp));

    // issue order: the older ranges' weights, the first range's activations, the newest range's weights
    __builtin_amdgcn_sched_barrier(0);
    static_for<PD - 1>([&](auto d) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < T; ++t) { load_w(d, t, decltype(d)::value); load_t(d, t, decltype(d)::value); }
    });
    __builtin_amdgcn_sched_barrier(0);
    copy_act(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < T; ++t) {
        load_w(std::integral_constant<int, PD - 1>{}, t, PD - 1);
        load_t(std::integral_constant<int, PD - 1>{}, t, PD - 1);
    }
    __builtin_amdgcn_sched_barrier(0);

    auto range = [&](int r, auto slot, auto tail) __attribute__((always_inline)) {
        constexpr int S = decltype(slot)::value;
        constexpr bool TAIL = decltype(tail)::value;
        // the copies of this range were issued before the LPS loads that followed them: they have landed
        // once at most LPS loads are outstanding.  The ranges behind the loop ask for nothing further (the
        // compiler would drop loads nobody uses, and the count with them) and wait for everything instead.
        constexpr int TOP_WAIT = TAIL ? 0 : LPS;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (TOP_WAIT & 15) | ((TOP_WAIT >> 4) << 14));
        asm volatile("" ::: "memory");
        v4u a[MB][4];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) a[mb][i] = *(const v4u*)(mine + (16 * mb + c) * 256 + (((4 * i + g) ^ c) << 4));
        // the reads are back before the next range's copies may overwrite the area
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        copy_act(r + 1 < NR ? r + 1 : r);          // (behind the last range: once more the same, unused)
        __builtin_amdgcn_sched_barrier(0);

        v4f asum[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) asum[mb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) asum[mb] = MT::mma(a[mb][i], ones, asum[mb]);

        // A tile in two halves, the second one tile behind the first, in one stretch of code, so that the
        // compiler can place the vector instructions of a fold between the MFMAs of the next tile (a wave
        // issues in order: what shall run under an MFMA has to stand behind it): (A) convert the tile's nibbles
        // and issue its MFMAs into one of two accumulator sets; (B) scale and zero point of the tile before,
        // fold.  Then the loads, in a fixed order: this tile's weights and the previous tile's table entries
        // PD ranges on.  One wait at the top covers the weights and, one load younger, the table entries.
        // (A tile the workgroup does not have is worked on all the same, on the bytes its loads fetched:
        // straight code, and nothing of it is stored.)
        v4f d[2][MB];
        static_for<T + 1>([&](auto tt) __attribute__((always_inline)) {
            constexpr int t = decltype(tt)::value;
            constexpr int tp = t > 0 ? t - 1 : 0;     // the tile whose fold runs here
            wait_tile();
            if constexpr (t < T) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) d[t & 1][mb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const v4u x = pk_operand(wq[S][t < T ? t : 0][i], kexp);
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) d[t & 1][mb] = MT::mma(a[mb][i], x, d[t & 1][mb]);
                }
            }
            if constexpr (t > 0) {
                const v2u sz = __builtin_amdgcn_permlane16_swap(tq[S][tp], tq[S][tp], false, false);
                const float s32 = f16_bits_to_f32(sz[0] >> t_shift);
                const float cz = OFF8 + f16_bits_to_f32(sz[1] >> t_shift);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        out[tp][mb][q] = __builtin_fmaf(s32, __builtin_fmaf(-cz, asum[mb][q], d[tp & 1][mb][q]), out[tp][mb][q]);
            }
            // (arithmetic may move across these; loads stay in their order)
            __builtin_amdgcn_sched_barrier(0xF);
            if constexpr (!TAIL && t < T) load_w(slot, t < T ? t : 0, r + PD);
            __builtin_amdgcn_sched_barrier(0xF);
            if constexpr (!TAIL && t > 0) load_t(slot, tp, r + PD);
            __builtin_amdgcn_sched_barrier(0xF);
        });
    };
    // whole rounds of PD ranges, then the ranges left over (the same code with the slots named at compile time)
    int r = 0;
    for (; r + PD <= NR; r += PD)
        static_for<PD>([&](auto d) __attribute__((always_inline)) { range(r + decltype(d)::value, d, std::false_type{}); });
    static_for<PD - 1>([&](auto d) __attribute__((always_inline)) {
        if (r + decltype(d)::value < NR) range(r + decltype(d)::value, d, std::true_type{});
    });

    // ---- the waves' parts, [wave][tile][mb][lane] as float4, added in wave order
    __syncthreads();
    v4f* const parts = (v4f*)smem;
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) parts[((wave * T + t) * MB + mb) * 64 + lane] = out[t][mb];
    __syncthreads();
    for (int idx = threadIdx.x; idx < ntile * MB * 64; idx += NW * 64) {
        const int t = idx / (MB * 64), rem = idx - t * (MB * 64);
        const int mb = rem >> 6, ln = rem & 63;
        v4f v = parts[(t * MB + mb) * 64 + ln];
#pragma unroll
        for (int w = 1; w < NW; ++w) v += parts[((w * T + t) * MB + mb) * 64 + ln];
        const int n = (tile0 + t) * 16 + (ln & 15);
        const float bias = p.bias ? load_as_f32(p.bias, n, p.bias_dtype) : 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int m = m0 + 16 * mb + 4 * (ln >> 4) + q;
            if (m < p.M) store_from_f32(p.out, (int64_t)m * p.ldc + n, v[q] + bias, p.out_dtype);
        }
    }
}

// ---- the repacking: one thread per 32-bit word of the packed form
__global__ __launch_bounds__(256) void prepack_w4_kernel(uint32_t* dst, const uint8_t* qw, const uint16_t* scale,
                                                         const uint16_t* zp, int N, int K, int64_t ldw, int64_t words) {
    constexpr int UNIT_WORDS = kPkUnitBytes / 4;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= words) return;
    const int KC = K >> 10;
    const int64_t u = idx / UNIT_WORDS;
    const int r = (int)(idx - u * UNIT_WORDS);
    const int tile = (int)(u / KC), kc = (int)(u - (int64_t)tile * KC);
    uint32_t word = 0;
    if (r < 2048) {
        const int b = r >> 8, l = (r >> 2) & 63, i = r & 3;
        const int ch = tile * 16 + (l & 15);
        const int k0 = kc * 1024 + b * 128 + i * 32 + (l >> 4) * 8;
        const uint8_t* src = qw + (int64_t)(ch >> 1) * ldw + k0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t nib = ((uint32_t)src[j] >> (4 * (ch & 1))) & 0xFu;
            word |= (nib ^ 8u) << (4 * ((j >> 1) + 4 * (j & 1)));
        }
    } else {
        const int r2 = r - 2048;                       // 64 words of scales, then 64 of zero points
        const uint16_t* tab = r2 < 64 ? scale : zp;
        if (tab) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int e = 2 * (r2 & 63) + h;       // entry [c][b]
                const int ch = tile * 16 + (e >> 3), g = kc * 8 + (e & 7);
                word |= (uint32_t)tab[(int64_t)g * N + ch] << (16 * h);
            }
        }
    }
    dst[idx] = word;
}

static bool pk_shape_ok(int64_t N, int64_t K, int64_t group) {
    if (group != 128 || N <= 0 || K <= 0 || N % 16 != 0 || K % 1024 != 0) return false;
    const int64_t KC = K / 1024;
    return KC >= 8 || KC == 4 || KC == 2 || KC == 1;
}

template <int ADT>
static void launch_pk(PkArgs& p, hipStream_t st) {
    const size_t lds = (size_t)kPkWaves * 2048 + (size_t)p.tpw * kPkWaves * 16 * sizeof(float);
    auto kfn = gemv_w4_prepacked_kernel<ADT>;
    static std::atomic<uint64_t> raised{0};
    allow_large_lds((const void*)kfn, raised);
    note_kernel("gemv_w4_prepacked_kernel", p.tpw);
    kfn<<<dim3((p.tiles + p.tpw - 1) / p.tpw), dim3(kPkWaves * 64), lds, st>>>(p);
}

template <int ADT, int MB, int NW, int T, int PD, bool NT>
static void launch_pk_rows_t(const PkArgs& p, int passes, hipStream_t st) {
    auto kfn = gemm_w4_prepacked_rows_kernel<ADT, MB, NW, T, PD, NT>;
    static std::atomic<uint64_t> raised{0};
    allow_large_lds((const void*)kfn, raised);
    note_kernel("gemm_w4_prepacked_rows_kernel", MB, T, passes);
    kfn<<<dim3((p.tiles + p.tpw - 1) / p.tpw, passes), dim3(NW * 64), (size_t)pk_rows_lds_bytes(MB, NW, T), st>>>(p);
}

// 2 or more rows: passes of 16, 32 or 64 rows; a single pass reads the weights with non-temporal loads.
// As many tiles per workgroup as give every CU one workgroup, at most kPkRowTiles; the kernel is built for 1, 2, 4
// or 7 and keeps the more ranges in flight the fewer tiles a range has.  Up to 32 rows: 8 waves; more: 4 waves
// (about 300 registers per lane).
template <int ADT>
static void launch_pk_rows(PkArgs& p, hipStream_t st) {
    const int tpw = (p.tiles + 255) / 256;
    p.tpw = tpw > kPkRowTiles ? kPkRowTiles : tpw;
    const int passes = (p.M + 63) / 64;
#define FNN_PK_ROWS(T, PD1, PD2, PD4)                                                \
    do {                                                                            \
        if (p.M <= 16) launch_pk_rows_t<ADT, 1, 8, T, PD1, true>(p, 1, st);          \
        else if (p.M <= 32) launch_pk_rows_t<ADT, 2, 8, T, PD2, true>(p, 1, st);     \
        else if (passes == 1) launch_pk_rows_t<ADT, 4, 4, T, PD4, true>(p, 1, st);   \
        else launch_pk_rows_t<ADT, 4, 4, T, PD4, false>(p, passes, st);              \
    } while (0)
    if (p.tpw == 1) FNN_PK_ROWS(1, 8, 4, 3);
    else if (p.tpw == 2) FNN_PK_ROWS(2, 6, 3, 3);
    else if (p.tpw <= 4) FNN_PK_ROWS(4, 4, 2, 2);
    else FNN_PK_ROWS(7, 2, 2, 2);
#undef FNN_PK_ROWS
}

}  // namespace fnn

using namespace fnn;

extern "C" size_t fnn_a16w4_prepacked_bytes(int64_t N, int64_t K, int64_t group) {
    if (!pk_shape_ok(N, K, group) || N > (1 << 30) || K > (1 << 30)) return 0;
    return (size_t)(N / 16) * (size_t)(K / 1024) * kPkUnitBytes;
}

extern "C" int fnn_a16w4_prepack(void* packed, const void* qw, const void* scale, const void* zp, int64_t N, int64_t K,
                                 int64_t ldw, int64_t group, int scale_dtype, int zp_dtype, void* stream) {
    const char* fn = "fnn_a16w4_prepack";
    if (!packed || !qw || !scale) { set_error("%s: null pointer argument", fn); return FNN_ERR_ARG; }
    if (N <= 0 || K <= 0 || ldw < K || N > (1 << 30) || K > (1 << 30)) {
        set_error("%s: bad shape N=%lld K=%lld ldw=%lld", fn, (long long)N, (long long)K, (long long)ldw);
        return FNN_ERR_ARG;
    }
    if (!pk_shape_ok(N, K, group)) {
        set_error("%s: the packed form needs N %% 16 == 0, K %% 1024 == 0 with K / 1024 in {1, 2, 4} or >= 8, and groups "
                  "of 128 (N=%lld K=%lld group=%lld)", fn, (long long)N, (long long)K, (long long)group);
        return FNN_ERR_UNSUPPORTED;
    }
    if (scale_dtype != FNN_F16 || (zp && zp_dtype != FNN_F16)) {
        set_error("%s: the packed form holds fp16 scales and zero points", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (((uintptr_t)packed % 16) != 0) { set_error("%s: the packed buffer must be 16-byte aligned", fn); return FNN_ERR_ARG; }
    const int64_t words = (int64_t)(fnn_a16w4_prepacked_bytes(N, K, group) / 4);
    const Call call(fn);
    note_kernel("prepack_w4_kernel");
    prepack_w4_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
        (uint32_t*)packed, (const uint8_t*)qw, (const uint16_t*)scale, (const uint16_t*)zp, (int)N, (int)K, ldw, words);
    return call.done();
}

extern "C" int fnn_gemm_a16w4_prepacked(void* out, const void* act, const void* packed, const void* bias, int64_t M,
                                        int64_t N, int64_t K, int64_t lda, int64_t ldc, int64_t group, int act_dtype,
                                        int out_dtype, int bias_dtype, void* stream) {
    const char* fn = "fnn_gemm_a16w4_prepacked";
    if (M != 0 && N != 0 && (!out || !act || !packed)) { set_error("%s: null pointer argument", fn); return FNN_ERR_ARG; }
    if (M < 0 || N < 0 || K <= 0 || lda < K || ldc < N) {
        set_error("%s: bad shape M=%lld N=%lld K=%lld lda=%lld ldc=%lld", fn, (long long)M, (long long)N, (long long)K,
                  (long long)lda, (long long)ldc);
        return FNN_ERR_ARG;
    }
    if (M == 0 || N == 0) return FNN_OK;
    if (!pk_shape_ok(N, K, group) || N > (1 << 30) || K > (1 << 30)) {
        set_error("%s: no packed form for N=%lld K=%lld group=%lld", fn, (long long)N, (long long)K, (long long)group);
        return FNN_ERR_UNSUPPORTED;
    }
    if (M > 1 && (64 * lda * 2 >= (1LL << 32) || (M + 63) / 64 > 65535)) {
        set_error("%s: M=%lld rows of stride %lld are beyond what the kernel addresses", fn, (long long)M, (long long)lda);
        return FNN_ERR_UNSUPPORTED;
    }
    if (!is16(act_dtype) || !is16(out_dtype) || (bias && !isflt(bias_dtype))) {
        set_error("%s: activations and output must be fp16 or bf16, the bias fp16, bf16 or fp32", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (((uintptr_t)packed % 16) != 0 || ((uintptr_t)act % 16) != 0 || (M > 1 && lda % 8 != 0)) {
        set_error("%s: the packed weights and the activation rows must be 16-byte aligned", fn);
        return FNN_ERR_ARG;
    }
    PkArgs p{};
    p.act = act; p.packed = (const char*)packed; p.bias = bias; p.out = out;
    p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldc = ldc;
    p.out_dtype = out_dtype; p.bias_dtype = bias_dtype;
    p.tiles = (int)(N / 16);
    // one workgroup per CU where the tiles allow it; a workgroup's parts must fit the LDS beside the activations
    int tpw = (p.tiles + 255) / 256;
    if (tpw > 128) tpw = 128;
    p.tpw = tpw;
    const Call call(fn);
    const hipStream_t st = (hipStream_t)stream;
    if (M > 1) {
        if (act_dtype == FNN_F16) launch_pk_rows<FNN_F16>(p, st);
        else launch_pk_rows<FNN_BF16>(p, st);
    } else if (act_dtype == FNN_F16) {
        launch_pk<FNN_F16>(p, st);
    } else {
        launch_pk<FNN_BF16>(p, st);
    }
    return call.done();
}
