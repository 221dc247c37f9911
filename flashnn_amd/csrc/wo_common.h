// Pieces shared by the weight-only GEMM kernels: the argument block, the MFMA wrappers and the
// integer -> fp16/bf16 conversions that run on exponent tricks.
#pragma once

#include "fnn_common.h"
#include "moe_common.h"

namespace fnn {

struct WoArgs {
    const void* act;
    const int8_t* qw;
    const void* scale;
    const void* zp;
    const void* bias;
    void* out;
    int M, N, K;          // N = output channels
    int64_t lda, ldw, ldc;
    int group;            // 0 = per channel
    int gshift;           // groups of 128 << gshift values (the panel and tiled kernels: table row of slab j is j >> gshift)
    int out_dtype, scale_dtype, zp_dtype, bias_dtype;
    int m_base;           // first activation row handled by this launch
    void* cvt_ws;         // scratch for bf16 activations converted to fp16 (NULL: none), cvt_ws_bytes of it
    size_t cvt_ws_bytes;
    const float* act_unscale;   // per activation row: what the output is multiplied by (NULL: nothing); set where
                                // the rows were scaled by a power of two on their way from bf16 to fp16
    int force_rt, force_mb;     // the panel kernel's blocks named by the caller: 16 force_rt weight rows per workgroup,
                                // 16 force_mb activation rows per pass (0: the launcher chooses)
};

// s if group == 128 << s (the group sizes whose tables the 128-value slabs of the panel and tiled kernels can
// walk: a slab lies within one group), else -1
inline int group_shift(int group) {
    for (int s = 0; s < 16; ++s)
        if (group == (128 << s)) return s;
    return -1;
}

constexpr int kWoWaves = 8;
constexpr int kPF = 8;    // weight loads in flight per lane
constexpr int kPFA = 2;   // activation steps in flight per lane

template <int ADT> struct MfmaT;
template <> struct MfmaT<FNN_F16> {
    typedef v8h vec;
    static constexpr uint32_t one2 = 0x3C003C00u;
    __device__ static __forceinline__ v4f mma(v4u a, v4u b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a),
                                                      __builtin_bit_cast(v8h, b), c, 0, 0, 0);
    }
};
template <> struct MfmaT<FNN_BF16> {
    typedef v8bf vec;
    static constexpr uint32_t one2 = 0x3F803F80u;
    __device__ static __forceinline__ v4f mma(v4u a, v4u b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a),
                                                       __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    }
};

// 16 int8 (k .. k+15 of one row) -> two MFMA operands in natural k order.
// Values come out as c + (v + 128) with c = 1024 (fp16) or 0 (bf16).
template <int ADT>
__device__ __forceinline__ void convert_w8(const v4u w, v4u& s0, v4u& s1) {
    uint32_t o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t x = w[q] ^ 0x80808080u;
        if constexpr (ADT == FNN_F16) {
            o[2 * q] = __builtin_amdgcn_perm(x, 0x64646464u, 0x00050004u);
            o[2 * q + 1] = __builtin_amdgcn_perm(x, 0x64646464u, 0x00070006u);
        } else {
            const uint32_t f0 = __float_as_uint((float)(x & 0xFFu));
            const uint32_t f1 = __float_as_uint((float)((x >> 8) & 0xFFu));
            const uint32_t f2 = __float_as_uint((float)((x >> 16) & 0xFFu));
            const uint32_t f3 = __float_as_uint((float)(x >> 24));
            o[2 * q] = __builtin_amdgcn_perm(f1, f0, 0x07060302u);
            o[2 * q + 1] = __builtin_amdgcn_perm(f3, f2, 0x07060302u);
        }
    }
    s0 = v4u{o[0], o[1], o[2], o[3]};
    s1 = v4u{o[4], o[5], o[6], o[7]};
}

// 16 bytes = 16 k of two channels (low nibble: even channel).  Each operand holds k in the
// order (0,2)(1,3)(4,6)(5,7); values are c + (v + 8), c = 1024 (fp16) / 128 (bf16).
template <int ADT>
__device__ __forceinline__ void convert_w4(const v4u w, v4u& e0, v4u& e1, v4u& o0, v4u& o1) {
    // (x & 0x000F000F) ^ c with c = exponent bits | 0x0008 per half: the xor both flips the
    // nibble's sign bit (two's complement -> offset by 8) and sets the exponent, because the two
    // bit sets are disjoint.  One 3-input bit operation per pair of weights.
    constexpr uint32_t msk = 0x000F000Fu;
    constexpr uint32_t cst = (ADT == FNN_F16 ? 0x64006400u : 0x43004300u) ^ 0x00080008u;
    uint32_t e[8], o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t x = w[q];
        e[2 * q] = (x & msk) ^ cst;
        e[2 * q + 1] = ((x >> 8) & msk) ^ cst;
        o[2 * q] = ((x >> 4) & msk) ^ cst;
        o[2 * q + 1] = ((x >> 12) & msk) ^ cst;
    }
    e0 = v4u{e[0], e[1], e[2], e[3]};
    e1 = v4u{e[4], e[5], e[6], e[7]};
    o0 = v4u{o[0], o[1], o[2], o[3]};
    o1 = v4u{o[4], o[5], o[6], o[7]};
}

// The reference's per-weight dequantisation for fp16 scales (flashnn/quant_gemm.py:14-17, 168): the weight
// minus its zero point, rounded to fp16, times the scale, rounded to fp16 again; the dot product then runs
// over these rounded weights.  x holds two weights as coff + q (the exponent-trick conversion, exact), so
// the first subtraction is exact and the other two operations round exactly as torch rounds them.
// Used where activations and scales are both fp16: the result then differs from the reference's only by
// the order of the fp32 additions.
// ZP = false: no zero points were given; the reference then subtracts zeros, which changes nothing.
template <bool ZP>
__device__ __forceinline__ uint32_t ref_dq_f16(uint32_t x, const v2h coff, const v2h zp, const v2h s) {
#pragma clang fp contract(off)
    v2h v = __builtin_bit_cast(v2h, x) - coff;
    if constexpr (ZP) v = v - zp;
    v = v * s;
    return __builtin_bit_cast(uint32_t, v);
}
template <bool ZP>
__device__ __forceinline__ v4u ref_dq_f16(v4u x, const v2h coff, const v2h zp, const v2h s) {
    return v4u{ref_dq_f16<ZP>(x[0], coff, zp, s), ref_dq_f16<ZP>(x[1], coff, zp, s), ref_dq_f16<ZP>(x[2], coff, zp, s),
               ref_dq_f16<ZP>(x[3], coff, zp, s)};
}
// The same for bf16 scales (the reference's torch path with bf16 tables): there is no packed bf16 arithmetic,
// so the two operations run in fp32 on the weight as a small whole number u = off + q (off: 8 for int4, 128 for
// int8) and v_cvt_pk_bf16_f32 rounds a pair to nearest even.
// Merged form, for whole zero points of at most 128: u * s - (off + zp) * s in one fma.  u * s (8 x 8 bits) and
// (off + zp) * s (9 x 8 bits) are exact in fp32, so the fma returns (q - zp) * s exactly (17 bits), and q - zp is
// a bf16 number: the one rounding of the pack is the reference's second rounding and its first changes nothing.
__device__ __forceinline__ uint32_t ref_dq_bf16_merged(float u0, float u1, float s, float neg_off_zp_s) {
    const v2f r = {__builtin_fmaf(u0, s, neg_off_zp_s), __builtin_fmaf(u1, s, neg_off_zp_s)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(r, v2bf));
}
// Two-step form, any zero point: (u - off) - zp is the fp32 rounding of q - zp (exact unless zp is below 2^-16 q,
// where the value is nowhere near a bf16 rounding boundary), rounded to bf16; times s (8 x 8 bits: exact), rounded.
__device__ __forceinline__ uint32_t ref_dq_bf16(float u0, float u1, float off, float zp, float s) {
#pragma clang fp contract(off)
    const v2f d = {(u0 - off) - zp, (u1 - off) - zp};
    const uint32_t db = __builtin_bit_cast(uint32_t, __builtin_convertvector(d, v2bf));
    const v2f r = {__uint_as_float(db << 16) * s, __uint_as_float(db & 0xFFFF0000u) * s};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(r, v2bf));
}
// The four bytes of x as fp32 (v_cvt_f32_ubyte0..3; x passes through an empty asm so that masks applied before
// are not folded into one bit-field extract per byte)
__device__ __forceinline__ void bytes_to_f32(uint32_t x, float (&f)[4]) {
    asm("" : "+v"(x));
    f[0] = (float)(x & 0xFFu);
    f[1] = (float)((x >> 8) & 0xFFu);
    f[2] = (float)((x >> 16) & 0xFFu);
    f[3] = (float)(x >> 24);
}

// Whole operand groups through ref_dq_bf16: c = -(off + zp) * s (used by the one-step form only).
// 16 int8 (k .. k+15 of one row) -> two bf16 MFMA operands in natural k order (as convert_w8)
template <bool ONE_STEP>
__device__ __forceinline__ void dq_w8_bf16(const v4u w, float s, float zp, float c, v4u& s0, v4u& s1) {
    uint32_t o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        float f[4];
        bytes_to_f32(w[q] ^ 0x80808080u, f);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            o[2 * q + i] = ONE_STEP ? ref_dq_bf16_merged(f[2 * i], f[2 * i + 1], s, c) : ref_dq_bf16(f[2 * i], f[2 * i + 1], 128.f, zp, s);
    }
    s0 = v4u{o[0], o[1], o[2], o[3]};
    s1 = v4u{o[4], o[5], o[6], o[7]};
}
// 16 bytes = 16 k of two channels (index 0: the even channel, low nibbles) -> bf16 operands; NAT: natural k order
// (as convert_w4_nat), else the order (0,2)(1,3)(4,6)(5,7) of convert_w4
template <bool NAT, bool ONE_STEP>
__device__ __forceinline__ void dq_w4_bf16(const v4u w, const float (&s)[2], const float (&zp)[2], const float (&c)[2],
                                           v4u& e0, v4u& e1, v4u& o0, v4u& o1) {
    uint32_t e[8], o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t x = w[q] ^ 0x88888888u;      // two's complement -> offset by 8
        float fe[4], fo[4];
        bytes_to_f32(x & 0x0F0F0F0Fu, fe);
        bytes_to_f32((x >> 4) & 0x0F0F0F0Fu, fo);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int k0 = NAT ? 2 * i : i, k1 = NAT ? 2 * i + 1 : i + 2;
            e[2 * q + i] = ONE_STEP ? ref_dq_bf16_merged(fe[k0], fe[k1], s[0], c[0]) : ref_dq_bf16(fe[k0], fe[k1], 8.f, zp[0], s[0]);
            o[2 * q + i] = ONE_STEP ? ref_dq_bf16_merged(fo[k0], fo[k1], s[1], c[1]) : ref_dq_bf16(fo[k0], fo[k1], 8.f, zp[1], s[1]);
        }
    }
    e0 = v4u{e[0], e[1], e[2], e[3]};
    e1 = v4u{e[4], e[5], e[6], e[7]};
    o0 = v4u{o[0], o[1], o[2], o[3]};
    o1 = v4u{o[4], o[5], o[6], o[7]};
}
// whether a bf16 zero point lets the one-step form stand for the reference's two roundings
__device__ __forceinline__ bool bf16_zp_is_whole(float z) { return z == rintf(z) && fabsf(z) <= 128.f; }

constexpr int FNN_I8 = 3;   // type code of int8 zero points (mixture-of-experts entry point only)

// The bias as the reference adds it: its int8 branch casts the product to the output type and then adds the
// bias in that type (flashnn/quant_gemm.py:168-173) - two roundings, which show where product and bias nearly
// cancel; its int4 branch adds in fp32 and rounds once (:201-204).  The caller rounds the returned sum to
// the output type.
template <int WBITS>
__device__ __forceinline__ float add_bias(float v, float bias, int out_dtype) {
    if constexpr (WBITS == 8) {
        if (out_dtype == FNN_F16) v = f16_bits_to_f32(f32_to_f16_bits(v));
        else if (out_dtype == FNN_BF16) v = bf16_bits_to_f32(f32_to_bf16_bits(v));
    }
    return v + bias;
}

__device__ __forceinline__ float load_zp_f32(const void* p, int64_t i, int dtype) {
    return dtype == FNN_I8 ? (float)((const int8_t*)p)[i] : load_as_f32(p, i, dtype);
}

// an fp16 bit pattern in both halves of a packed pair
__device__ __forceinline__ v2h pair_of_f16_bits(uint32_t h) {
    return __builtin_bit_cast(v2h, (h & 0xFFFFu) * 0x10001u);
}

// reorder 8 consecutive 16-bit values to (0,2)(1,3)(4,6)(5,7)
__device__ __forceinline__ v4u perm_act_w4(const v4u a) {
    return v4u{__builtin_amdgcn_perm(a[1], a[0], 0x05040100u), __builtin_amdgcn_perm(a[1], a[0], 0x07060302u),
               __builtin_amdgcn_perm(a[3], a[2], 0x05040100u), __builtin_amdgcn_perm(a[3], a[2], 0x07060302u)};
}

// 16 bytes = 16 k of two channels -> operands in natural k order (one byte shuffle per dword
// puts the nibbles of k and k+1 into the two halves of a dword).
template <int ADT>
__device__ __forceinline__ void convert_w4_nat(const v4u w, v4u& e0, v4u& e1, v4u& o0, v4u& o1) {
    constexpr uint32_t msk = 0x000F000Fu;
    constexpr uint32_t cst = (ADT == FNN_F16 ? 0x64006400u : 0x43004300u) ^ 0x00080008u;
    uint32_t e[8], o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t y = __builtin_amdgcn_perm(w[q], w[q], 0x03010200u);   // bytes k0 k2 k1 k3
        e[2 * q] = (y & msk) ^ cst;
        e[2 * q + 1] = ((y >> 8) & msk) ^ cst;
        o[2 * q] = ((y >> 4) & msk) ^ cst;
        o[2 * q + 1] = ((y >> 12) & msk) ^ cst;
    }
    e0 = v4u{e[0], e[1], e[2], e[3]};
    e1 = v4u{e[4], e[5], e[6], e[7]};
    o0 = v4u{o[0], o[1], o[2], o[3]};
    o1 = v4u{o[4], o[5], o[6], o[7]};
}


// The same for fp16 operands with no shift for the odd channel: its nibble stays at bits 4..7 of each half, where
// under the exponent of 64 a mantissa step is 1/16, so the operand is 64 + (v + 8) (the even channel's: 1024 + (v + 8)).
__device__ __forceinline__ void convert_w4_nat_f16_2off(const v4u w, v4u& e0, v4u& e1, v4u& o0, v4u& o1) {
    constexpr uint32_t m0 = 0x000F000Fu, c0 = 0x64006400u ^ 0x00080008u;
    constexpr uint32_t m1 = 0x00F000F0u, c1 = 0x54005400u ^ 0x00800080u;
    uint32_t e[8], o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t y = __builtin_amdgcn_perm(w[q], w[q], 0x03010200u);   // bytes k0 k2 k1 k3
        const uint32_t y2 = y >> 8;
        e[2 * q] = (y & m0) ^ c0;
        o[2 * q] = (y & m1) ^ c1;
        e[2 * q + 1] = (y2 & m0) ^ c0;
        o[2 * q + 1] = (y2 & m1) ^ c1;
    }
    e0 = v4u{e[0], e[1], e[2], e[3]};
    e1 = v4u{e[4], e[5], e[6], e[7]};
    o0 = v4u{o[0], o[1], o[2], o[3]};
    o1 = v4u{o[4], o[5], o[6], o[7]};
}

// gemm_weight_only.hip: where the caller gave scratch and the tables are fp16 (per channel or per group of
// 128), converts the bf16 activation rows of p to fp16 rows in the scratch, each row scaled by a power of two
// so that every value is representable, and fills q with the same problem on those rows (q.act_unscale
// holding the inverse scales); false, with nothing launched, if that does not apply
bool convert_act_to_f16(const WoArgs& p, WoArgs& q, hipStream_t st);
size_t act_f16_ws_bytes(int64_t M, int64_t K);
// gemm_wo_panel.hip: 9 .. a few hundred activation rows; false if the shape does not suit it
bool launch_wo_panel(WoArgs& p, int wbits, int act_dtype, hipStream_t st);
// gemm_wo_tile.hip: more than 64 activation rows, tiled MFMA kernel; false if the shape does not suit it
bool launch_wo_tile(WoArgs& p, int wbits, int act_dtype, hipStream_t st);
// ... and the number of tiles (workgroups) it would launch for this problem
int wo_tile_count(const WoArgs& p, int wbits);
// ... its mixture-of-experts form (int4, per-channel tables, blocks of 128 rows or more); false otherwise
bool launch_wo_tile_moe(WoArgs& p, const MoeArgs& q, int act_dtype, hipStream_t st);
// the int4 per-channel kernel over gathered rows of a mixture of experts; false if the shape does not suit it
bool launch_wo_panel_moe(WoArgs& p, const MoeArgs& q, int act_dtype, hipStream_t st);

}  // namespace fnn
