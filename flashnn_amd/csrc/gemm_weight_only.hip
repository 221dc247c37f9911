// Weight-only GEMMs for gfx950 (fp16/bf16 activations, int8 or packed int4 weights):
//   out[m,n] = sum_k act[m,k] * (w[n,k] - zp[g(k),n]) * scale[g(k),n]  (+ bias[n])
//
// Streaming kernel (decode shapes; K % 64 == 0, 16-byte aligned rows)
//   * a 512-thread workgroup (8 waves) owns one tile of 16 weight rows (16 output channels
//     for int8, 32 for packed int4) and up to 64 activation rows; the waves split K;
//   * every lane streams its weight row with 16-byte loads kept PF steps ahead in
//     registers (no LDS, no barriers in the loop), converts the integers to the
//     activation type in registers and feeds them to v_mfma_f32_16x16x32_{f16,bf16} as the
//     "A" operand; the activations are the "B" operand (columns beyond M are zero);
//   * integer -> float conversion uses exponent tricks instead of per-element converts:
//       int4:  (nibble ^ 8) | 0x4300  is the bf16 number 128 + (v + 8),
//              (nibble ^ 8) | 0x6400  is the fp16 number 1024 + (v + 8);
//       int8 -> fp16: byte ^ 0x80 placed under 0x64 gives 1024 + (v + 128);
//       int8 -> bf16: v_cvt_f32_ubyte of byte ^ 0x80, upper 16 bits (exact: 8 bits).
//     The constant offset c is removed together with the zero point:
//       sum_k (c + v_k - zp) a_k  =  acc - (c + zp) * sum_k a_k,
//     where sum_k a_k comes from one more MFMA against a matrix of ones;
//   * group scales are applied whenever a K-group ends (fp32), per-channel scales once;
//   * the 8 partial tiles are added in a fixed order through LDS (deterministic, no
//     atomics), then bias, rounding and the store.
//
// Any other shape takes a guarded one-output-per-thread kernel.
//
// Reference semantics: flashnn/quant_gemm.py:148-206; layouts
// flashnn/triton_kernels/gemm_a16w4.py:163-182 (nibble order), :296-297 (scale rows).
#include "fnn_common.h"

#include <type_traits>

#include "wo_common.h"

namespace fnn {


// G32: tables per group of 32 values.  A 64-value step is then two groups, and the two MFMAs of a step must each
// cover one of them: a lane takes values 8 lg .. 8 lg + 7 of either half of the step (two 8-byte weight loads
// and two activation pieces 32 values apart) instead of 16 consecutive ones, and the sums are folded after
// each half.
template <int WBITS, int ADT, int MB, bool GROUPED, bool G32 = false>
__global__ __launch_bounds__(kWoWaves * 64) void gemm_wo_stream_kernel(const WoArgs p) {
    static_assert(!G32 || GROUPED, "groups of 32 are group tables");
    typedef MfmaT<ADT> MT;
    constexpr int NH = WBITS == 4 ? 2 : 1;      // channel halves per weight row (int4: even/odd)
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    __shared__ float red[kWoWaves][MB][NH][4][64];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 15;   // weight row within the tile (A operand) / activation row (B operand)
    const int lg = lane >> 4;   // k sub-block of the lane

    // XCD-aware tile order: ids congruent mod 8 share an L2; give each XCD a contiguous band so
    // that neighbouring tiles (which share cache lines of the scale rows) meet in the same L2.
    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = (wrows + 15) / 16;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    const int row0 = tile * 16;

    const int steps = p.K / 64;
    const int s_begin = (int)((int64_t)steps * wave / kWoWaves);
    const int s_end = (int)((int64_t)steps * (wave + 1) / kWoWaves);

    const int wrow = min(row0 + li, wrows - 1);
    const char* wptr = (const char*)p.qw + (int64_t)wrow * p.ldw + lg * (G32 ? 8 : 16);
    const uint16_t* aptr[MB];
    bool avalid[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = p.m_base + mb * 16 + li;
        avalid[mb] = m < p.M;
        aptr[mb] = (const uint16_t*)p.act + (int64_t)min(m, p.M - 1) * p.lda + lg * (G32 ? 8 : 16);
    }

    auto load_w = [&](int step) -> v4u {
        const int s = min(step, s_end - 1);
        if constexpr (G32) {
            const v2u lo = *(const v2u*)(wptr + (int64_t)s * 64), hi = *(const v2u*)(wptr + (int64_t)s * 64 + 32);
            return v4u{lo[0], lo[1], hi[0], hi[1]};
        } else {
            return *(const v4u*)(wptr + (int64_t)s * 64);
        }
    };
    auto load_a = [&](int mb, int step, int half) -> v4u {
        const int s = min(step, s_end - 1);
        return avalid[mb] ? *(const v4u*)(aptr[mb] + (int64_t)s * 64 + half * (G32 ? 32 : 8)) : v4u{0, 0, 0, 0};
    };

    v4f outv[MB][NH], accg[MB][NH], asum[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        asum[mb] = v4f{0, 0, 0, 0};
#pragma unroll
        for (int h = 0; h < NH; ++h) { outv[mb][h] = v4f{0, 0, 0, 0}; accg[mb][h] = v4f{0, 0, 0, 0}; }
    }

    // channel of output register r, half h of this lane
    auto chan = [&](int h, int r) -> int {
        const int wr = row0 + 4 * lg + r;
        return WBITS == 4 ? 2 * wr + h : wr;
    };
    // fold the running group sums into the outputs with the scales of K-group `grp`
    auto fold = [&](int grp) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = min(chan(h, r), p.N - 1);
                const int64_t idx = GROUPED ? (int64_t)grp * p.N + n : n;
                const float sc = load_as_f32(p.scale, idx, p.scale_dtype);
                const float zc = c_off + (p.zp ? load_as_f32(p.zp, idx, p.zp_dtype) : 0.f);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    outv[mb][h][r] += sc * (accg[mb][h][r] - zc * asum[mb][r]);
                    accg[mb][h][r] = 0.f;
                }
            }
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) asum[mb] = v4f{0, 0, 0, 0};
    };

    if (s_begin < s_end) {
        v4u wq[kPF];
        v4u aq[kPFA][MB][2];
#pragma unroll
        for (int i = 0; i < kPF; ++i) wq[i] = load_w(s_begin + i);
#pragma unroll
        for (int i = 0; i < kPFA; ++i)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                aq[i][mb][0] = load_a(mb, s_begin + i, 0);
                aq[i][mb][1] = load_a(mb, s_begin + i, 1);
            }
        const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
        const int gsteps = GROUPED ? p.group / 64 : 1;

        for (int sb = s_begin; sb < s_end; sb += kPF) {
#pragma unroll
            for (int i = 0; i < kPF; ++i) {
                const int step = sb + i;
                if (step < s_end) {
                    const v4u w = wq[i];
                    wq[i] = load_w(step + kPF);
                    v4u a[MB][2];
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        a[mb][0] = aq[i % kPFA][mb][0];
                        a[mb][1] = aq[i % kPFA][mb][1];
                        aq[i % kPFA][mb][0] = load_a(mb, step + kPFA, 0);
                        aq[i % kPFA][mb][1] = load_a(mb, step + kPFA, 1);
                    }
                    if constexpr (G32) {
                        v4u e[2], o[2];
                        if constexpr (WBITS == 4) convert_w4<ADT>(w, e[0], e[1], o[0], o[1]);
                        else convert_w8<ADT>(w, e[0], e[1]);
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb) {
                                const v4u b = WBITS == 4 ? perm_act_w4(a[mb][hf]) : a[mb][hf];
                                accg[mb][0] = MT::mma(e[hf], b, accg[mb][0]);
                                if constexpr (WBITS == 4) accg[mb][1] = MT::mma(o[hf], b, accg[mb][1]);
                                asum[mb] = MT::mma(ones, b, asum[mb]);
                            }
                            fold(2 * step + hf);
                        }
                    } else if constexpr (WBITS == 4) {
                        v4u e0, e1, o0, o1;
                        convert_w4<ADT>(w, e0, e1, o0, o1);
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) {
                            const v4u b0 = perm_act_w4(a[mb][0]);
                            const v4u b1 = perm_act_w4(a[mb][1]);
                            accg[mb][0] = MT::mma(e0, b0, accg[mb][0]);
                            accg[mb][1] = MT::mma(o0, b0, accg[mb][1]);
                            asum[mb] = MT::mma(ones, b0, asum[mb]);
                            accg[mb][0] = MT::mma(e1, b1, accg[mb][0]);
                            accg[mb][1] = MT::mma(o1, b1, accg[mb][1]);
                            asum[mb] = MT::mma(ones, b1, asum[mb]);
                        }
                    } else {
                        v4u s0, s1;
                        convert_w8<ADT>(w, s0, s1);
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) {
                            accg[mb][0] = MT::mma(s0, a[mb][0], accg[mb][0]);
                            asum[mb] = MT::mma(ones, a[mb][0], asum[mb]);
                            accg[mb][0] = MT::mma(s1, a[mb][1], accg[mb][0]);
                            asum[mb] = MT::mma(ones, a[mb][1], asum[mb]);
                        }
                    }
                    if constexpr (GROUPED && !G32) {
                        if ((step + 1) % gsteps == 0 || step + 1 == s_end) fold(step / gsteps);
                    }
                }
            }
        }
        if constexpr (!GROUPED) fold(0);
    }

    // ---- add the 8 partial tiles in wave order, then bias / rounding / store ----
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave][mb][h][r][lane] = outv[mb][h][r];
    __syncthreads();
    constexpr int ELEMS = MB * NH * 4 * 64;
    for (int e = threadIdx.x; e < ELEMS; e += kWoWaves * 64) {
        const int l = e & 63;
        const int r = (e >> 6) & 3;
        const int h = NH == 2 ? (e >> 8) & 1 : 0;
        const int mb = e / (NH * 256);
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kWoWaves; ++w) v += red[w][mb][h][r][l];
        const int m = p.m_base + mb * 16 + (l & 15);
        const int wr = row0 + 4 * (l >> 4) + r;
        const int n = WBITS == 4 ? 2 * wr + h : wr;
        if (m < p.M && n < p.N) {
            if (p.bias) v = add_bias<WBITS>(v, load_as_f32(p.bias, n, p.bias_dtype), p.out_dtype);
            store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
        }
    }
}



// Stage the scales and zero points of NC consecutive channels (all K-groups) in LDS as fp32:
// s_lds[g*NC + c] = scale, z_lds[g*NC + c] = scale * (c_off + zp).  16-bit scale type SDT, same
// type for the zero points, N a multiple of NC and 16-byte aligned tables (checked on the
// host): every thread loads 16-byte pieces, all loads of a batch before the first store, so a
// batch costs one memory latency.
template <int SDT, int NC>
__device__ __forceinline__ void fill_scales_lds(float* s_lds, float* z_lds, const WoArgs& p, int n0,
                                                int ngroups, float c_off, int tid, int nthreads) {
    constexpr int VPR = NC / 8;   // 16-byte pieces per group row
    const int nvec = ngroups * VPR;
    for (int v0 = 0; v0 < nvec; v0 += 2 * nthreads) {
        v4u sv[2], zv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int e = min(v0 + u * nthreads + tid, nvec - 1);
            const int64_t off = (int64_t)(e / VPR) * p.N + n0 + (e % VPR) * 8;
            sv[u] = *(const v4u*)((const uint16_t*)p.scale + off);
            zv[u] = p.zp ? *(const v4u*)((const uint16_t*)p.zp + off) : v4u{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int e = v0 + u * nthreads + tid;
            if (e < nvec) {
                float sc[8], zo[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    sc[2 * j] = bits_to_f32<SDT>(sv[u][j] & 0xFFFFu);
                    sc[2 * j + 1] = bits_to_f32<SDT>(sv[u][j] >> 16);
                    zo[2 * j] = sc[2 * j] * (c_off + bits_to_f32<SDT>(zv[u][j] & 0xFFFFu));
                    zo[2 * j + 1] = sc[2 * j + 1] * (c_off + bits_to_f32<SDT>(zv[u][j] >> 16));
                }
                float* sd = s_lds + (e / VPR) * NC + (e % VPR) * 8;
                float* zd = z_lds + (e / VPR) * NC + (e % VPR) * 8;
                *(v4f*)sd = v4f{sc[0], sc[1], sc[2], sc[3]};
                *(v4f*)(sd + 4) = v4f{sc[4], sc[5], sc[6], sc[7]};
                *(v4f*)zd = v4f{zo[0], zo[1], zo[2], zo[3]};
                *(v4f*)(zd + 4) = v4f{zo[4], zo[5], zo[6], zo[7]};
            }
        }
    }
}

// ------------------------------------------------------------------ decode kernel (M <= 8)
// A 256-thread workgroup (4 waves, splitting K) owns 8 weight rows (8 channels for int8,
// 16 for packed int4): with N = 28672 int4 channels that is 1792 workgroups, exactly 7 per CU.
// The 16 rows of the MFMA "A" operand are used twice: lane row i holds weight row (i & 7) for
// the first (i < 8) or second (i >= 8) 16-byte half of a 32-byte K segment, so one load
// instruction of a wave covers 8 rows x 128 contiguous bytes and every loaded byte is used.
// The 16 columns of the "B" operand are used the same way: column j holds activation row
// (j & 7) for the first or second half.  Of the 16x16 result only the two 8x8 blocks on
// the diagonal (same half on both sides) are meaningful; they are added at the end.
// Scales and zero points of the tile (all K-groups) and, when they fit, the activation rows
// are staged in LDS once per workgroup; weights stream through registers kPF loads ahead.
constexpr int kDecWaves = 4;

template <int WBITS, int ADT, bool GROUPED, bool ACT_LDS>
__global__ __launch_bounds__(kDecWaves * 64) void gemm_wo_decode_kernel(const WoArgs p) {
    typedef MfmaT<ADT> MT;
    constexpr int NH = WBITS == 4 ? 2 : 1;
    constexpr int NC = 8 * NH;                 // channels per tile
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int half = li >> 3;     // which 16-byte half of the lane group's 32-byte K segment
    const int r8 = li & 7;        // weight row (A side) / activation row (B side)

    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = (wrows + 7) / 8;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    const int row0 = tile * 8;
    const int n0 = row0 * NH;

    const int steps = p.K / 128;
    const int s_begin = (int)((int64_t)steps * wave / kDecWaves);
    const int s_end = (int)((int64_t)steps * (wave + 1) / kDecWaves);
    const int ngroups = GROUPED ? p.K / p.group : 1;

    // LDS carve-up: [scale ngroups*NC f32][zoff ngroups*NC f32][red 4*NH*4*64 f32][acts]
    float* s_lds = (float*)smem;
    float* z_lds = s_lds + ngroups * NC;
    float* red = z_lds + ngroups * NC;
    uint16_t* a_lds = (uint16_t*)(red + kDecWaves * NH * 4 * 64);
    const int a_stride = p.K + 32;   // elements; the pad staggers the rows over the banks

    // ---- issue the first weight loads, then fill LDS while they are in flight ----
    const char* wptr = (const char*)p.qw + (int64_t)min(row0 + r8, wrows - 1) * p.ldw + lg * 32 + half * 16;
    auto load_w = [&](int step) -> v4u {
        const int s = min(step, s_end - 1);
        return __builtin_nontemporal_load((const v4u*)(wptr + (int64_t)s * 128));
    };
    v4u wq[kPF];
    if (s_begin < s_end) {
#pragma unroll
        for (int i = 0; i < kPF; ++i) wq[i] = load_w(s_begin + i);
    }

    for (int e = threadIdx.x; e < ngroups * NC; e += kDecWaves * 64) {
        const int g = e / NC, c = e % NC;
        const int64_t idx = (int64_t)g * p.N + min(n0 + c, p.N - 1);
        const float sc = load_as_f32(p.scale, idx, p.scale_dtype);
        const float z = p.zp ? load_as_f32(p.zp, idx, p.zp_dtype) : 0.f;
        s_lds[e] = sc;
        z_lds[e] = sc * (c_off + z);
    }
    if constexpr (ACT_LDS) {
        const int chunks = p.K / 8;
        for (int e = threadIdx.x; e < p.M * chunks; e += kDecWaves * 64) {
            const int m = e / chunks, c = e % chunks;
            v4u v = *(const v4u*)((const uint16_t*)p.act + (int64_t)m * p.lda + c * 8);
            if constexpr (WBITS == 4) v = perm_act_w4(v);
            *(v4u*)(a_lds + m * a_stride + c * 8) = v;
        }
    }
    __syncthreads();

    // activation operand of this lane for K step `step`, sub-slot `slot` (8 values)
    const bool avalid = r8 < p.M;
    const int koff = lg * 32 + half * 16;
    const uint16_t* aptr = (const uint16_t*)p.act + (int64_t)min(r8, p.M - 1) * p.lda + koff;
    auto load_a_gbl = [&](int step, int slot) -> v4u {
        const int s = min(step, s_end - 1);
        return avalid ? *(const v4u*)(aptr + (int64_t)s * 128 + slot * 8) : v4u{0, 0, 0, 0};
    };
    auto load_a_lds = [&](int step, int slot) -> v4u {
        return avalid ? *(const v4u*)(a_lds + r8 * a_stride + step * 128 + koff + slot * 8) : v4u{0, 0, 0, 0};
    };

    v4f outv[NH], accg[NH], asum = v4f{0, 0, 0, 0};
#pragma unroll
    for (int h = 0; h < NH; ++h) { outv[h] = v4f{0, 0, 0, 0}; accg[h] = v4f{0, 0, 0, 0}; }

    // result register r of this lane is weight row (4*lg + r) & 7: channels NH*(4*(lg&1)+r)+h
    auto fold = [&](int grp) {
        const float* sp = s_lds + grp * NC + NH * 4 * (lg & 1);
        const float* zp = z_lds + grp * NC + NH * 4 * (lg & 1);
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                outv[h][r] += sp[NH * r + h] * accg[h][r] - zp[NH * r + h] * asum[r];
                accg[h][r] = 0.f;
            }
        asum = v4f{0, 0, 0, 0};
    };

    if (s_begin < s_end) {
        v4u aq[kPFA][2];
        if constexpr (!ACT_LDS) {
#pragma unroll
            for (int i = 0; i < kPFA; ++i) {
                aq[i][0] = load_a_gbl(s_begin + i, 0);
                aq[i][1] = load_a_gbl(s_begin + i, 1);
            }
        }
        const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
        const int gsteps = GROUPED ? p.group / 128 : 1;
        for (int sb = s_begin; sb < s_end; sb += kPF) {
#pragma unroll
            for (int i = 0; i < kPF; ++i) {
                const int step = sb + i;
                if (step < s_end) {
                    const v4u w = wq[i];
                    wq[i] = load_w(step + kPF);
                    v4u a0, a1;
                    if constexpr (ACT_LDS) {
                        a0 = load_a_lds(step, 0);
                        a1 = load_a_lds(step, 1);
                    } else {
                        a0 = aq[i % kPFA][0];
                        a1 = aq[i % kPFA][1];
                        aq[i % kPFA][0] = load_a_gbl(step + kPFA, 0);
                        aq[i % kPFA][1] = load_a_gbl(step + kPFA, 1);
                        if constexpr (WBITS == 4) { a0 = perm_act_w4(a0); a1 = perm_act_w4(a1); }
                    }
                    if constexpr (WBITS == 4) {
                        v4u e0, e1, o0, o1;
                        convert_w4<ADT>(w, e0, e1, o0, o1);
                        accg[0] = MT::mma(e0, a0, accg[0]);
                        accg[1] = MT::mma(o0, a0, accg[1]);
                        asum = MT::mma(ones, a0, asum);
                        accg[0] = MT::mma(e1, a1, accg[0]);
                        accg[1] = MT::mma(o1, a1, accg[1]);
                        asum = MT::mma(ones, a1, asum);
                    } else {
                        v4u s0, s1;
                        convert_w8<ADT>(w, s0, s1);
                        accg[0] = MT::mma(s0, a0, accg[0]);
                        asum = MT::mma(ones, a0, asum);
                        accg[0] = MT::mma(s1, a1, accg[0]);
                        asum = MT::mma(ones, a1, asum);
                    }
                    if constexpr (GROUPED) {
                        if ((step + 1) % gsteps == 0 || step + 1 == s_end) fold(step / gsteps);
                    }
                }
            }
        }
        if constexpr (!GROUPED) fold(0);
    }

    // ---- add the partial tiles of the 4 waves and the two diagonal blocks ----
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((wave * NH + h) * 4 + r) * 64 + lane] = outv[h][r];
    __syncthreads();
    for (int e = threadIdx.x; e < p.M * NC; e += kDecWaves * 64) {
        const int m = e / NC, c = e % NC;
        const int row = c / NH, h = c % NH;          // weight row 0..7 of the tile
        const int r = row & 3;
        const int lane1 = m + 16 * (row >> 2);              // result row `row`,     column m
        const int lane2 = (m + 8) + 16 * ((row + 8) >> 2);  // result row `row`+8,   column m+8
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kDecWaves; ++w)
            v += red[((w * NH + h) * 4 + r) * 64 + lane1] + red[((w * NH + h) * 4 + r) * 64 + lane2];
        const int n = n0 + c;
        if (n < p.N) {
            if (p.bias) v = add_bias<WBITS>(v, load_as_f32(p.bias, n, p.bias_dtype), p.out_dtype);
            store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
        }
    }
}


// --------------------------------------------- decode kernel, activations staged in LDS
// Same tiling as gemm_wo_decode_kernel (8 weight rows per 256-thread workgroup, the two
// diagonal 8x8 blocks of the 16x16 MFMA result) with the per-step VALU work cut down:
//   * G128 (group size 128 = one 128-byte K step): the 8 result columns of a block are
//     shared by MP activation rows and 8/MP consecutive K-groups.  Column gslot*MP + m gets
//     the activations of row m only in the steps of group slot gslot (a zeroed LDS
//     region otherwise), so 8/MP groups accumulate side by side and the scales are
//     applied once per 8/MP steps instead of every step;
//   * sign flip, nibble mask and exponent insertion are one 3-input bit operation;
//   * the wave index is made scalar so the K loop is scalar control flow, the weight
//     address is a scalar base plus a per-lane 32-bit offset.
// REFQ (1, or 2 with zero points; fp16 activations, per-channel fp16 scales and zero points): every weight is dequantised and rounded
// to fp16 as the reference's torch path does before the dot product (ref_dq_f16), and the scale tables, the
// MFMAs against ones and the fold are not needed.
// REFQ 3 (4 with zero points): the same with fp16 tables per group of 32 or 64 values of K.  A lane's 16
// weights of a step lie in one group; its scale and zero point come from an LDS table of (scale, zero point)
// pairs, [K / group][channels of the tile], one 4-byte read per channel and step.
template <int WBITS, int ADT, bool G128, int MP, int CH, bool FULL, int REFQ = 0>
__global__ __launch_bounds__(kDecWaves * 64) void gemm_wo_decode_lds_kernel(const WoArgs p) {
    static_assert(!REFQ || !G128, "reference rounding: tables per channel or per small group");
    static_assert(REFQ < 3 || ADT == FNN_F16, "reference rounding with small groups: fp16");
    constexpr bool RQG = REFQ >= 3;              // tables per group of 32 or 64
    constexpr bool RQZ = REFQ == 2 || REFQ == 4;
    // bf16 activations with per-channel bf16 tables: both roundings to bf16, worked in fp32 (ref_dq_bf16)
    constexpr bool RQBF = REFQ != 0 && ADT == FNN_BF16;
    typedef MfmaT<ADT> MT;
    constexpr int NH = WBITS == 4 ? 2 : 1;
    constexpr int NC = 8 * NH;
    constexpr int GS = G128 ? 8 / MP : 1;       // K-groups accumulated side by side
    constexpr int UN = 8;                        // weight loads in flight per lane
    // CH = steps per straight-line chunk; FULL = every wave owns whole chunks (no guards)
    constexpr int ZERO_BYTES = CH * 256 + 32;
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int half = li >> 3;
    const int j7 = li & 7;

    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = (wrows + 7) / 8;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= tiles) return;
    const int row0 = tile * 8;
    const int n0 = row0 * NH;

    const int steps = p.K / 128;
    // waves take whole blocks of 8 steps so that group slots line up with step indices
    const int nblk = (steps + 7) / 8;
    const int s_begin = (nblk * wave / kDecWaves) * 8;
    const int s_end = min((nblk * (wave + 1) / kDecWaves) * 8, steps);
    const int ngroups = G128 ? steps : RQG ? p.K / p.group : 1;

    // LDS: [zeros][scale ngroups*NC f32][zoff ngroups*NC f32][red 4*NH*4*64 f32][acts]
    // (RQG: the first table holds the (scale, zero point) pairs of fp16 instead, the second is unused)
    float* s_lds = (float*)(smem + ZERO_BYTES);
    float* z_lds = s_lds + ngroups * NC;
    float* red = z_lds + ngroups * NC;
    uint16_t* a_lds = (uint16_t*)(red + kDecWaves * NH * 4 * 64);
    const int a_stride = p.K + 32;

    const int wrow_l = min(row0 + j7, wrows - 1) - row0;
    const uint32_t w_off = (uint32_t)wrow_l * (uint32_t)p.ldw + lg * 32 + half * 16;
    const char* w_tile = (const char*)p.qw + (int64_t)row0 * p.ldw;
    auto load_w = [&](int step) -> v4u {
        const char* base = w_tile + (int64_t)min(step, s_end - 1) * 128;   // scalar
        return __builtin_nontemporal_load((const v4u*)(base + w_off));
    };
    // REFQ: the scale and zero point of this lane's weight row (two channels per row with int4 weights),
    // requested ahead of the weights: loads return in order, and the first conversion needs them
    uint32_t rq_sb[NH], rq_zb[NH];
    if constexpr (REFQ == 1 || REFQ == 2) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const int n = min(n0 + j7 * NH + h, p.N - 1);
            rq_sb[h] = ((const uint16_t*)p.scale)[n];
            rq_zb[h] = REFQ == 2 ? ((const uint16_t*)p.zp)[n] : 0u;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    v4u wq[UN];
    if (s_begin < s_end) {
#pragma unroll
        for (int i = 0; i < UN; ++i) wq[i] = load_w(s_begin + i);
    }
    v2h rq_s[NH], rq_z[NH];
    const v2h rq_c = pair_of_f16_bits(WBITS == 4 ? 0x6408u : 0x6480u);   // 1032 / 1152: what the conversion adds
    float bq_s[2], bq_z[2], bq_c[2];
    bool whole_zp = true;    // wave-uniform: every zero point of the wave's rows is whole and at most 128 (one-step form)
    if constexpr (REFQ == 1 || REFQ == 2) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            if constexpr (RQBF) {
                bq_s[h] = bf16_bits_to_f32(rq_sb[h]);
                bq_z[h] = bf16_bits_to_f32(rq_zb[h]);
                bq_c[h] = -((WBITS == 4 ? 8.f : 128.f) + bq_z[h]) * bq_s[h];
                whole_zp = whole_zp && bf16_zp_is_whole(bq_z[h]);
            } else {
                rq_s[h] = pair_of_f16_bits(rq_sb[h]);
                rq_z[h] = pair_of_f16_bits(rq_zb[h]);
            }
        }
        if constexpr (RQBF && REFQ == 2) whole_zp = __builtin_amdgcn_ballot_w64(!whole_zp) == 0;
    }

    for (int e = threadIdx.x; e < ZERO_BYTES / 4; e += kDecWaves * 64) ((uint32_t*)smem)[e] = 0;
    // Fill LDS in batches: all loads of a batch are issued before the first store, so a batch
    // costs one memory latency (a load-store loop would pay it once per element).
    constexpr int NT = kDecWaves * 64;
    const int chunks = p.K / 8;   // 16-byte pieces per activation row
    // the first batch of activations is asked for before the scale tables are filled, so that the two
    // fills cost one memory latency between them, not one each (a decode launch is a handful of latencies)
    v4u v_first[4];
    {
        const v4u* src = (const v4u*)p.act;
#pragma unroll
        for (int u = 0; u < 4; ++u) v_first[u] = src[min(u * NT + (int)threadIdx.x, chunks - 1)];
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!REFQ) {
        if (p.scale_dtype == FNN_F16) fill_scales_lds<FNN_F16, NC>(s_lds, z_lds, p, n0, ngroups, c_off, threadIdx.x, NT);
        else fill_scales_lds<FNN_BF16, NC>(s_lds, z_lds, p, n0, ngroups, c_off, threadIdx.x, NT);
    }
    if constexpr (RQG) {
        // (scale | zero point << 16) of group g, channel c at word g * NC + c; loads in batches of four
        uint32_t* const tab = (uint32_t*)s_lds;
        const int total = ngroups * NC;
        for (int e0 = 0; e0 < total; e0 += 4 * NT) {
            uint32_t sv[4], zv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = min(e0 + u * NT + (int)threadIdx.x, total - 1);
                const int64_t idx = (int64_t)(e / NC) * p.N + min(n0 + e % NC, p.N - 1);
                sv[u] = ((const uint16_t*)p.scale)[idx];
                zv[u] = RQZ ? (uint32_t)((const uint16_t*)p.zp)[idx] : 0u;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = e0 + u * NT + threadIdx.x;
                if (e < total) tab[e] = sv[u] | (zv[u] << 16);
            }
        }
    }
    {
        for (int m = 0; m < p.M; ++m) {
            const v4u* src = (const v4u*)((const uint16_t*)p.act + (int64_t)m * p.lda);
            v4u* dst = (v4u*)(a_lds + m * a_stride);
            for (int c0 = 0; c0 < chunks; c0 += 4 * NT) {
                v4u v[4];
                const bool first = m == 0 && c0 == 0;   // uniform
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    v[u] = first ? v_first[u] : src[min(c0 + u * NT + (int)threadIdx.x, chunks - 1)];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int c = c0 + u * NT + threadIdx.x;
                    if (c < chunks) dst[c] = WBITS == 4 ? perm_act_w4(v[u]) : v[u];
                }
            }
        }
    }
    __syncthreads();

    // B-operand source of this lane: column j7 = gslot*MP + m
    const int m_col = G128 ? (j7 % MP) : j7;
    const int gslot = G128 ? (j7 / MP) : 0;
    const bool col_valid = m_col < p.M;
    bool use[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) use[i] = col_valid && (i % GS) == gslot;
    const int koff = lg * 32 + half * 16;
    // byte addresses in LDS; step s adds s*256
    uint32_t a_real = (uint32_t)((const char*)(a_lds + m_col * a_stride + koff) - smem) + s_begin * 256;
    const uint32_t a_zero = 0;
    uint32_t sz_addr = (uint32_t)((const char*)(s_lds + (s_begin + gslot) * (G128 ? NC : 0) + NH * 4 * (lg & 1)) - smem);
    const uint32_t z_delta = (uint32_t)(ngroups * NC * 4);

    // RQG: word address of this lane's table entries at step 0 (group of its K segment, its weight row's
    // channels); a step adds 128 / group groups
    const int rqg_gps = RQG ? 128 / p.group : 0;
    const uint32_t rqg_base = RQG ? (uint32_t)((const char*)s_lds - smem) +
                                        (uint32_t)(((lg * 32 + half * 16) / (RQG ? p.group : 1)) * NC + j7 * NH) * 4u : 0u;
    const uint32_t rqg_step = (uint32_t)(rqg_gps * NC * 4);

    v4f outv[NH], accg[NH], asum;
#pragma unroll
    for (int h = 0; h < NH; ++h) { outv[h] = v4f{0, 0, 0, 0}; accg[h] = v4f{0, 0, 0, 0}; }
    asum = v4f{0, 0, 0, 0};
    const v4f zero4 = v4f{0, 0, 0, 0};

    auto fold = [&](uint32_t addr) {
        if constexpr (REFQ) {
#pragma unroll
            for (int h = 0; h < NH; ++h) outv[h] = accg[h];
            return;
        }
        float sv[NH * 4], zv[NH * 4];
#pragma unroll
        for (int q = 0; q < NH; ++q) {
            const v4f a = *(const v4f*)(smem + addr + q * 16);
            const v4f b = *(const v4f*)(smem + addr + z_delta + q * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) { sv[q * 4 + e] = a[e]; zv[q * 4 + e] = b[e]; }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int h = 0; h < NH; ++h)
                outv[h][r] += sv[NH * r + h] * accg[h][r] - zv[NH * r + h] * asum[r];
    };

    // The K range of a wave is processed in chunks of CH steps.  A chunk is straight-line code:
    // UN loads are in flight at its start, steps 0..CH-UN-1 each issue the load UN steps ahead,
    // so the wait counts are exact and nothing is carried over a loop edge in registers.
    const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
    auto run = [&](auto one_step_tag) {
    constexpr bool ONE_STEP = decltype(one_step_tag)::value;
    for (int sb = s_begin; sb < s_end; sb += CH) {
        if (sb != s_begin) {
#pragma unroll
            for (int i = 0; i < UN; ++i) wq[i] = load_w(sb + i);
        }
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const int step = sb + i;
            if (FULL || step < s_end) {
                const v4u w = wq[i % UN];
                const uint32_t aa = (use[i % 8] ? a_real : a_zero) + i * 256;
                const v4u a0 = *(const v4u*)(smem + aa);
                const v4u a1 = *(const v4u*)(smem + aa + 16);
                const bool first = G128 ? (i % GS == 0) : (step == s_begin);
                if constexpr (RQG) {
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        const uint32_t t = *(const uint32_t*)(smem + rqg_base + (uint32_t)step * rqg_step + h * 4);
                        rq_s[h] = pair_of_f16_bits(t);
                        rq_z[h] = pair_of_f16_bits(t >> 16);
                    }
                }
                if constexpr (WBITS == 4) {
                    v4u e0, e1, o0, o1;
                    if constexpr (RQBF) dq_w4_bf16<false, ONE_STEP>(w, bq_s, bq_z, bq_c, e0, e1, o0, o1);
                    else convert_w4<ADT>(w, e0, e1, o0, o1);
                    // refill the queue slot only after its old value is dead, so that both live
                    // in the same registers
                    if (i + UN < CH) wq[i % UN] = load_w(step + UN);
                    if constexpr (REFQ != 0 && !RQBF) {
                        e0 = ref_dq_f16<RQZ>(e0, rq_c, rq_z[0], rq_s[0]);
                        e1 = ref_dq_f16<RQZ>(e1, rq_c, rq_z[0], rq_s[0]);
                        o0 = ref_dq_f16<RQZ>(o0, rq_c, rq_z[NH - 1], rq_s[NH - 1]);
                        o1 = ref_dq_f16<RQZ>(o1, rq_c, rq_z[NH - 1], rq_s[NH - 1]);
                    }
                    accg[0] = MT::mma(e0, a0, first ? zero4 : accg[0]);
                    accg[1] = MT::mma(o0, a0, first ? zero4 : accg[1]);
                    if constexpr (!REFQ) asum = MT::mma(ones, a0, first ? zero4 : asum);
                    accg[0] = MT::mma(e1, a1, accg[0]);
                    accg[1] = MT::mma(o1, a1, accg[1]);
                    if constexpr (!REFQ) asum = MT::mma(ones, a1, asum);
                } else {
                    v4u s0, s1;
                    if constexpr (RQBF) dq_w8_bf16<ONE_STEP>(w, bq_s[0], bq_z[0], bq_c[0], s0, s1);
                    else convert_w8<ADT>(w, s0, s1);
                    if (i + UN < CH) wq[i % UN] = load_w(step + UN);
                    if constexpr (REFQ != 0 && !RQBF) {
                        s0 = ref_dq_f16<RQZ>(s0, rq_c, rq_z[0], rq_s[0]);
                        s1 = ref_dq_f16<RQZ>(s1, rq_c, rq_z[0], rq_s[0]);
                    }
                    accg[0] = MT::mma(s0, a0, first ? zero4 : accg[0]);
                    if constexpr (!REFQ) asum = MT::mma(ones, a0, first ? zero4 : asum);
                    accg[0] = MT::mma(s1, a1, accg[0]);
                    if constexpr (!REFQ) asum = MT::mma(ones, a1, asum);
                }
                if constexpr (G128) {
                    if (i % GS == GS - 1 || (!FULL && step + 1 == s_end))
                        fold(sz_addr + (i / GS) * GS * NC * 4);
                }
            }
            // keep every step's refill load inside its step: the scheduler would otherwise
            // sink the loads to shorten their live ranges and empty the queue
            __builtin_amdgcn_sched_barrier(0);
        }
        a_real += CH * 256;
        if constexpr (G128) sz_addr += CH * NC * 4;
    }
    };
    if constexpr (RQBF && REFQ == 2) {
        if (whole_zp) run(std::true_type{});
        else run(std::false_type{});
    } else {
        run(std::true_type{});
    }
    if constexpr (!G128) {
        if (s_begin < s_end) fold(sz_addr);
    }

#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((wave * NH + h) * 4 + r) * 64 + lane] = outv[h][r];
    __syncthreads();
    for (int e = threadIdx.x; e < p.M * NC; e += kDecWaves * 64) {
        const int m = e / NC, c = e % NC;
        const int row = c / NH, h = c % NH;
        const int r = row & 3;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kDecWaves; ++w)
#pragma unroll
            for (int gs = 0; gs < GS; ++gs) {
                const int col = gs * (G128 ? MP : 0) + m;
                const int lane1 = col + 16 * (row >> 2);
                const int lane2 = (col + 8) + 16 * ((row + 8) >> 2);
                v += red[((w * NH + h) * 4 + r) * 64 + lane1] + red[((w * NH + h) * 4 + r) * 64 + lane2];
            }
        const int n = n0 + c;
        if (n < p.N) {
            if (p.bias) v = add_bias<WBITS>(v, load_as_f32(p.bias, n, p.bias_dtype), p.out_dtype);
            store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
        }
    }
}


// ------------------------------------------------ GEMV kernel: one wave streams one tile
// For many output channels (tiles >= 4 x CUs) the K split across waves is dropped: a
// workgroup has one wave per tile of 8 weight rows, each wave walks the whole K range of its
// tile with UN 16-byte loads in flight, and the grid is sized to one workgroup per CU
// (N = 28672 int4 channels: 1792 tiles = 256 workgroups x 7 waves).  Long streams keep the
// load queue full for the whole kernel, there is no cross-wave reduction, and every CU gets
// the same number of bytes.  Activations (M <= 4 rows) are staged in LDS once per workgroup,
// the scales of a tile once per wave; the MFMA layout, the group slots and the integer
// conversion are those of gemm_wo_decode_lds_kernel.
constexpr int kGemvMaxWaves = 8;

template <int WBITS, int ADT, bool G128, int MP, int UN, bool FULL>
__global__ __launch_bounds__(kGemvMaxWaves * 64) void gemm_wo_gemv_kernel(const WoArgs p, const int wpw) {
    typedef MfmaT<ADT> MT;
    constexpr int NH = WBITS == 4 ? 2 : 1;
    constexpr int NC = 8 * NH;
    constexpr int GS = G128 ? 8 / MP : 1;
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int half = li >> 3;
    const int j7 = li & 7;

    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = (wrows + 7) / 8;
    const int tile = blockIdx.x * wpw + wave;
    const bool tile_ok = tile < tiles;           // wave-uniform
    const int row0 = min(tile, tiles - 1) * 8;
    const int n0 = row0 * NH;

    const int steps = p.K / 128;
    const int ngroups = G128 ? steps : 1;

    // LDS: [32 B of zeros][activations M x (K+32)][per wave: scale, zoff (ngroups*NC f32 each)]
    const int a_stride = p.K + 32;
    uint16_t* a_lds = (uint16_t*)(smem + 32);
    float* s_lds = (float*)(smem + 32 + (size_t)p.M * a_stride * 2) + (size_t)wave * ngroups * NC * 2;
    float* z_lds = s_lds + ngroups * NC;

    const int wrow_l = min(row0 + j7, wrows - 1) - row0;
    const uint32_t w_off = (uint32_t)wrow_l * (uint32_t)p.ldw + lg * 32 + half * 16;
    const char* w_tile = (const char*)p.qw + (int64_t)row0 * p.ldw;
    auto load_w = [&](int step) -> v4u {
        const char* base = w_tile + (int64_t)min(step, steps - 1) * 128;   // scalar
        return __builtin_nontemporal_load((const v4u*)(base + w_off));
    };
    // ---- start-up: every load is issued before the first wait ----
    // The small tables go first (vector memory returns in order): scales and zero points of the
    // tile, the activation rows, then the first UN weight pieces.  The tables are written to LDS
    // while the weight loads are still in flight.
    constexpr int VPR = NC / 8;   // 16-byte pieces per scale row of the tile
    constexpr int SB = 2;         // scale batches staged in registers
    constexpr int AB = 4;         // activation batches per row staged in registers
    const int nvec = ngroups * VPR;
    const int chunks = p.K / 8;
    const int nt = blockDim.x;
    const bool has_zp = p.zp != nullptr;
    const uint16_t* zp_tab = has_zp ? (const uint16_t*)p.zp : (const uint16_t*)p.scale;
    v4u sv[SB], zv[SB];
#pragma unroll
    for (int u = 0; u < SB; ++u) {
        const int e = min(u * 64 + lane, nvec - 1);
        const int64_t off = (int64_t)(e / VPR) * p.N + n0 + (e % VPR) * 8;
        sv[u] = *(const v4u*)((const uint16_t*)p.scale + off);
        zv[u] = *(const v4u*)(zp_tab + off);
    }
    constexpr int MROWS = G128 ? (MP < 4 ? MP : 4) : 4;   // activation rows staged (M <= MROWS)
    v4u av[MROWS][AB];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
        const v4u* src = (const v4u*)((const uint16_t*)p.act + (int64_t)min(m, p.M - 1) * p.lda);
#pragma unroll
        for (int u = 0; u < AB; ++u) {
            // batches beyond the row length are skipped (uniform), not clamped: a clamped batch would
            // still cost the copy unit a full instruction per wave
            if (u * nt < chunks) av[m][u] = src[min(u * nt + (int)threadIdx.x, chunks - 1)];
            else av[m][u] = v4u{0, 0, 0, 0};
        }
    }
    v4u wq[UN];
#pragma unroll
    for (int i = 0; i < UN; ++i) wq[i] = load_w(i);

    if (threadIdx.x < 8) ((uint32_t*)smem)[threadIdx.x] = 0;
    const bool s_f16 = p.scale_dtype == FNN_F16;
#pragma unroll
    for (int u = 0; u < SB; ++u) {
        const int e = u * 64 + lane;
        if (e < nvec) {
            float sc[8], zo[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t sb = (sv[u][j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                const uint32_t zb = (zv[u][j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                sc[j] = s_f16 ? f16_bits_to_f32(sb) : bf16_bits_to_f32(sb);
                const float z = s_f16 ? f16_bits_to_f32(zb) : bf16_bits_to_f32(zb);
                zo[j] = sc[j] * (c_off + (has_zp ? z : 0.f));
            }
            float* sd = s_lds + (e / VPR) * NC + (e % VPR) * 8;
            float* zd = z_lds + (e / VPR) * NC + (e % VPR) * 8;
            *(v4f*)sd = v4f{sc[0], sc[1], sc[2], sc[3]};
            *(v4f*)(sd + 4) = v4f{sc[4], sc[5], sc[6], sc[7]};
            *(v4f*)zd = v4f{zo[0], zo[1], zo[2], zo[3]};
            *(v4f*)(zd + 4) = v4f{zo[4], zo[5], zo[6], zo[7]};
        }
    }
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
        v4u* dst = (v4u*)(a_lds + m * a_stride);
#pragma unroll
        for (int u = 0; u < AB; ++u) {
            const int c = u * nt + threadIdx.x;
            if (m < p.M && c < chunks) dst[c] = WBITS == 4 ? perm_act_w4(av[m][u]) : av[m][u];
        }
    }
    // whatever did not fit the staged batches (very long K)
    if (nvec > SB * 64) {
        float* so = s_lds + SB * 64 / VPR * NC;
        float* zo = z_lds + SB * 64 / VPR * NC;
        WoArgs q = p;
        q.scale = (const uint16_t*)p.scale + (int64_t)(SB * 64 / VPR) * p.N;
        if (has_zp) q.zp = (const uint16_t*)p.zp + (int64_t)(SB * 64 / VPR) * p.N;
        if (s_f16) fill_scales_lds<FNN_F16, NC>(so, zo, q, n0, ngroups - SB * 64 / VPR, c_off, lane, 64);
        else fill_scales_lds<FNN_BF16, NC>(so, zo, q, n0, ngroups - SB * 64 / VPR, c_off, lane, 64);
    }
    if (chunks > AB * nt) {
        for (int m = 0; m < p.M; ++m) {
            const v4u* src = (const v4u*)((const uint16_t*)p.act + (int64_t)m * p.lda);
            v4u* dst = (v4u*)(a_lds + m * a_stride);
            for (int c = AB * nt + threadIdx.x; c < chunks; c += nt)
                dst[c] = WBITS == 4 ? perm_act_w4(src[c]) : src[c];
        }
    }
    __syncthreads();

    const int m_col = G128 ? (j7 % MP) : j7;
    const int gslot = G128 ? (j7 / MP) : 0;
    const bool col_valid = m_col < p.M;
    bool use[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) use[i] = col_valid && (i % GS) == gslot;
    const int koff = lg * 32 + half * 16;
    uint32_t a_real = (uint32_t)((const char*)(a_lds + m_col * a_stride + koff) - smem);
    uint32_t sz_addr = (uint32_t)((const char*)(s_lds + gslot * (G128 ? NC : 0) + NH * 4 * (lg & 1)) - smem);
    const uint32_t z_delta = (uint32_t)(ngroups * NC * 4);

    v4f outv[NH], accg[NH], asum;
#pragma unroll
    for (int h = 0; h < NH; ++h) { outv[h] = v4f{0, 0, 0, 0}; accg[h] = v4f{0, 0, 0, 0}; }
    asum = v4f{0, 0, 0, 0};
    const v4f zero4 = v4f{0, 0, 0, 0};

    auto fold = [&](uint32_t addr) {
        float sv[NH * 4], zv[NH * 4];
#pragma unroll
        for (int q = 0; q < NH; ++q) {
            const v4f a = *(const v4f*)(smem + addr + q * 16);
            const v4f b = *(const v4f*)(smem + addr + z_delta + q * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) { sv[q * 4 + e] = a[e]; zv[q * 4 + e] = b[e]; }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int h = 0; h < NH; ++h)
                outv[h][r] += sv[NH * r + h] * accg[h][r] - zv[NH * r + h] * asum[r];
    };

    // Queue slots are refilled BURST at a time, after the last of them has been consumed (so old
    // and new value share registers): DRAM then sees 8 rows x BURST*128 contiguous bytes per
    // burst instead of single 128-byte pieces, which keeps more of its row buffers useful.
    constexpr int BURST = UN >= 16 ? 4 : 1;
    auto refill = [&](int i, int sb) {
        if (i % BURST == BURST - 1) {
#pragma unroll
            for (int b = 0; b < BURST; ++b) wq[i - (BURST - 1) + b] = load_w(sb + i - (BURST - 1) + b + UN);
        }
    };
    const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
    for (int sb = 0; sb < steps; sb += UN) {
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const int step = sb + i;
            if (FULL || step < steps) {
                const v4u w = wq[i];
                const uint32_t aa = use[i % 8] ? a_real + i * 256 : 0u;
                const v4u a0 = *(const v4u*)(smem + aa);
                const v4u a1 = *(const v4u*)(smem + aa + 16);
                const bool first = G128 ? (i % GS == 0) : (step == 0);
                if constexpr (WBITS == 4) {
                    v4u e0, e1, o0, o1;
                    convert_w4<ADT>(w, e0, e1, o0, o1);
                    refill(i, sb);
                    accg[0] = MT::mma(e0, a0, first ? zero4 : accg[0]);
                    accg[1] = MT::mma(o0, a0, first ? zero4 : accg[1]);
                    asum = MT::mma(ones, a0, first ? zero4 : asum);
                    accg[0] = MT::mma(e1, a1, accg[0]);
                    accg[1] = MT::mma(o1, a1, accg[1]);
                    asum = MT::mma(ones, a1, asum);
                } else {
                    v4u s0, s1;
                    convert_w8<ADT>(w, s0, s1);
                    refill(i, sb);
                    accg[0] = MT::mma(s0, a0, first ? zero4 : accg[0]);
                    asum = MT::mma(ones, a0, first ? zero4 : asum);
                    accg[0] = MT::mma(s1, a1, accg[0]);
                    asum = MT::mma(ones, a1, asum);
                }
                if constexpr (G128) {
                    if (i % GS == GS - 1 || (!FULL && step + 1 == steps))
                        fold(sz_addr + (i / GS) * GS * NC * 4);
                }
            }
            __builtin_amdgcn_sched_barrier(0);   // keep each refill load inside its step
        }
        a_real += UN * 256;
        if constexpr (G128) sz_addr += UN * NC * 4;
    }
    if constexpr (!G128) fold(sz_addr);

    // ---- per-wave reduction of the group-slot columns and the two diagonal blocks ----
    // the wave's own scale area is free now and private to it
    float* red = s_lds;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[(h * 4 + r) * 64 + lane] = outv[h][r];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): this wave's LDS writes are done
    for (int e = lane; e < p.M * NC; e += 64) {
        const int m = e / NC, c = e % NC;
        const int row = c / NH, h = c % NH;
        const int r = row & 3;
        float v = 0.f;
#pragma unroll
        for (int gs = 0; gs < GS; ++gs) {
            const int col = gs * (G128 ? MP : 0) + m;
            const int lane1 = col + 16 * (row >> 2);
            const int lane2 = (col + 8) + 16 * ((row + 8) >> 2);
            v += red[(h * 4 + r) * 64 + lane1] + red[(h * 4 + r) * 64 + lane2];
        }
        const int n = n0 + c;
        if (tile_ok && n < p.N) {
            if (p.bias) v = add_bias<WBITS>(v, load_as_f32(p.bias, n, p.bias_dtype), p.out_dtype);
            store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
        }
    }
}

// ------------------------------------------------ GEMV kernel, flattened: eight equal chunks per CU
// One wave per tile leaves a CU with as many waves as it has tiles - seven at N = 28672 int4 channels, on
// four SIMDs: three SIMDs carry two streams and one carries one, and the kernel ends when the doubled-up
// ones do.  Here the wpw tiles of a workgroup times the K/128 steps of a tile are one sequence of
// wpw * steps steps, cut into eight equal, contiguous chunks, one per wave: two waves on every SIMD, each
// with the same number of bytes to stream.  A chunk is at most one tile long, so it covers the end of one
// tile and the beginning of the next; the two partial results are kept apart, written to LDS, and the
// parts of every tile are added in ascending K order by one wave (a fixed order: the result does not
// depend on timing).  Chunks, tiles and the 8-step blocks of the group slots all begin at multiples of
// eight steps (checked on the host), so a block never straddles two tiles.  Group size 128, M <= 4.
//
// Start-up is a matter of how many cache lines the CU has to ask for before the first weights arrive.  The
// scale and zero-point tables are [K/128][N]: the 16 channels of one tile are 32 bytes of each row, so a
// wave fetching its own tile's tables asks for one line per group and table (the wpw tiles of a workgroup
// for the same lines again).  The workgroup's tiles are neighbours, so it fetches the tables of all of
// them together instead, wpw * 32 contiguous bytes per row, with all its threads, into one shared LDS
// table: an eighth of the requests.
//
// A wave executes about one instruction every 2 ns here, so what stands between the kernel's start and its
// first loads is kept short: where a chunk begins (tile and step) and which chunks make up a tile are
// worked out on the host and passed as packed 4-bit fields, the weight loads are issued first, and the
// tables are fetched by 16 lanes per row, which needs no division.  fp16 tables only.
struct GemvFlatPlan {
    uint32_t tA;      // 4 bits per wave: the tile (of the workgroup) its chunk begins in
    uint32_t sA8;     // 4 bits per wave: the step it begins at, in units of 8
    uint32_t len8;    // 4 bits per wave: the length of its chunk, in units of 8 steps
    uint32_t wfirst;  // 4 bits per tile: the first chunk that overlaps it
    uint32_t wlast;   // 4 bits per tile: the last one
};

template <int WBITS, int ADT, int MP>
__global__ __launch_bounds__(512) void gemm_wo_gemv_flat_kernel(const WoArgs p, const int wpw, const GemvFlatPlan plan) {
    typedef MfmaT<ADT> MT;
    constexpr int NH = WBITS == 4 ? 2 : 1;
    constexpr int NC = 8 * NH;
    constexpr int GS = 8 / MP;
    constexpr int UN = 8;
    constexpr int NW = 8;
    constexpr int nt = NW * 64;
    constexpr float c_off = WBITS == 4 ? (ADT == FNN_F16 ? 1024.f + 8.f : 128.f + 8.f)
                                       : (ADT == FNN_F16 ? 1024.f + 128.f : 128.f);
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int half = li >> 3;
    const int j7 = li & 7;

    const int steps = p.K / 128;
    const int chunk = ((plan.len8 >> (4 * wave)) & 15) * 8;   // steps of this wave, a multiple of 8, at most `steps`
    const int tA = (plan.tA >> (4 * wave)) & 15;   // the chunk begins in tile tA of the workgroup, at step sA
    const int sA = ((plan.sA8 >> (4 * wave)) & 15) * 8;
    const int len1 = min(chunk, steps - sA);       // steps in tile tA; the other chunk - len1 are in tile tA + 1
    // workgroups id, id + 8, id + 16 .. share an XCD and its L2: they take neighbouring tiles, whose table rows
    // share cache lines (a tile's 32 bytes of a table row are a quarter of a line)
    const int per_xcd = gridDim.x >> 3;            // the grid is a multiple of 8 (host-checked)
    const int tile0 = ((blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3)) * wpw;

    // LDS: [32 B of zeros][activations M x (K+32)][per wave: 2 x (scale, zoff) of 8 groups x NC f32][parts 8 x 2 x PART f32]
    constexpr int PART = NH * 4 * 64;              // floats of one partial result
    constexpr int TBLK = 8 * NC;                   // floats of one table of one block of eight groups
    const int a_stride = p.K + 32;
    uint16_t* a_lds = (uint16_t*)(smem + 32);
    float* const tabs = (float*)(smem + 32 + (size_t)p.M * a_stride * 2);
    float* const my_tab = tabs + wave * (4 * TBLK);            // [parity][scale | zoff][8 groups][NC]
    float* const parts = tabs + NW * 4 * TBLK;

    const uint32_t w_off = (uint32_t)j7 * (uint32_t)p.ldw + lg * 32 + half * 16;
    const char* const wA = (const char*)p.qw + (int64_t)(tile0 + tA) * 8 * p.ldw + (int64_t)sA * 128;
    const char* const wB = (const char*)p.qw + (int64_t)(tile0 + tA + 1) * 8 * p.ldw - (int64_t)len1 * 128;
    auto load_w = [&](int f) -> v4u {
        const int g = min(f, chunk - 1);
        const char* base = (g < len1 ? wA : wB) + (int64_t)g * 128;   // scalar
        return __builtin_nontemporal_load((const v4u*)(base + w_off));
    };
    // ---- tables: the scales and zero points of a block of eight steps (eight groups x the tile's NC
    // channels: 2 x 16-byte pieces per group and table) are fetched one block ahead by 16 lanes of the wave,
    // converted, and passed to the fold through a wave-private LDS area - no staging of whole tables at the
    // start (a burst of small scattered requests in front of the weight stream), no barrier.
    const bool has_zp = p.zp != nullptr;
    const uint16_t* zp_src = has_zp ? (const uint16_t*)p.zp : (const uint16_t*)p.scale;
    const float zmul = has_zp ? 1.f : 0.f;
    const uint32_t tab_lane = (uint32_t)((lane / (NC / 8)) & 7) * (uint32_t)p.N * 2 + (lane % (NC / 8)) * 16;   // bytes: group row, piece
    auto load_tabs = [&](int sb, v4u& sv, v4u& zv) {   // block of steps sb .. sb + 7 of the chunk (clamped)
        const int b = min(sb, chunk - 8);
        const int tile = tile0 + tA + (b < len1 ? 0 : 1);
        const int grp = b < len1 ? sA + b : b - len1;
        const int64_t off = ((int64_t)grp * p.N + (int64_t)tile * NC) * 2;        // scalar, bytes
        sv = *(const v4u*)((const char*)p.scale + off + tab_lane);
        zv = *(const v4u*)((const char*)zp_src + off + tab_lane);
    };
    auto stage_tabs = [&](int parity, const v4u sv, const v4u zv) {
        {
            float sc[8], zo[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t sb = (sv[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                const uint32_t zb = (zv[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                sc[j] = f16_bits_to_f32(sb);
                zo[j] = sc[j] * (c_off + zmul * f16_bits_to_f32(zb));
            }
            if (lane < 8 * (NC / 8)) {             // 8 groups x NC / 8 pieces
                float* sd = my_tab + parity * 2 * TBLK + (lane / (NC / 8)) * NC + (lane % (NC / 8)) * 8;
                float* zd = sd + TBLK;
                *(v4f*)sd = v4f{sc[0], sc[1], sc[2], sc[3]};
                *(v4f*)(sd + 4) = v4f{sc[4], sc[5], sc[6], sc[7]};
                *(v4f*)zd = v4f{zo[0], zo[1], zo[2], zo[3]};
                *(v4f*)(zd + 4) = v4f{zo[4], zo[5], zo[6], zo[7]};
            }
        }
    };
    // ---- start-up: every load is issued before the first wait, in the order in which the data is needed
    // (loads return in order): the activations, which every wave needs at its first step and which come from
    // the L2; the tables of the first block; the first UN weight pieces.  One bare barrier (a __syncthreads()
    // would wait for every load in flight) publishes the activations.
    constexpr int AB = 4;
    const int chunks = p.K / 8;
    constexpr int MROWS = MP < 4 ? MP : 4;
    v4u av[MROWS][AB];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
        const v4u* src = (const v4u*)((const uint16_t*)p.act + (int64_t)min(m, p.M - 1) * p.lda);
#pragma unroll
        for (int u = 0; u < AB; ++u) {
            if (u * nt < chunks) av[m][u] = src[min(u * nt + (int)threadIdx.x, chunks - 1)];
            else av[m][u] = v4u{0, 0, 0, 0};
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    v4u tsv, tzv;
    load_tabs(0, tsv, tzv);
    __builtin_amdgcn_sched_barrier(0);
    v4u wq[UN];
#pragma unroll
    for (int i = 0; i < UN; ++i) wq[i] = load_w(i);
    __builtin_amdgcn_sched_barrier(0);

    if (threadIdx.x < 8) ((uint32_t*)smem)[threadIdx.x] = 0;
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
        v4u* dst = (v4u*)(a_lds + m * a_stride);
#pragma unroll
        for (int u = 0; u < AB; ++u) {
            const int c = u * nt + threadIdx.x;
            if (m < p.M && c < chunks) dst[c] = WBITS == 4 ? perm_act_w4(av[m][u]) : av[m][u];
        }
    }
    // (K <= AB * 512 * 8 = 16384 is checked on the host: the staged batches hold a whole row)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);            // lgkmcnt(0): this wave's LDS writes are done
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    const int m_col = j7 % MP;
    const int gslot = j7 / MP;
    const bool col_valid = m_col < p.M;
    bool use[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) use[i] = col_valid && (i % GS) == gslot;
    const int koff = lg * 32 + half * 16;
    const uint32_t a_base = (uint32_t)((const char*)(a_lds + m_col * a_stride + koff) - smem);
    uint32_t a_real = a_base + sA * 256;
    // table entry of (group slot, this lane's channels) in the wave's area of the current block
    constexpr uint32_t rowb = NC * 4;              // bytes of a table row
    const uint32_t sz_lane = (uint32_t)((const char*)(my_tab + NH * 4 * (lg & 1)) - smem) + gslot * rowb;
    constexpr uint32_t z_delta = TBLK * 4;

    v4f outv[NH], outA[NH], accg[NH], asum;
#pragma unroll
    for (int h = 0; h < NH; ++h) { outv[h] = v4f{0, 0, 0, 0}; outA[h] = v4f{0, 0, 0, 0}; accg[h] = v4f{0, 0, 0, 0}; }
    asum = v4f{0, 0, 0, 0};
    const v4f zero4 = v4f{0, 0, 0, 0};

    auto fold = [&](uint32_t addr) {
        float sv[NH * 4], zv[NH * 4];
#pragma unroll
        for (int q = 0; q < NH; ++q) {
            const v4f a = *(const v4f*)(smem + addr + q * 16);
            const v4f b = *(const v4f*)(smem + addr + z_delta + q * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) { sv[q * 4 + e] = a[e]; zv[q * 4 + e] = b[e]; }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int h = 0; h < NH; ++h)
                outv[h][r] += sv[NH * r + h] * accg[h][r] - zv[NH * r + h] * asum[r];
    };

    const v4u ones = v4u{MT::one2, MT::one2, MT::one2, MT::one2};
    int parity = 0;
    for (int sb = 0; sb < chunk; sb += UN) {
        if (sb == len1) {   // the chunk moves on to the next tile: a new result, K starts over
#pragma unroll
            for (int h = 0; h < NH; ++h) { outA[h] = outv[h]; outv[h] = v4f{0, 0, 0, 0}; }
            a_real = a_base;
        }
        // this block's tables go to LDS (the area of the block before last is free: LDS operations of a
        // wave complete in order), the next block's are requested
        stage_tabs(parity, tsv, tzv);
        load_tabs(sb + UN, tsv, tzv);
        const uint32_t sz_addr = sz_lane + parity * (2 * TBLK * 4);
        parity ^= 1;
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const v4u w = wq[i];
            const uint32_t aa = use[i % 8] ? a_real + i * 256 : 0u;
            const v4u a0 = *(const v4u*)(smem + aa);
            const v4u a1 = *(const v4u*)(smem + aa + 16);
            const bool first = i % GS == 0;
            if constexpr (WBITS == 4) {
                v4u e0, e1, o0, o1;
                convert_w4<ADT>(w, e0, e1, o0, o1);
                wq[i] = load_w(sb + i + UN);
                accg[0] = MT::mma(e0, a0, first ? zero4 : accg[0]);
                accg[1] = MT::mma(o0, a0, first ? zero4 : accg[1]);
                asum = MT::mma(ones, a0, first ? zero4 : asum);
                accg[0] = MT::mma(e1, a1, accg[0]);
                accg[1] = MT::mma(o1, a1, accg[1]);
                asum = MT::mma(ones, a1, asum);
            } else {
                v4u s0, s1;
                convert_w8<ADT>(w, s0, s1);
                wq[i] = load_w(sb + i + UN);
                accg[0] = MT::mma(s0, a0, first ? zero4 : accg[0]);
                asum = MT::mma(ones, a0, first ? zero4 : asum);
                accg[0] = MT::mma(s1, a1, accg[0]);
                asum = MT::mma(ones, a1, asum);
            }
            if (i % GS == GS - 1) fold(sz_addr + (i / GS) * GS * rowb);
            __builtin_amdgcn_sched_barrier(0);   // keep each refill load inside its step
        }
        a_real += UN * 256;
    }
    if (len1 == chunk) {   // (wave-uniform) the whole chunk lay in tile tA
#pragma unroll
        for (int h = 0; h < NH; ++h) { outA[h] = outv[h]; outv[h] = v4f{0, 0, 0, 0}; }
    }

    // ---- the group-slot columns of a result are added within the wave: column gs * MP + m of a half holds
    // activation row m, so a butterfly over the lane bits above log2(MP) leaves every lane of a half with
    // the sum for its m.  Then the two partial results go to LDS, part 0 = tile tA, part 1 = tile tA + 1.
    float* const mine = parts + (size_t)wave * 2 * PART;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float a = outA[h][r], b = outv[h][r];
#pragma unroll
            for (int o = MP; o < 8; o <<= 1) { a += __shfl_xor(a, o, 64); b += __shfl_xor(b, o, 64); }
            mine[(h * 4 + r) * 64 + lane] = a;
            mine[PART + (h * 4 + r) * 64 + lane] = b;
        }
    __syncthreads();
    // ---- wave t adds the parts of tile t in ascending K order and stores it: the chunks that overlap
    // steps [t * steps, (t + 1) * steps) of the workgroup's sequence, at most three
    if (wave >= wpw) return;
    const int t = wave;
    const int w_first = (plan.wfirst >> (4 * t)) & 15, w_last = (plan.wlast >> (4 * t)) & 15;
    const int n0 = (tile0 + t) * NC;
    if (lane < p.M * NC) {
        const int m = lane / NC, c = lane % NC;
        const int row = c / NH, h = c % NH;
        const int r = row & 3;
        // the two diagonal blocks of the MFMA result: columns 0..7 of lane rows 0..1, columns 8..15 of lane rows 2..3
        const int lane1 = m + 16 * (row >> 2);
        const int lane2 = (m + 8) + 16 * ((row + 8) >> 2);
        float v = 0.f;
        for (int w = w_first; w <= w_last; ++w) {
            const int tw = (plan.tA >> (4 * w)) & 15;   // the tile chunk w begins in: part 0 if it is t, else part 1
            const float* part = parts + (size_t)w * 2 * PART + (tw == t ? 0 : PART);
            v += part[(h * 4 + r) * 64 + lane1] + part[(h * 4 + r) * 64 + lane2];
        }
        const int n = n0 + c;
        if (p.bias) v = add_bias<WBITS>(v, load_as_f32(p.bias, n, p.bias_dtype), p.out_dtype);
        store_from_f32(p.out, (int64_t)m * p.ldc + n, v, p.out_dtype);
    }
}

// ------------------------------------------------------------------ guarded fallback
template <int WBITS, int ADT>
__global__ __launch_bounds__(256) void gemm_wo_any_kernel(const WoArgs p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * p.N) return;
    const int m = (int)(idx / p.N), n = (int)(idx % p.N);
    const uint16_t* a = (const uint16_t*)p.act + (int64_t)m * p.lda;
    const int8_t* w = p.qw + (int64_t)(WBITS == 4 ? n >> 1 : n) * p.ldw;
    const int g = p.group > 0 ? p.group : p.K;
    float total = 0.f;
    for (int k0 = 0; k0 < p.K; k0 += g) {
        const int64_t si = p.group > 0 ? (int64_t)(k0 / g) * p.N + n : n;
        const float sc = load_as_f32(p.scale, si, p.scale_dtype);
        const float z = p.zp ? load_as_f32(p.zp, si, p.zp_dtype) : 0.f;
        float part = 0.f;
        const int k1 = min(k0 + g, p.K);
        for (int k = k0; k < k1; ++k) {
            int q = w[k];
            if constexpr (WBITS == 4) q = (n & 1) ? (q >> 4) : ((int)((uint32_t)q << 28) >> 28);
            part += bits_to_f32<ADT>(a[k]) * ((float)q - z);
        }
        total += sc * part;
    }
    if (p.bias) total = add_bias<WBITS>(total, load_as_f32(p.bias, n, p.bias_dtype), p.out_dtype);
    store_from_f32(p.out, (int64_t)m * p.ldc + n, total, p.out_dtype);
}

// ------------------------------------------------------------------------ dispatch
template <int WBITS, int ADT, int MB>
static void launch_stream(WoArgs& p, hipStream_t st) {
    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = (wrows + 15) / 16;
    const dim3 grid(((tiles + 7) / 8) * 8), block(kWoWaves * 64);
    note_kernel("gemm_wo_stream_kernel", WBITS, MB, p.group);
    if (p.group == 32) gemm_wo_stream_kernel<WBITS, ADT, MB, true, true><<<grid, block, 0, st>>>(p);
    else if (p.group > 0) gemm_wo_stream_kernel<WBITS, ADT, MB, true><<<grid, block, 0, st>>>(p);
    else gemm_wo_stream_kernel<WBITS, ADT, MB, false><<<grid, block, 0, st>>>(p);
}

// the decode kernels keep a copy of the activation rows in LDS up to this size
constexpr size_t kDecodeActLdsBytes = 33 * 1024;

// gemv_only: take the one-wave-per-tile kernel or nothing; lds_only: nothing where the activations do not fit the
// kernel's LDS copy (the kernel without that copy is not wanted)
template <int WBITS, int ADT>
static bool launch_decode(WoArgs& p, hipStream_t st, bool gemv_only, bool lds_only = false) {
    constexpr int NH = WBITS == 4 ? 2 : 1;
    if (p.M > 8 || p.K % 128 != 0) return false;
    // groups of 32 or 64: only with fp16 activations and fp16 tables (every weight dequantised to fp16 first)
    const bool small_groups = (p.group == 32 || p.group == 64) && ADT == FNN_F16 && p.scale_dtype == FNN_F16 &&
                              (!p.zp || p.zp_dtype == FNN_F16);
    if (p.group > 0 && p.group % 128 != 0 && !small_groups) return false;
    const int ngroups = p.group > 0 ? p.K / p.group : 1;
    const size_t fixed = (size_t)ngroups * 8 * NH * 8 + (size_t)kDecWaves * NH * 4 * 64 * 4;
    if (fixed > 40 * 1024) return false;
    const size_t act_bytes = (size_t)p.M * (p.K + 32) * 2;
    const bool act_lds = act_bytes <= kDecodeActLdsBytes;
    const int wrows = WBITS == 4 ? p.N / 2 : p.N;
    const int tiles = (wrows + 7) / 8;
    const dim3 grid(((tiles + 7) / 8) * 8), block(kDecWaves * 64);
    p.m_base = 0;
    // the LDS-staged kernels read the scale tables in 16-byte pieces
    const bool tables16 = is16(p.scale_dtype) && (!p.zp || p.zp_dtype == p.scale_dtype) &&
                          p.N % (8 * NH) == 0 && ((uintptr_t)p.scale % 16) == 0 &&
                          (!p.zp || ((uintptr_t)p.zp % 16) == 0);
    // many tiles and group tables: one wave per tile, one workgroup per CU.  (With per-channel scales the
    // same organisation was measured slower than the K-split kernel below - A16W8 K=4096 N=11008 M=1: 12.5
    // against 10.7 us - so those shapes do not come here.)
    if (tables16 && p.group == 128 && p.M <= 4 && tiles >= 4 * 256) {
        int wpw = (tiles + 255) / 256;
        const int ngr = p.group > 0 ? p.K / 128 : 1;
        while (wpw > kGemvMaxWaves) wpw = (wpw + 1) / 2;
        const size_t need = 32 + act_bytes + (size_t)wpw * ngr * 8 * NH * 8;
        // ask for more than half of the 160 KB so that two workgroups never share a CU
        const size_t smem = need > 84 * 1024 ? need : 84 * 1024;
        // the wave's scale area doubles as its reduction scratch (NH*4*64 floats)
        if (need <= 150 * 1024 && (size_t)ngr * 8 * NH * 2 >= (size_t)NH * 4 * 64) {
            const dim3 g2((tiles + wpw - 1) / wpw), b2(wpw * 64);
            const bool full = (p.K / 128) % 8 == 0;
            // eight equal chunks per workgroup where the tiles do not already make eight waves of equal length
            {
                const int steps = p.K / 128;
                const int chunk = wpw * steps / 8;
                // zeros, activations, per wave two blocks of two fp32 tables (8 groups x the tile's channels), 16 partial results
                const size_t need_f = 32 + act_bytes + (size_t)8 * 4 * 8 * 8 * NH * 4 + (size_t)16 * NH * 4 * 64 * 4;
                const bool flat = wpw < 8 && p.M * 8 * NH <= 64 && wrows % 8 == 0 && tiles % wpw == 0 && steps % 8 == 0 &&
                                  (wpw * steps) % 64 == 0 && chunk <= steps && steps <= 64 && wpw * NH <= 16 && p.K <= 16384 &&
                                  p.scale_dtype == FNN_F16 && need_f <= 160 * 1024 && (tiles / wpw) % 8 == 0;
                if (flat) {
                    const size_t smem_f = need_f > 84 * 1024 ? need_f : 84 * 1024;
                    // The four waves a workgroup starts first are served first by their SIMDs and run ahead of the
                    // four that share those SIMDs; with equal chunks they finish a fifth earlier and the stream
                    // then runs on half the loads in flight.  Where the arithmetic allows it they get a seventh
                    // more steps than the others (64 and 48 of 448) and all eight finish together.
                    int len[8];
                    for (int w = 0; w < 8; ++w) len[w] = chunk;
                    if (chunk % 8 == 0 && chunk + 8 <= steps && chunk >= 16) {
                        for (int w = 0; w < 4; ++w) { len[w] = chunk + 8; len[w + 4] = chunk - 8; }
                    }
                    GemvFlatPlan plan{0, 0, 0, 0, 0};
                    int beg[9];
                    beg[0] = 0;
                    for (int w = 0; w < 8; ++w) {
                        const int ta = beg[w] / steps;
                        plan.tA |= (uint32_t)ta << (4 * w);
                        plan.sA8 |= (uint32_t)((beg[w] - ta * steps) / 8) << (4 * w);
                        plan.len8 |= (uint32_t)(len[w] / 8) << (4 * w);
                        beg[w + 1] = beg[w] + len[w];
                    }
                    for (int t = 0; t < wpw; ++t) {
                        int wf = 0, wl = 0;
                        for (int w = 0; w < 8; ++w) {
                            if (beg[w + 1] <= t * steps) wf = w + 1;
                            if (beg[w] < (t + 1) * steps) wl = w;
                        }
                        plan.wfirst |= (uint32_t)wf << (4 * t);
                        plan.wlast |= (uint32_t)wl << (4 * t);
                    }
#define FNN_GEMV_FLAT(MPV)                                                                                    \
    do {                                                                                                      \
        auto kfn = gemm_wo_gemv_flat_kernel<WBITS, ADT, MPV>;                                                  \
        static std::atomic<uint64_t> raised{0};                                                               \
        allow_large_lds((const void*)kfn, raised);                                                            \
        note_kernel("gemm_wo_gemv_flat_kernel", WBITS, MPV, wpw);                                             \
        kfn<<<g2, dim3(512), smem_f, st>>>(p, wpw, plan);                                                     \
    } while (0)
                    if (p.M == 1) FNN_GEMV_FLAT(1);
                    else if (p.M == 2) FNN_GEMV_FLAT(2);
                    else FNN_GEMV_FLAT(4);
#undef FNN_GEMV_FLAT
                    return true;
                }
            }
#define FNN_GEMV(G, MPV)                                                                                  \
    do {                                                                                                  \
        auto kfn = full ? gemm_wo_gemv_kernel<WBITS, ADT, G, MPV, 8, true>                               \
                        : gemm_wo_gemv_kernel<WBITS, ADT, G, MPV, 8, false>;                             \
        static std::atomic<uint64_t> raised[2] = {{0}, {0}};                                              \
        allow_large_lds((const void*)kfn, raised[full]);                                                  \
        note_kernel("gemm_wo_gemv_kernel", WBITS, MPV, wpw);                                              \
        kfn<<<g2, b2, smem, st>>>(p, wpw);                                                                \
    } while (0)
            if (p.M == 1) FNN_GEMV(true, 1);
            else if (p.M == 2) FNN_GEMV(true, 2);
            else FNN_GEMV(true, 4);
#undef FNN_GEMV
            return true;
        }
    }
    if (gemv_only) return false;
    // (the small-group tables are read element by element: any N, any alignment)
    if (act_lds && (small_groups || (tables16 && (p.group == 0 || p.group == 128)))) {
        const int steps = p.K / 128;
        const bool full16 = steps % (kDecWaves * 16) == 0, full8 = steps % (kDecWaves * 8) == 0;
        const size_t smem = fixed + act_bytes + 16 * 256 + 32;
        if (smem > 64 * 1024) return false;   // beyond what a launch may ask for without raising the kernel's limit
#define FNN_DEC(G, MPV, ...)                                                                         \
    do {                                                                                             \
        note_kernel(refq ? "gemm_wo_decode_lds_kernel(per-weight rounding)" : "gemm_wo_decode_lds_kernel", WBITS, MPV, \
                    full16 ? 16 : full8 ? 8 : -16);                                                  \
        if (full16) gemm_wo_decode_lds_kernel<WBITS, ADT, G, MPV, 16, true, ##__VA_ARGS__><<<grid, block, smem, st>>>(p); \
        else if (full8) gemm_wo_decode_lds_kernel<WBITS, ADT, G, MPV, 8, true, ##__VA_ARGS__><<<grid, block, smem, st>>>(p); \
        else gemm_wo_decode_lds_kernel<WBITS, ADT, G, MPV, 16, false, ##__VA_ARGS__><<<grid, block, smem, st>>>(p);  \
    } while (0)
        // per-channel scales (and zero points) of the activations' 16-bit type, or fp16 everything with small
        // groups: the reference's own per-weight rounding
        // (not int4 weights under bf16: see launch_wo_panel)
        constexpr bool CAN_REFQ = ADT == FNN_F16 || WBITS == 8;
        const bool refq = (CAN_REFQ && p.group == 0 && p.scale_dtype == ADT && (!p.zp || p.zp_dtype == ADT)) || small_groups;
        if constexpr (ADT == FNN_F16) {
            if (small_groups && p.zp) FNN_DEC(false, 8, 4);
            else if (small_groups) FNN_DEC(false, 8, 3);
        }
        if constexpr (CAN_REFQ) {
            if (refq && !small_groups) {
                if (p.zp) FNN_DEC(false, 8, 2);
                else FNN_DEC(false, 8, 1);
            }
        }
        if (refq) {}
        else if (p.group == 0) FNN_DEC(false, 8);
        else if (p.M == 1) FNN_DEC(true, 1);
        else if (p.M == 2) FNN_DEC(true, 2);
        else if (p.M <= 4) FNN_DEC(true, 4);
        else FNN_DEC(true, 8);
#undef FNN_DEC
        return true;
    }
    if (small_groups || lds_only) return false;      // the kernel below walks groups of whole 128-value steps
    const size_t smem = fixed + (act_lds ? act_bytes : 0);
    if (smem > 64 * 1024) return false;
    note_kernel("gemm_wo_decode_kernel", WBITS, p.group, act_lds);
    if (p.group > 0) {
        if (act_lds) gemm_wo_decode_kernel<WBITS, ADT, true, true><<<grid, block, smem, st>>>(p);
        else gemm_wo_decode_kernel<WBITS, ADT, true, false><<<grid, block, smem, st>>>(p);
    } else {
        if (act_lds) gemm_wo_decode_kernel<WBITS, ADT, false, true><<<grid, block, smem, st>>>(p);
        else gemm_wo_decode_kernel<WBITS, ADT, false, false><<<grid, block, smem, st>>>(p);
    }
    return true;
}

// ---- bf16 activation rows -> fp16 rows (for the kernels that round every weight as the reference does)
// One 256-thread workgroup per row.  The row's largest magnitude is brought to [2^13, 2^14) by a power of two,
// so every bf16 value (8 significant bits) whose magnitude is within 2^-30 of the row's largest becomes an
// fp16 value without loss and nothing overflows; smaller ones lose low bits that could not move the output.
// The inverse power goes to unscale[row]; rows of zeros or with non-finite values are left unscaled.
__global__ __launch_bounds__(256) void act_bf16_to_f16_kernel(uint16_t* dst, float* unscale, const uint16_t* src, int K,
                                                              int64_t lda) {
    __shared__ uint32_t smax[4];
    const int row = blockIdx.x;
    const uint16_t* in = src + (int64_t)row * lda;
    uint16_t* out = dst + (int64_t)row * K;
    uint32_t mx = 0;            // magnitudes compare like their bit patterns
    for (int k = threadIdx.x * 8; k < K; k += 256 * 8) {
        const v4u v = *(const v4u*)(in + k);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            mx = max(mx, v[i] & 0x7FFFu);
            mx = max(mx, (v[i] >> 16) & 0x7FFFu);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = max(max(smax[0], smax[1]), max(smax[2], smax[3]));
    const int ex = (int)(mx >> 7);
    const int sh = (ex == 0 || ex == 255) ? 0 : max(-100, min(100, 13 - (ex - 127)));
    const float up = __uint_as_float((uint32_t)(127 + sh) << 23);
    if (threadIdx.x == 0) unscale[row] = __uint_as_float((uint32_t)(127 - sh) << 23);
    for (int k = threadIdx.x * 8; k < K; k += 256 * 8) {
        const v4u v = *(const v4u*)(in + k);
        v4u o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = __uint_as_float(v[i] << 16) * up, hi = __uint_as_float(v[i] & 0xFFFF0000u) * up;
            o[i] = f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
        }
        *(v4u*)(out + k) = o;
    }
}

size_t act_f16_ws_bytes(int64_t M, int64_t K) { return (size_t)((M * K * 2 + 255) / 256 * 256) + (size_t)M * sizeof(float); }

bool convert_act_to_f16(const WoArgs& p, WoArgs& q, hipStream_t st) {
    if (!p.cvt_ws || p.cvt_ws_bytes < act_f16_ws_bytes(p.M, p.K) || ((uintptr_t)p.cvt_ws % 16) != 0) return false;
    if (p.scale_dtype != FNN_F16 || (p.zp && p.zp_dtype != FNN_F16) || (p.group != 0 && group_shift(p.group) < 0)) return false;
    if (p.K % 8 != 0 || p.lda % 8 != 0 || ((uintptr_t)p.act % 16) != 0 || p.m_base != 0) return false;
    q = p;
    q.act = p.cvt_ws;
    q.lda = p.K;
    q.act_unscale = (const float*)((char*)p.cvt_ws + (size_t)(((int64_t)p.M * p.K * 2 + 255) / 256 * 256));
    q.cvt_ws = nullptr;
    q.cvt_ws_bytes = 0;
    note_kernel("act_bf16_to_f16_kernel");
    act_bf16_to_f16_kernel<<<dim3(p.M), dim3(256), 0, st>>>((uint16_t*)p.cvt_ws, (float*)q.act_unscale,
                                                            (const uint16_t*)p.act, p.K, p.lda);
    return true;
}

// Any number of rows through the decode kernels, as many rows a pass as they take (8, 4, 2 or 1: their
// activations and group tables have to fit the LDS); false, with nothing launched, if they do not take the
// shape at all.  Every pass reads the weights again: for the shapes that would otherwise fall to the
// one-thread-per-output kernel (groups of 32 with more than 8 rows: 0.5 - 130 ms there, 20 to 100 times less
// here).
template <int WBITS, int ADT>
static bool decode_in_passes(const WoArgs& p, hipStream_t st) {
    const int esz = p.out_dtype == FNN_F32 ? 4 : 2;
    for (int rows = 8; rows >= 1; rows >>= 1) {
        for (int m0 = 0; m0 < p.M; m0 += rows) {
            WoArgs q = p;
            q.act = (const char*)p.act + (int64_t)m0 * p.lda * 2;
            q.out = (char*)p.out + (int64_t)m0 * p.ldc * esz;
            q.M = p.M - m0 < rows ? p.M - m0 : rows;
            if (!launch_decode<WBITS, ADT>(q, st, false)) {
                if (m0 != 0) return true;      // (cannot happen: a pass of fewer rows needs less than the first)
                break;
            }
            if (m0 + rows >= p.M) return true;
        }
    }
    return false;
}

template <int WBITS, int ADT>
static void dispatch_wo(WoArgs& p, hipStream_t st) {
    const bool aligned = p.K % 64 == 0 && p.ldw % 16 == 0 && p.lda % 8 == 0 && ((uintptr_t)p.qw % 16) == 0 &&
                         ((uintptr_t)p.act % 16) == 0;
    const bool fast = aligned && (p.group == 0 || p.group % 64 == 0 || p.group == 32);
    // per-channel scales with K a multiple of 32 only: the panel kernel handles the partial last slab
    if (p.group == 0 && p.K % 128 != 0 && launch_wo_panel(p, WBITS, ADT, st)) return;
    // groups of 32, up to 8 rows, fp16 throughout: the decode kernel that rounds every dequantised weight to fp16
    // as the reference does, fewer rows at a time where its tables do not fit for all; everything else with
    // groups of 32 goes to the stream kernel at the end
    if (aligned && p.group == 32 && p.M <= 8 && decode_in_passes<WBITS, ADT>(p, st)) return;
    if (!fast) {
        const int64_t total = (int64_t)p.M * p.N;
        note_kernel("gemm_wo_any_kernel", WBITS);
        gemm_wo_any_kernel<WBITS, ADT><<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st>>>(p);
        return;
    }
    // Measured order of preference: the one-wave-per-tile kernel for up to 4 rows over int4 weights
    // with many tiles (and for a single row over int8 weights); from 2 rows on the panel kernel,
    // whose waves share the activations through LDS; the other decode kernels for a single row and
    // for the shapes the panel kernel does not take.
    if (p.M <= 4 && (WBITS == 4 || p.M == 1) && launch_decode<WBITS, ADT>(p, st, true)) return;
    // 2 to 4 rows over at most 4096 weight rows: such a call is a handful of memory latencies, and the decode kernel
    // (512 workgroups at most, K split over the waves of each, the activations copied to LDS once) gets through them
    // sooner than the panel kernel's slab pipeline with its barrier per slab.  Measured under a captured graph with
    // rotating weights, panel / decode kernel, us - int8 per channel N=K=4096: M=2 8.7 / 6.8, M=4 8.6 / 7.6; N=2048
    // K=2048 5.9 / 4.4; N=2048 K=8192 M=2 10.2 / 6.5; int4 g128 N=K=4096 8.7 / 6.4 and 8.7 / 6.9; N=8192 K=4096 9.6 /
    // 8.2 and 9.5 / 9.1.  With more weight rows every workgroup's own copy of the activations (M K 2 bytes against the
    // 8 K bytes of its weights) costs more than the latencies saved: int8 N=8192 K=2048 7.7 / 8.7, N=4608 K=3584
    // 8.7 / 9.5.  Inside the rule the decode kernel is behind by at most 9 % (int4 N=4608 K=3584 M=4 8.5 / 9.3).
    // Both kernels round alike (per weight with per-channel tables of the activations' type, in fp32 otherwise).
    if (p.M >= 2 && p.M <= 4 && (WBITS == 4 ? p.N / 2 : p.N) <= 4096 && launch_decode<WBITS, ADT>(p, st, false, true)) return;
    // More than 64 rows: the tiled kernel dequantises every weight once per 128 or 256 rows (the panel kernel
    // takes 64 a pass), but a tile is one workgroup walking all of K: with 128 tiles or fewer half the CUs
    // or more stand idle while the others each need about 1.3 us per 128 values of K, and 64-row passes of the
    // panel kernel finish sooner (fp16 rows, int4 g128, tiled / passes: M=128 N=4096 K=11008 102 / 31 us, M=256
    // N=K=8192 83 / 58 us, M=512 N=K=4096 46 / 33 us; from 172 tiles on the tiled kernel wins: M=256 N=11008
    // K=4096 45 / 57 us, M=128 N=28672 K=8192 90 / 109 us; int8 weights alike).
    if (p.M > 64) {
        const bool fills = wo_tile_count(p, WBITS) > 128;
        if (fills && launch_wo_tile(p, WBITS, ADT, st)) return;
        if (launch_wo_panel(p, WBITS, ADT, st)) return;
        if (!fills && launch_wo_tile(p, WBITS, ADT, st)) return;
    }
    // groups of 64, up to 8 rows, fp16 throughout: the decode kernel rounds every dequantised weight to fp16 as the
    // reference does (flashnn/quant_gemm.py:14-36), the panel kernel scales group sums in fp32
    if (p.group == 64 && p.M <= 8 && ADT == FNN_F16 && p.scale_dtype == FNN_F16 && (!p.zp || p.zp_dtype == FNN_F16) &&
        launch_decode<WBITS, ADT>(p, st, false))
        return;
    // One row: the decode kernels, except where they are the slower choice (measured under a captured graph,
    // rotating weights, decode / panel kernel): rows too long for the decode kernel's LDS copy of the activations
    // (K > 16864: int4 g128 N=8192 K=28672 54.9 / 30.7 us, N=3584 K=18944 34.8 / 21.4 us; int8 per channel 54.2 /
    // 37.8 and 31.1 / 18.4 us), and int8 weights with per-channel tables over many channels when K / 128 is not a
    // multiple of 32, where the decode kernel runs its guarded form (N=15360 K=5120 21.0 / 16.2 us, N=27648
    // 33.4 / 28.3 us, N=37888 K=3584 40.3 / 30.4 us; with 4096 to 5120 channels the two are equal).
    const bool one_row_on_panel = p.M == 1 && ((size_t)(p.K + 32) * 2 > kDecodeActLdsBytes ||
                                               (WBITS == 8 && p.group == 0 && (p.K / 128) % 32 != 0 && p.N >= 12288));
    if ((p.M >= 2 || one_row_on_panel) && launch_wo_panel(p, WBITS, ADT, st)) return;
    if (launch_decode<WBITS, ADT>(p, st, false)) return;
    // up to 64 activation rows per pass over the weights
    for (int m0 = 0; m0 < p.M; m0 += 64) {
        p.m_base = m0;
        const int rem = p.M - m0;
        if (rem <= 16) launch_stream<WBITS, ADT, 1>(p, st);
        else if (rem <= 32) launch_stream<WBITS, ADT, 2>(p, st);
        else launch_stream<WBITS, ADT, 4>(p, st);
    }
}

template <int WBITS>
static int run_wo(const char* fn, void* out, const void* act, const void* qw, const void* scale,
                  const void* bias, const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda,
                  int64_t ldw, int64_t ldc, int64_t group, int act_dtype, int out_dtype,
                  int scale_dtype, int zp_dtype, int bias_dtype, void* stream, void* workspace = nullptr,
                  size_t ws_bytes = 0, int block_m = 0, int block_n = 0) {
    // an empty tensor has no address: pointers are only required when there is something to compute
    if (M != 0 && N != 0 && (!out || !act || !qw || !scale)) { set_error("%s: null pointer argument", fn); return FNN_ERR_ARG; }
    if (M < 0 || N < 0 || K <= 0 || lda < K || ldw < K || ldc < N || group < 0) {
        set_error("%s: bad shape M=%lld N=%lld K=%lld lda=%lld ldw=%lld ldc=%lld group=%lld", fn,
                  (long long)M, (long long)N, (long long)K, (long long)lda, (long long)ldw,
                  (long long)ldc, (long long)group);
        return FNN_ERR_ARG;
    }
    if (WBITS == 4 && (N & 1)) { set_error("%s: N must be even for packed int4 weights", fn); return FNN_ERR_ARG; }
    if (group > 0 && K % group != 0) { set_error("%s: K=%lld is not a multiple of the group size %lld", fn, (long long)K, (long long)group); return FNN_ERR_ARG; }
    if (!is16(act_dtype) || !is16(out_dtype)) { set_error("%s: activations and output must be fp16 or bf16", fn); return FNN_ERR_UNSUPPORTED; }
    if (!isflt(scale_dtype) || (zp && !isflt(zp_dtype)) || (bias && !isflt(bias_dtype))) {
        set_error("%s: scale / zero-point / bias type must be fp16, bf16 or fp32", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30) || lda > (1LL << 30) || ldw > (1LL << 30)) {
        set_error("%s: shape or row stride too large", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (M == 0 || N == 0) return FNN_OK;
    WoArgs p{};
    p.act = act; p.qw = (const int8_t*)qw; p.scale = scale; p.zp = zp; p.bias = bias; p.out = out;
    p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = lda; p.ldw = ldw; p.ldc = ldc; p.group = (int)group;
    p.out_dtype = out_dtype; p.scale_dtype = scale_dtype; p.zp_dtype = zp_dtype; p.bias_dtype = bias_dtype;
    if (ws_bytes > 0 && !workspace) { set_error("%s: a workspace size without a workspace", fn); return FNN_ERR_ARG; }
    p.cvt_ws = workspace; p.cvt_ws_bytes = ws_bytes;
    if (block_m != 0 || block_n != 0) {
        // Blocks named by the caller (a recorded configuration, or a candidate being timed): the few-row kernel
        // with block_m activation rows per pass and block_n output channels per workgroup, for up to 64 rows -
        // the range in which it is the launcher's own choice from two rows on.  Refused where the launcher's
        // choice rounds every weight as the reference does and this kernel would not (groups of 64, up to 8 rows,
        // fp16 throughout), so that a named block never changes how the result is rounded.
        constexpr int NH = WBITS == 4 ? 2 : 1;
        const bool rounds_elsewhere = group == 64 && M <= 8 && act_dtype == FNN_F16 && scale_dtype == FNN_F16 &&
                                      (!zp || zp_dtype == FNN_F16);
        if (M > 64 || block_m % 16 != 0 || block_n % (16 * NH) != 0 || rounds_elsewhere) {
            set_error("%s: blocks of %d rows x %d channels are not available for M=%lld group=%lld", fn, block_m, block_n,
                      (long long)M, (long long)group);
            return FNN_ERR_UNSUPPORTED;
        }
        p.force_mb = block_m / 16;
        p.force_rt = block_n / (16 * NH);
        const Call call(fn);
        if (!launch_wo_panel(p, WBITS, act_dtype, (hipStream_t)stream)) {
            set_error("%s: the few-row kernel does not take this problem with blocks of %d rows x %d channels", fn, block_m, block_n);
            return FNN_ERR_UNSUPPORTED;
        }
        return call.done();
    }
    const Call call(fn);
    if (act_dtype == FNN_F16) dispatch_wo<WBITS, FNN_F16>(p, (hipStream_t)stream);
    else dispatch_wo<WBITS, FNN_BF16>(p, (hipStream_t)stream);
    return call.done();
}

}  // namespace fnn

using namespace fnn;

extern "C" int fnn_gemm_a16w8(void* out, const void* act, const void* qw, const void* scale,
                              const void* bias, const void* zp, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldw, int64_t ldc, int64_t group, int act_dtype,
                              int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                              void* stream) {
    return run_wo<8>("fnn_gemm_a16w8", out, act, qw, scale, bias, zp, M, N, K, lda, ldw, ldc, group,
                     act_dtype, out_dtype, scale_dtype, zp_dtype, bias_dtype, stream);
}

extern "C" int fnn_gemm_a16w4(void* out, const void* act, const void* qw, const void* scale,
                              const void* bias, const void* zp, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldw, int64_t ldc, int64_t group, int act_dtype,
                              int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                              void* stream) {
    return run_wo<4>("fnn_gemm_a16w4", out, act, qw, scale, bias, zp, M, N, K, lda, ldw, ldc, group,
                     act_dtype, out_dtype, scale_dtype, zp_dtype, bias_dtype, stream);
}

extern "C" int fnn_gemm_a16w8_tiled(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                                    const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                                    int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype,
                                    int bias_dtype, int block_m, int block_n, void* stream) {
    if (block_m <= 0 || block_n <= 0) { set_error("fnn_gemm_a16w8_tiled: block_m and block_n must be positive"); return FNN_ERR_ARG; }
    return run_wo<8>("fnn_gemm_a16w8_tiled", out, act, qw, scale, bias, zp, M, N, K, lda, ldw, ldc, group, act_dtype,
                     out_dtype, scale_dtype, zp_dtype, bias_dtype, stream, nullptr, 0, block_m, block_n);
}

extern "C" int fnn_gemm_a16w4_tiled(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                                    const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                                    int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype,
                                    int bias_dtype, int block_m, int block_n, void* stream) {
    if (block_m <= 0 || block_n <= 0) { set_error("fnn_gemm_a16w4_tiled: block_m and block_n must be positive"); return FNN_ERR_ARG; }
    return run_wo<4>("fnn_gemm_a16w4_tiled", out, act, qw, scale, bias, zp, M, N, K, lda, ldw, ldc, group, act_dtype,
                     out_dtype, scale_dtype, zp_dtype, bias_dtype, stream, nullptr, 0, block_m, block_n);
}

extern "C" size_t fnn_gemm_weight_only_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int act_dtype,
                                                       int scale_dtype) {
    // bf16 activations with fp16 tables, more than 64 rows (the tiled kernel): the rows are converted to fp16
    // once, so that every weight can be rounded as the reference rounds it
    if (M <= 64 || N <= 0 || K <= 0 || K % 8 != 0 || M > (1 << 30) || K > (1 << 30)) return 0;
    if (act_dtype != FNN_BF16 || scale_dtype != FNN_F16 || (group != 0 && (group_shift((int)group) < 0 || K % group != 0))) return 0;
    // ... where the tiled kernel takes the call (dispatch_wo): a shape it accepts, and more than 128 tiles or
    // rows too short for the panel kernel (the count of 128-row tiles decides for 256-row tiles as well)
    if (N % 128 != 0 || K % 256 != 0 || K < 512) return 0;
    if (((M + 127) / 128) * (N / 128) <= 128 && K >= 1024) return 0;
    return act_f16_ws_bytes(M, K);
}

extern "C" int fnn_gemm_a16w8_ws(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                                 const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                                 int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype,
                                 int bias_dtype, void* workspace, size_t ws_bytes, void* stream) {
    return run_wo<8>("fnn_gemm_a16w8_ws", out, act, qw, scale, bias, zp, M, N, K, lda, ldw, ldc, group, act_dtype,
                     out_dtype, scale_dtype, zp_dtype, bias_dtype, stream, workspace, ws_bytes);
}

extern "C" int fnn_gemm_a16w4_ws(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                                 const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                                 int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype,
                                 int bias_dtype, void* workspace, size_t ws_bytes, void* stream) {
    return run_wo<4>("fnn_gemm_a16w4_ws", out, act, qw, scale, bias, zp, M, N, K, lda, ldw, ldc, group, act_dtype,
                     out_dtype, scale_dtype, zp_dtype, bias_dtype, stream, workspace, ws_bytes);
}

// ------------------------------------------------------------------ mixture of experts, int4 weights
namespace fnn {

// Any shape, per-channel or grouped scales with any strides: one thread per output value.
// out[t, n] = sum over K blocks g of scale[e, n, g] * sum_{k in g} act[t / top_k, k] * (nibble(e, n, k) - zp[e, n, g])
template <int ADT>
__global__ __launch_bounds__(256) void moe_a16w4_any_kernel(const WoArgs p, const MoeArgs q) {
    const int sidx = blockIdx.x;
    if (sidx >= q.ntpp[0]) return;
    const int tok = q.sorted_ids[sidx];
    if (tok >= q.num_valid) return;
    const int n = blockIdx.y * 256 + threadIdx.x;
    if (n >= p.N) return;
    const int expert = q.expert_ids[sidx / q.block_m];
    const uint16_t* a = (const uint16_t*)p.act + (int64_t)(tok / q.top_k) * p.lda;
    const int8_t* w = p.qw + (int64_t)expert * q.stride_be + (int64_t)(n >> 1) * p.ldw;
    const int g = p.group > 0 ? p.group : p.K;
    float acc = 0.f;
    for (int k0 = 0, kb = 0; k0 < p.K; k0 += g, ++kb) {
        const float zp = p.zp ? load_zp_f32(p.zp, expert * q.stride_zp_be + n * q.stride_zp_n + kb * q.stride_zp_k, p.zp_dtype)
                              : 0.f;
        float part = 0.f;
        const int k1 = min(k0 + g, p.K);
        for (int k = k0; k < k1; ++k) {
            const int b = w[k];
            const int nib = (n & 1) ? (b >> 4) : ((int)(int8_t)((uint8_t)b << 4) >> 4);
            part += bits_to_f32<ADT>(a[k]) * ((float)nib - zp);
        }
        acc += part * load_as_f32(p.scale, expert * q.stride_scale_be + n * q.stride_scale_n + kb * q.stride_scale_k,
                                  p.scale_dtype);
    }
    if (q.mul_w) acc *= load_as_f32(q.topk_w, tok, q.topk_w_dtype);
    ((uint16_t*)p.out)[(int64_t)tok * p.ldc + n] = (uint16_t)f32_to_bits<ADT>(acc);
}

}  // namespace fnn

extern "C" int fnn_fused_moe_a16w4(void* c, const void* a, const void* b, const void* scale_b,
                                   const void* zero_points, const void* topk_weights,
                                   const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                   const int32_t* num_tokens_post_padded, int64_t N, int64_t K, int64_t EM,
                                   int64_t num_valid_tokens, int64_t lda, int64_t stride_be, int64_t ldb,
                                   int64_t ldc, int64_t stride_scale_be, int64_t stride_scale_n,
                                   int64_t stride_scale_k, int64_t stride_zp_be, int64_t stride_zp_n,
                                   int64_t stride_zp_k, int group, int mul_routed_weight, int top_k, int block_m,
                                   int act_dtype, int scale_dtype, int zp_dtype, int topk_weights_dtype,
                                   void* stream) {
    using namespace fnn;
    const char* fn = "fnn_fused_moe_a16w4";
    if (!c || !a || !b || !scale_b || !sorted_token_ids || !expert_ids || !num_tokens_post_padded ||
        (mul_routed_weight && !topk_weights)) {
        set_error("%s: null pointer argument", fn);
        return FNN_ERR_ARG;
    }
    if (N < 0 || K <= 0 || EM < 0 || num_valid_tokens < 0 || top_k <= 0 || block_m <= 0 || lda < K || ldb < K ||
        ldc < 2 * N || group < 0 || (group > 0 && K % group != 0)) {
        set_error("%s: bad shape N=%lld K=%lld EM=%lld tokens=%lld top_k=%d block_m=%d group=%d", fn, (long long)N,
                  (long long)K, (long long)EM, (long long)num_valid_tokens, top_k, block_m, group);
        return FNN_ERR_ARG;
    }
    if (2 * N > 0x7FFFFFFFLL || K > 0x7FFFFFFFLL || EM > 0x7FFFFFFFLL || num_valid_tokens > 0x7FFFFFFFLL) {
        set_error("%s: shape too large", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (!is16(act_dtype)) { set_error("%s: activations must be float16 or bfloat16", fn); return FNN_ERR_UNSUPPORTED; }
    if (!isflt(scale_dtype) || (zero_points && !isflt(zp_dtype) && zp_dtype != FNN_I8) ||
        (mul_routed_weight && !isflt(topk_weights_dtype))) {
        set_error("%s: bad scale, zero point or routing weight type", fn);
        return FNN_ERR_UNSUPPORTED;
    }
    if (N == 0 || EM == 0 || num_valid_tokens == 0) return FNN_OK;
    WoArgs p{};
    p.act = a; p.qw = (const int8_t*)b; p.scale = scale_b; p.zp = zero_points; p.bias = nullptr; p.out = c;
    p.M = (int)EM; p.N = (int)(2 * N); p.K = (int)K; p.lda = lda; p.ldw = ldb; p.ldc = ldc; p.group = group;
    p.out_dtype = act_dtype; p.scale_dtype = scale_dtype; p.zp_dtype = zp_dtype; p.bias_dtype = act_dtype;
    MoeArgs q{};
    q.sorted_ids = sorted_token_ids; q.expert_ids = expert_ids; q.ntpp = num_tokens_post_padded;
    q.topk_w = topk_weights; q.topk_w_dtype = topk_weights_dtype; q.mul_w = mul_routed_weight ? 1 : 0;
    q.top_k = top_k; q.block_m = block_m; q.num_valid = (int)num_valid_tokens; q.EM = (int)EM;
    q.stride_be = stride_be; q.stride_scale_be = stride_scale_be; q.stride_zp_be = stride_zp_be;
    q.stride_scale_n = stride_scale_n; q.stride_scale_k = stride_scale_k;
    q.stride_zp_n = stride_zp_n; q.stride_zp_k = stride_zp_k;
    hipStream_t st = (hipStream_t)stream;
    // the weight-streaming kernel takes per-channel tables and groups of 128 (launch_wo_panel_moe checks the layout
    // and the types)
    const bool fast = group == 0 || group == 128;
    const Call call(fn);
    if (!(launch_wo_tile_moe(p, q, act_dtype, st) || (fast && launch_wo_panel_moe(p, q, act_dtype, st)))) {
        const dim3 grid((unsigned)EM, (unsigned)((2 * N + 255) / 256));
        note_kernel("moe_a16w4_any_kernel");
        if (act_dtype == FNN_F16) moe_a16w4_any_kernel<FNN_F16><<<grid, dim3(256), 0, st>>>(p, q);
        else moe_a16w4_any_kernel<FNN_BF16><<<grid, dim3(256), 0, st>>>(p, q);
    }
    return call.done();
}
