"""CPU oracle for the FLASHNN quantized-GEMM path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU and with every rounding step written out, the
arithmetic of the reference's torch path for the operators the HIP library
implements.  It is imported only by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py - never by the flashnn_amd package.

Functions take/return numpy arrays.  16-bit floating inputs are passed as float32
arrays holding exactly representable values together with a dtype tag ("f16" or
"bf16"); helpers at the bottom convert from/to torch tensors.

Reference statements followed (all under /root/reference):
  dynamic_quantize      flashnn/quant_gemm.py:53-57
  gemm_a8w8_*           flashnn/quant_gemm.py:96-104, triton_kernels/gemm_a8w8.py:135-173
  weight_only_*         flashnn/quant_gemm.py:14-36, 148-206
  rmsnorm_dquant        flashnn/norm.py:45-60
  rmsnorm               flashnn/norm.py:25-33
  layernorm(_dquant)    flashnn/norm.py:82-85, 112-119 (torch.nn.functional.layer_norm)

How each function is pinned (tests/test_oracle.py):
  dynamic_quantize   against the literal torch-op formula on CPU tensors (the third
                     party arithmetic the reference calls), a per-element brute force
                     with numpy.float16 scalars, row invariants (max|q| = 127, sign,
                     |q*s - x| bound) and hand-computed rows;
  gemm_a8w8_acc      against a pure-Python triple loop, numpy int64 matmul,
                     torch._int_mm, the C restatement oracle/int8_gemm.c, identity and
                     saturation cases (K=4096 of (-128)*(-128) = 67108864);
  gemm_a8w8          float64 closed form within 1 ulp of the output type;
  unpack_int4        against a per-byte Python loop and an all-256-bytes table;
  weight_only        against a float64 brute force on small shapes and the
                     scale=1, zp=0 integer special case;
  rmsnorm_dquant     against the literal torch-op formula (<= 1 LSB on elements whose
                     pre-round fraction is at a tie, because torch sums x^2 in its own
                     fp32 order) and float64 closed forms.
  rmsnorm            against the literal torch-op formula (1 ulp of the output type where
                     the mean differs in its last bit), a constant-row closed form;
  layernorm          against torch.nn.functional.layer_norm on CPU tensors (1 ulp of the
                     output type: torch's moments are taken in an order of its own),
                     a float64 evaluation, zero-mean / unit-variance invariants and
                     closed forms (constant row -> bias);
  layernorm_dquant   its quantisation step is dynamic_quantize applied to layernorm's
                     rounded output (checked to be literally that), against the torch
                     ops within one quantisation step where the 1-ulp cases above land
                     on a tie.
The reference's tests hold no golden vectors for this path (they regenerate seeded
inputs on a GPU), so no fixture of theirs exists to check against; the int4 branch has
no reference test at all and is pinned by the formula at quant_gemm.py:174-204 only.
"""
from __future__ import annotations

import numpy as np

F16 = "f16"
BF16 = "bf16"
F32 = "f32"


# --------------------------------------------------------------------------- rounding
def round_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bfloat16 (ties to even); result as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).copy()
    nan = np.isnan(x)
    if nan.any():
        out[nan] = np.nan
    return out


def round_f16(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest float16 (ties to even); result as float32."""
    with np.errstate(over="ignore"):
        return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == F16:
        return round_f16(x)
    if dtype == BF16:
        return round_bf16(x)
    if dtype == F32:
        return np.asarray(x, dtype=np.float32)
    raise ValueError(dtype)


# ------------------------------------------------------------------- dynamic quantize
def dynamic_quantize(x: np.ndarray, dtype: str, scale_dtype: str | None = None, clamp: bool = True):
    """Per-token symmetric int8 quantisation in the input type.

    flashnn/quant_gemm.py:53-57:  max = |x|.max(-1); scale = max / 127.0;
    out = round(x / scale); return out.int8, scale.half().
    torch evaluates each 16-bit elementwise op in fp32 and rounds the result to the
    tensor type, so there are two roundings to `dtype` before the round-half-even.
    Rows that are entirely zero are undefined in the reference (0/0); here, and in
    the HIP kernel, they give q = 0 and scale = 0.
    Returns (q int8 [M,K], scale float16 [M]); with `scale_dtype` given, the scale is
    returned unconverted instead, as float32 values representable in that type.
    The reference's torch path does not clamp here; with bf16 inputs the scale can round down
    far enough for the row maximum to quantise to 128, which the conversion to int8 wraps to
    -128: the sign of the row's largest activation (about 2 % of N(0,1) rows of 1024 values;
    fp16 inputs never exceed 127).  The reference's own kernel for this operator cannot exceed
    +-127 (triton_kernels/dynamic_quant.py:65-67), LayernormDquant clamps (flashnn/norm.py:118),
    and so does this oracle by default, as the HIP kernel does: `clamp` = clamp to [-128, 127];
    clamp=False is the literal torch formula.  The two differ only where the unclamped value is 128.
    """
    x = np.asarray(x, dtype=np.float32)
    mx = np.abs(x).max(axis=-1, keepdims=True)
    scale = round_to(mx / np.float32(127.0), dtype)
    with np.errstate(divide="ignore", invalid="ignore"):
        t = round_to(x / scale, dtype)
    q = np.rint(t)
    if clamp:
        q = np.clip(q, -128.0, 127.0)
    q = np.where(scale == 0, np.float32(0), q)
    if scale_dtype is not None:
        assert scale_dtype == dtype
        return q.astype(np.int8), scale.reshape(x.shape[:-1])
    with np.errstate(over="ignore"):
        s16 = scale.astype(np.float16)
    return q.astype(np.int8), s16.reshape(x.shape[:-1])


# ----------------------------------------------------------------------- A8W8 GEMM
def gemm_a8w8_acc(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Exact integer accumulators acc[m,n] = sum_k a[m,k]*b[n,k] as int32.

    This is what the reference's kernel holds before its epilogue
    (triton_kernels/gemm_a8w8.py:135-150).  Evaluated with float32 BLAS on K-chunks of
    1024: |partial| <= 128*128*1024 = 2^24, so every chunk is exact in float32; chunks
    are added in int64.
    """
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == np.int8 and b.dtype == np.int8 and a.shape[1] == b.shape[1]
    M, K = a.shape
    N = b.shape[0]
    acc = np.zeros((M, N), dtype=np.int64)
    for k0 in range(0, K, 1024):
        pa = a[:, k0:k0 + 1024].astype(np.float32)
        pb = b[:, k0:k0 + 1024].astype(np.float32)
        acc += (pa @ pb.T).astype(np.int64)
    assert np.abs(acc).max(initial=0) < 2 ** 31
    return acc.astype(np.int32)


def gemm_a8w8(a, b, alpha_row, alpha_col, out_dtype: str) -> np.ndarray:
    """A8W8 output from the exact accumulators, in float64 then rounded once.

    flashnn/quant_gemm.py:96-104 forms float(a)@float(b) * (alpha_row x alpha_col);
    triton_kernels/gemm_a8w8.py:166-173 forms int32 acc * fp32(alpha_row) *
    fp32(alpha_col).  Both approximate acc*ar*ac; this returns that product evaluated
    in float64 and rounded to the output type (float32 array of representable values).
    """
    acc = gemm_a8w8_acc(a, b).astype(np.float64)
    ar = np.asarray(alpha_row, dtype=np.float64).reshape(-1, 1)
    ac = np.asarray(alpha_col, dtype=np.float64).reshape(1, -1)
    return round_to((acc * ar * ac).astype(np.float32), out_dtype)


def gemm_a8w8_epilogue_fp32(acc, alpha_row, alpha_col, out_dtype: str) -> np.ndarray:
    """The fp32 epilogue order of triton_kernels/gemm_a8w8.py:166-173:
    float(acc) * fp32(alpha_row[m]) then * fp32(alpha_col[n]), rounded to out_dtype."""
    x = np.asarray(acc).astype(np.float32)
    ar = np.asarray(alpha_row, dtype=np.float32).reshape(-1, 1)
    ac = np.asarray(alpha_col, dtype=np.float32).reshape(1, -1)
    return round_to((x * ar) * ac, out_dtype)


def fused_moe_a8w8(a, b, c, alpha_row, alpha_col, topk_weights, sorted_token_ids, expert_ids,
                   num_tokens_post_padded, mul_routed_weight: bool, top_k: int, block_m: int, out_dtype: str):
    """Mixture-of-experts A8W8 GEMM, flashnn/triton_kernels/fused_moe_a8w8.py:74-173, block by block as
    the kernel walks them: sorted rows [i*block_m, (i+1)*block_m) below num_tokens_post_padded (:94-96)
    use expert expert_ids[i] (:107); routed row t = sorted_token_ids[..] is valid if t < M*top_k (:98);
    its token is a[t // top_k] (:102-104); acc is the int32 contraction with b[e] (:118-144); then
    fp32(acc) * alpha_row[t // top_k], * alpha_col[e, n] (:150-157), * topk_weights[t] if asked (:159-161),
    each product rounded to fp32, one rounding to the output type (:163, fp16 in the reference), stored
    at c[t] (:166-168).  `c` ([M*top_k, N] float32 holding out_dtype values) is updated in place and
    returned: rows no valid sorted row names keep what they held.

    The reference has no test or torch path for this function.  Pinned by: a per-element Python loop on
    tiny inputs, the reduction to gemm_a8w8_epilogue_fp32 when every row goes to one expert, and
    invariance under permutations of the sorted list within an expert (tests/test_oracle.py)."""
    a = np.asarray(a)
    b = np.asarray(b)
    ar = np.asarray(alpha_row, dtype=np.float32).reshape(-1)
    ac = np.asarray(alpha_col, dtype=np.float32).reshape(b.shape[0], b.shape[1])
    w = None if topk_weights is None else np.asarray(topk_weights, dtype=np.float32).reshape(-1)
    sorted_token_ids = np.asarray(sorted_token_ids).reshape(-1)
    num_valid = c.shape[0]
    used = int(np.asarray(num_tokens_post_padded).reshape(-1)[0])
    for blk in range((len(sorted_token_ids) + block_m - 1) // block_m):
        if blk * block_m >= used:
            break
        e = int(np.asarray(expert_ids).reshape(-1)[blk])
        toks = sorted_token_ids[blk * block_m:(blk + 1) * block_m]
        toks = toks[toks < num_valid].astype(np.int64)
        if toks.size == 0:
            continue
        acc = gemm_a8w8_acc(a[toks // top_k], b[e]).astype(np.float32)
        x = (acc * ar[toks // top_k].reshape(-1, 1)).astype(np.float32)
        x = (x * ac[e].reshape(1, -1)).astype(np.float32)
        if mul_routed_weight:
            x = (x * w[toks].reshape(-1, 1)).astype(np.float32)
        c[toks] = round_to(x, out_dtype)
    return c


# ------------------------------------------------------------------ weight-only GEMM
def unpack_int4(qw: np.ndarray) -> np.ndarray:
    """[N/2,K] packed bytes -> [N,K] int8 in [-8,7].

    flashnn/quant_gemm.py:175-190: low nibble -> channel 2j, high nibble -> 2j+1,
    values > 7 get their upper bits set (two's complement sign extension).
    """
    u = np.asarray(qw).view(np.uint8)
    lo = (u & 0x0F).astype(np.int16)
    hi = (u >> 4).astype(np.int16)
    lo = np.where(lo > 7, lo - 16, lo)
    hi = np.where(hi > 7, hi - 16, hi)
    n2, k = u.shape
    out = np.empty((2 * n2, k), dtype=np.int8)
    out[0::2] = lo
    out[1::2] = hi
    return out


def pack_int4(w: np.ndarray) -> np.ndarray:
    """Inverse of unpack_int4: [N,K] ints in [-8,7] -> [N/2,K] int8 bytes."""
    w = np.asarray(w).astype(np.int16)
    assert w.min() >= -8 and w.max() <= 7 and w.shape[0] % 2 == 0
    lo = (w[0::2] & 0xF).astype(np.uint8)
    hi = (w[1::2] & 0xF).astype(np.uint8)
    return (lo | (hi << 4)).astype(np.uint8).view(np.int8)


# ---- the packed form of int4 weights for the one-token decode (no counterpart in the reference: these two
# functions restate the layout that flashnn_amd/csrc/gemm_wo_prepacked.hip documents, one as array
# reshapes, the other address by address, so that each checks the other and the kernel's repacking)
PREPACK_UNIT_BYTES = 8 * 1024 + 2 * 256


def prepack_a16w4(qw: np.ndarray, scale: np.ndarray, zp) -> np.ndarray:
    """[N/2, K] packed bytes of the reference layout (flashnn/quant_gemm.py:175-190) plus [K/128, N] fp16
    scales and zero points (None: zeros) -> the packed stream, as uint8.

    Units in the order [tile of 16 channels][range of 1024 values of K]; a unit is 8 groups x (4 eighths x 16
    channels x 4 words) 32-bit words of nibbles, then scales [channel][group], then zero points."""
    u = (unpack_int4(qw).astype(np.int16) + 8).astype(np.uint32)          # the weight as 0..15
    N, K = u.shape
    assert N % 16 == 0 and K % 1024 == 0
    T, KC = N // 16, K // 1024
    scale = np.asarray(scale, dtype=np.float16)
    zp = np.zeros_like(scale) if zp is None else np.asarray(zp, dtype=np.float16)
    assert scale.shape == (K // 128, N) and zp.shape == scale.shape
    v = u.reshape(T, 16, KC, 8, 4, 4, 8)                                  # tile, c, kc, b, i, g, j
    word = np.zeros(v.shape[:-1], dtype=np.uint32)
    for j in range(8):
        word |= v[..., j] << np.uint32(4 * ((j >> 1) + 4 * (j & 1)))
    nib = np.ascontiguousarray(word.transpose(0, 2, 3, 5, 1, 4)).astype("<u4")   # tile, kc, b, g, c, i
    nib = nib.reshape(T, KC, 8 * 16 * 4 * 4).view(np.uint8)
    def table(t):
        t = t.reshape(KC, 8, T, 16).transpose(2, 0, 3, 1)                  # tile, kc, c, b
        return np.ascontiguousarray(t).astype("<f2").reshape(T, KC, 128).view(np.uint8)
    out = np.concatenate([nib, table(scale), table(zp)], axis=2)
    assert out.shape == (T, KC, PREPACK_UNIT_BYTES)
    return np.ascontiguousarray(out).reshape(-1)


def unpack_prepacked_a16w4(buf: np.ndarray, N: int, K: int):
    """The inverse of prepack_a16w4, walking the stream address by address: returns (qw [N/2, K] int8 in
    the reference layout, scale [K/128, N] fp16, zp [K/128, N] fp16)."""
    buf = np.asarray(buf, dtype=np.uint8)
    T, KC = N // 16, K // 1024
    assert buf.size == T * KC * PREPACK_UNIT_BYTES
    w = np.zeros((N, K), dtype=np.int8)
    scale = np.zeros((K // 128, N), dtype=np.float16)
    zp = np.zeros((K // 128, N), dtype=np.float16)
    for tile in range(T):
        for kc in range(KC):
            unit = buf[(tile * KC + kc) * PREPACK_UNIT_BYTES:][:PREPACK_UNIT_BYTES]
            for b in range(8):
                for piece in range(64):                     # 16 bytes of channel c, eighths g of four runs of 32
                    g, c = piece >> 4, piece & 15
                    raw = unit[1024 * b + 16 * piece:][:16].view("<u4")
                    for i in range(4):
                        k = 1024 * kc + 128 * b + 32 * i + 8 * g
                        for j in range(8):
                            nibble = (int(raw[i]) >> (4 * ((j >> 1) + 4 * (j & 1)))) & 0xF
                            w[16 * tile + c, k + j] = nibble - 8
            tabs = unit[8192:].view("<f2")
            for c in range(16):
                for b in range(8):
                    scale[8 * kc + b, 16 * tile + c] = tabs[8 * c + b]
                    zp[8 * kc + b, 16 * tile + c] = tabs[128 + 8 * c + b]
    return pack_int4(w), scale, zp


def dequantize_weights(w_nk, scale, zp, scale_dtype: str, group: int) -> np.ndarray:
    """Dequantised weights [K,N] as float32, with the reference's roundings.

    per channel (group == 0), flashnn/quant_gemm.py:14-17: (w - zp) * scale evaluated
    in the scale type (each op rounded to it);
    per group, flashnn/quant_gemm.py:20-36: the same per K-block, then stored into a
    float16 buffer (one more rounding to f16).
    """
    w = np.asarray(w_nk).astype(np.float32).T  # [K,N]
    K, N = w.shape
    s = np.asarray(scale, dtype=np.float32)
    if group == 0:
        s = s.reshape(1, N)
        z = np.zeros_like(s) if zp is None else np.asarray(zp, dtype=np.float32).reshape(1, N)
        return round_to(round_to(w - z, scale_dtype) * s, scale_dtype)
    assert K % group == 0 and s.shape == (K // group, N)
    z = np.zeros_like(s) if zp is None else np.asarray(zp, dtype=np.float32).reshape(s.shape)
    se = np.repeat(s, group, axis=0)
    ze = np.repeat(z, group, axis=0)
    d = round_to(round_to(w - ze, scale_dtype) * se, scale_dtype)
    return round_f16(d)


def weight_only_gemm(act, w_nk, scale, zp, bias, scale_dtype: str, out_dtype: str,
                     group: int, int4_order: bool) -> np.ndarray:
    """GemmWeightOnly._torch_impl, flashnn/quant_gemm.py:148-206.

    act [M,K] float32 (exact 16-bit values); w_nk [N,K] integer weights (already
    unpacked for int4).  fp32 matmul of act with the dequantised weights.  The int8
    branch rounds to the output type and then adds the bias in the output type
    (:168-173); the int4 branch adds the bias in fp32 and rounds once (:201-204).
    """
    dq = dequantize_weights(w_nk, scale, zp, scale_dtype, group)
    out = np.asarray(act, dtype=np.float32) @ dq
    if int4_order:
        if bias is not None:
            out = out + np.asarray(bias, dtype=np.float32).reshape(1, -1)
        return round_to(out, out_dtype)
    out = round_to(out, out_dtype)
    if bias is not None:
        out = round_to(out + np.asarray(bias, dtype=np.float32).reshape(1, -1), out_dtype)
    return out


def weight_only_gemm_f64(act, w_nk, scale, zp, bias, group: int) -> np.ndarray:
    """The mathematical value sum_k act*(w - zp)*scale + bias in float64 (no roundings)."""
    w = np.asarray(w_nk).astype(np.float64).T
    K, N = w.shape
    s = np.asarray(scale, dtype=np.float64)
    if group == 0:
        s = s.reshape(1, N)
        z = np.zeros_like(s) if zp is None else np.asarray(zp, dtype=np.float64).reshape(1, N)
    else:
        s = np.repeat(s.reshape(K // group, N), group, axis=0)
        z = (np.zeros_like(s) if zp is None
             else np.repeat(np.asarray(zp, dtype=np.float64).reshape(K // group, N), group, axis=0))
    out = np.asarray(act, dtype=np.float64) @ ((w - z) * s)
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.float64).reshape(1, -1)
    return out


def fused_moe_a16w4(a, b_packed, c, scale_b, zero_points, topk_weights, sorted_token_ids, expert_ids,
                    num_tokens_post_padded, mul_routed_weight: bool, top_k: int, block_m: int,
                    act_dtype: str, scale_dtype: str):
    """Mixture-of-experts A16W4 GEMM, flashnn/triton_kernels/fused_moe_a16w4.py.  Routing as in
    fused_moe_a8w8.  b_packed [E, N, K] bytes unpack to 2N channels, low nibble = channel 2j (:146-147).
    Per channel (scale_b [E, 2N], kernel :50-206): the integers nibble - zp are exact in the activation
    type (:148-151); fp32 dot product with the tokens (:153); times scale in fp32 (:160-164).
    Per K block (scale_b [E, 2N, K/g], kernel :209-323): (nibble - zp) * scale is formed in the scale
    type (:281-303, a rounding per weight), then the fp32 dot product (:306).  Then times
    topk_weights[t] if asked and one rounding to the activation type (:166-170, :311-315).
    Dot products are taken in float64 and rounded to fp32 (any fp32 summation order is within a few
    ulp of that).  `c` ([M*top_k, 2N] float32) is updated in place and returned.

    The reference has no test or torch path for this function.  Pinned by a float64 per-element loop on
    tiny inputs, the exact integer case and the reduction to weight_only_gemm_f64 (tests/test_oracle.py)."""
    a = np.asarray(a, dtype=np.float32)
    b_packed = np.asarray(b_packed)
    E = b_packed.shape[0]
    s = np.asarray(scale_b, dtype=np.float32)
    z = None if zero_points is None else np.asarray(zero_points, dtype=np.float32)
    w = None if topk_weights is None else np.asarray(topk_weights, dtype=np.float32).reshape(-1)
    sorted_token_ids = np.asarray(sorted_token_ids).reshape(-1)
    num_valid = c.shape[0]
    used = int(np.asarray(num_tokens_post_padded).reshape(-1)[0])
    K = a.shape[1]
    for blk in range((len(sorted_token_ids) + block_m - 1) // block_m):
        if blk * block_m >= used:
            break
        e = int(np.asarray(expert_ids).reshape(-1)[blk])
        toks = sorted_token_ids[blk * block_m:(blk + 1) * block_m]
        toks = toks[toks < num_valid].astype(np.int64)
        if toks.size == 0:
            continue
        wi = unpack_int4(b_packed[e]).astype(np.float32)            # [2N, K]
        act = a[toks // top_k].astype(np.float64)
        if s.ndim == 2:
            zz = 0.0 if z is None else z[e].reshape(-1, 1)
            x = (act @ (wi - zz).astype(np.float64).T).astype(np.float32)
            x = (x * s[e].reshape(1, -1)).astype(np.float32)
        else:
            g = K // s.shape[-1]
            zz = 0.0 if z is None else np.repeat(z[e], g, axis=1)
            dq = round_to(((wi - zz) * np.repeat(s[e], g, axis=1)).astype(np.float32), scale_dtype)
            x = (act @ dq.astype(np.float64).T).astype(np.float32)
        if mul_routed_weight:
            x = (x * w[toks].reshape(-1, 1)).astype(np.float32)
        c[toks] = round_to(x, act_dtype)
    return c


# --------------------------------------------------------------------- RMSNorm+quant
def rmsnorm_dquant(x, gamma, eps: float, dtype: str):
    """Fused RMSNorm + per-token int8 quantisation, flashnn/norm.py:45-60.

    fp32 throughout: n = x * rsqrt(mean(x^2) + eps) * gamma; scale = max|n| / 127;
    q = clamp(round_half_even(n / scale), -128, 127); scale is returned in the input
    type.  x^2 is exact in fp32 for 16-bit inputs; the sum is taken in float64 and
    rounded once to fp32 (torch adds the same exact terms in an fp32 order of its own,
    which can differ from this in the last bit of the mean).  rsqrt is 1/sqrt with both
    steps correctly rounded, as torch's CPU kernel computes it.
    Returns (q int8 [M,K], scale float32 array of values representable in `dtype`).
    """
    x = np.asarray(x, dtype=np.float32)
    g = np.asarray(gamma, dtype=np.float32).reshape(1, -1)
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    ssq = (x2.astype(np.float64) ** 2).sum(axis=-1, keepdims=True).astype(np.float32)
    mean = ssq / np.float32(K)
    rs = np.float32(1.0) / np.sqrt(mean + np.float32(eps))
    n = (x2 * rs) * g
    mx = np.abs(n).max(axis=-1, keepdims=True)
    scale = mx / np.float32(127.0)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.rint(n / scale)
    q = np.clip(q, -128.0, 127.0)
    q = np.where(scale == 0, np.float32(0), q)
    return (q.astype(np.int8).reshape(x.shape),
            round_to(scale, dtype).reshape(x.shape[:-1]))


def rmsnorm(x, gamma, eps: float, dtype: str) -> np.ndarray:
    """RMSNorm._torch_impl, flashnn/norm.py:25-33: n = x * rsqrt(mean(x^2) + eps) in fp32,
    rounded to the input type, then multiplied by gamma.  With gamma in the input type the
    product is formed in that type: the exact product of two 16-bit floats rounded once, which
    equals the fp32 product rounded to the type.  With an fp32 gamma torch returns fp32; this
    function (like the Triton launcher, rms_norm.py:68-83 + `.type_as(x)`) returns the input
    type, i.e. that fp32 product rounded once more.  Mean of squares as in rmsnorm_dquant."""
    x = np.asarray(x, dtype=np.float32)
    g = np.asarray(gamma, dtype=np.float32).reshape(1, -1)
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    ssq = (x2.astype(np.float64) ** 2).sum(axis=-1, keepdims=True).astype(np.float32)
    rs = np.float32(1.0) / np.sqrt(ssq / np.float32(K) + np.float32(eps))
    n = round_to(x2 * rs, dtype)
    return round_to(n * g, dtype).reshape(x.shape)


def layernorm(x, gamma, beta, eps: float, dtype: str) -> np.ndarray:
    """torch.nn.functional.layer_norm over the last dimension (flashnn/norm.py:82-85) for 16-bit
    inputs: moments and the affine map in fp32, one rounding to the input type at the end.
    mean = sum(x)/K and var = sum(x^2)/K - (sum(x)/K)^2 evaluated in float64 (both sums are exact
    there for 16-bit inputs, so their order does not matter) and rounded once to fp32;
    rstd = 1/sqrt(var + eps) with both steps rounded; y = ((x - mean) * rstd) * gamma + beta, every
    operation rounded to fp32."""
    x = np.asarray(x, dtype=np.float32)
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    g = np.asarray(gamma, dtype=np.float32).reshape(1, -1)
    b = np.asarray(beta, dtype=np.float32).reshape(1, -1)
    x64 = x2.astype(np.float64)
    m64 = x64.sum(axis=-1, keepdims=True) / K
    mean = m64.astype(np.float32)
    var = np.maximum((x64 * x64).sum(axis=-1, keepdims=True) / K - m64 * m64, 0.0).astype(np.float32)
    d = x2 - mean
    rstd = np.float32(1.0) / np.sqrt(var + np.float32(eps))
    y = (d * rstd) * g + b
    return round_to(y.astype(np.float32), dtype).reshape(x.shape)


def layernorm_dquant(x, gamma, beta, eps: float, dtype: str):
    """LayernormDquant._torch_impl, flashnn/norm.py:112-119: layer_norm's output (in the input
    type), then max / 127, division, round and clamp - all on tensors of the input type, i.e.
    exactly dynamic_quantize of the rounded output, plus the clamp (which binds for bf16, where
    the row maximum can quantise to 128).
    Returns (q int8 like x, scale [rows, 1] as float32 values representable in `dtype`)."""
    y = layernorm(x, gamma, beta, eps, dtype)
    q, s = dynamic_quantize(y.reshape(-1, y.shape[-1]), dtype, scale_dtype=dtype, clamp=True)
    return q.reshape(y.shape), s.reshape(-1, 1)


# ------------------------------------------------------------------------ torch glue
def tag_of(t) -> str:
    import torch
    return {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}[t.dtype]


def to_np(t) -> np.ndarray:
    """torch tensor -> numpy; 16-bit floats are widened (exactly) to float32."""
    import torch
    t = t.detach().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        t = t.float()
    return t.contiguous().numpy()
