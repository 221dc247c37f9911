"""The operators of this package written with plain torch tensor operations: what a module computes after
set_use_triton(False), on any device.  One function per formula, shared by the modules that need it; each
names the reference lines whose results it reproduces.  Nothing here is used by the native path."""
import torch

INT8_LO, INT8_HI = -128, 127


def rows_to_int8(x, scale_shape=None):
    """Symmetric per-row quantisation in x's own dtype: scale = max|row| / 127, q = round(x / scale) kept
    inside int8.  The division and the rounding happen in x.dtype, so a half input is rounded twice, as in
    flashnn/quant_gemm.py:47-51 (DynamicQuantize), flashnn/norm.py:51-56 and :115-119 (the two fused norms,
    which pass fp32).  For bf16 the quotient of the row maximum can round up to 128: it is held at 127,
    where a bare cast to int8 would wrap to -128.  Returns (int8 like x, scale [rows, 1] in x.dtype)."""
    scale = torch.amax(x.abs(), dim=-1, keepdim=True).div(127.0)
    q = torch.div(x, scale).round_().clamp_(INT8_LO, INT8_HI).to(torch.int8)
    if scale_shape is not None:
        scale = scale.reshape(scale_shape)
    return q, scale


def rms_normalise(x32, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, on an fp32 tensor (flashnn/norm.py:25-26)."""
    return x32 * torch.rsqrt(torch.mean(x32 * x32, dim=-1, keepdim=True).add_(eps))


def rmsnorm(x, weight, eps):
    """flashnn/norm.py:31-33: normalise in fp32, return to x.dtype, then multiply by the weight."""
    return rms_normalise(x.float(), eps).to(x.dtype) * weight


def rmsnorm_to_int8(x, weight, eps):
    """flashnn/norm.py:46-60: fp32 RMS norm times weight, then per-row int8; scale [rows] in x.dtype."""
    y = rms_normalise(x.float(), eps).mul_(weight)
    q, scale = rows_to_int8(y, x.shape[:-1])
    return q, scale.to(x.dtype)


def layernorm(x, dims, weight, bias, eps):
    """flashnn/norm.py:82-83."""
    return torch.nn.functional.layer_norm(x, dims, weight, bias, eps)


def layernorm_to_int8(x, dims, weight, bias, eps):
    """flashnn/norm.py:112-120: layer norm in x.dtype, then per-row int8; scale [rows, 1]."""
    return rows_to_int8(layernorm(x, dims, weight, bias, eps), (-1, 1))


def a8w8(a, b, alpha_row, alpha_col, out_ty):
    """flashnn/quant_gemm.py:95-101: the integer product through fp32, times the outer product of the two
    scale vectors (formed first, in the scales' dtype), cast to out_ty."""
    acc = a.float() @ b.float().t()
    outer = alpha_row.reshape(-1, 1) * alpha_col.reshape(1, -1)
    return (acc * outer).to(out_ty)


def unpack_int4_rows(packed):
    """int8 [N/2, K] holding two signed nibbles per byte -> int8 [K, N], the low nibble in the even
    column (flashnn/quant_gemm.py:171-181).  Arithmetic shifts on int8 sign-extend the nibbles."""
    lo = (packed << 4) >> 4
    hi = packed >> 4
    return torch.stack((lo.t(), hi.t()), dim=2).reshape(packed.shape[1], -1)


def dequantize_per_channel(w_kn, scales, zero_points):
    """(w - zp) * s with [1, N] tables, in the tables' dtype (flashnn/quant_gemm.py:14-17)."""
    return (w_kn if zero_points is None else w_kn - zero_points) * scales


def dequantize_per_block(w_kn, scales, zero_points, block):
    """(w - zp) * s with [K/block, N] tables, returned as fp16 (flashnn/quant_gemm.py:20-36)."""
    assert w_kn.dim() == 2, "block_fake_quant only support tensor with dim=2."
    assert w_kn.shape[0] // block == scales.shape[0]
    K, N = w_kn.shape
    g = w_kn.reshape(K // block, block, N)
    if zero_points is not None:
        g = g - zero_points.unsqueeze(1)
    return (g * scales.unsqueeze(1)).reshape(K, N).to(torch.half)


def weight_only(act, w_kn, scale_w, bias, zero_points, out_ty, round_before_bias):
    """flashnn/quant_gemm.py:183-203: dequantise, multiply in fp32, add the bias.  round_before_bias: the
    int8 path casts the product to out_ty before the bias is added, the int4 path after."""
    s = scale_w.squeeze()
    if s.dim() == 1:
        dq = dequantize_per_channel(w_kn, s.unsqueeze(0), zero_points)
    else:
        dq = dequantize_per_block(w_kn, s, zero_points, act.shape[1] // s.shape[0])
    out = act.float() @ dq.float()
    if round_before_bias:
        out = out.to(out_ty)
    if bias is not None:
        out += bias
    return out.to(out_ty)
