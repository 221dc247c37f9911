"""Torch-op restatement of the reference's torch path.  TEST INFRASTRUCTURE ONLY.

These functions call the same torch primitives, in the same order, as the reference's
`_torch_impl` methods, so that (a) the explicit-rounding oracle in flashnn_oracle.py can
be checked against the third-party arithmetic the reference really runs, and (b)
bench.py can time the reference's CPU path on the host cores.  Imported only by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg.
"""
import torch


def dynamic_quantize(x):
    """flashnn/quant_gemm.py:53-57."""
    mx = x.abs().max(-1, keepdim=True)[0]
    scale = mx / 127.0
    out = torch.round(x / scale)
    return out.to(torch.int8), scale.half().squeeze(-1)


def gemm_a8w8(a, b, alpha_row, alpha_col, out_ty):
    """flashnn/quant_gemm.py:96-104 (fp32 matmul, scale outer product in the scale type)."""
    x = torch.matmul(a.to(torch.float32), b.transpose(0, 1).to(torch.float32))
    scale = torch.matmul(torch.squeeze(alpha_row).flatten().unsqueeze(-1),
                         torch.squeeze(alpha_col).flatten().unsqueeze(0))
    return torch.mul(x, scale).to(out_ty)


def _channel_dequantize(x, scales, zero_points=None):
    """flashnn/quant_gemm.py:14-17."""
    if zero_points is None:
        zero_points = torch.zeros_like(scales)
    return (x - zero_points) * scales


def _block_dequantize(x, scales, block_size, zero_points=None):
    """flashnn/quant_gemm.py:20-36 (result buffer is float16)."""
    res = torch.zeros_like(x, dtype=torch.half)
    if zero_points is None:
        zero_points = torch.zeros_like(scales)
    for i in range(scales.shape[0]):
        blk = x[i * block_size:(i + 1) * block_size, :]
        res[i * block_size:(i + 1) * block_size, :] = (blk - zero_points[i]) * scales[i]
    return res


def unpack_int4(quant_w):
    """flashnn/quant_gemm.py:175-190: [N/2,K] bytes -> [K,N] int8 in [-8,7]."""
    lo = (quant_w & 0x0F).to(torch.int8)
    lo = torch.where(lo > 7, lo | 0xF0, lo).to(torch.int8).transpose(0, 1)
    hi = (((quant_w & 0xF0) >> 4) & 0x0F).to(torch.int8)
    hi = torch.where(hi > 7, (hi | 0xF0).to(torch.int8), hi).to(torch.int8).transpose(0, 1)
    b = torch.stack((lo, hi), dim=2)
    return b.view(lo.size(0), -1)


def gemm_weight_only(act, quant_w, scale_w, bias, zero_points, out_ty):
    """flashnn/quant_gemm.py:148-206."""
    if quant_w.size(0) == scale_w.size(-1):
        w = quant_w.transpose(0, 1)
        int4 = False
    elif quant_w.size(0) * 2 == scale_w.size(-1):
        w = unpack_int4(quant_w)
        int4 = True
    else:
        raise AssertionError("Gemm WeightOnly only support int8 or int4x2")
    scale_w = scale_w.squeeze()
    if scale_w.dim() == 1:
        dq = _channel_dequantize(w, scale_w.unsqueeze(0), zero_points=zero_points)
    else:
        dq = _block_dequantize(w, scale_w, int(act.shape[1] / scale_w.shape[0]),
                               zero_points=zero_points)
    out = torch.matmul(act.to(torch.float32), dq.to(torch.float32))
    if int4:
        if bias is not None:
            out += bias
        return out.to(out_ty)
    out = out.to(out_ty)
    if bias is not None:
        out += bias
    return out.to(out_ty)


def rmsnorm_dquant(x, weight, eps):
    """flashnn/norm.py:45-60."""
    xf = x.float()
    n = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    n *= weight
    mx = torch.max(torch.abs(n), dim=-1, keepdim=True)[0]
    scale = mx / 127.0
    q = torch.clamp(torch.round(n / scale), -128.0, 127.0)
    return q.to(torch.int8), scale.reshape(x.shape[:-1]).type_as(x)


def rmsnorm(x, weight, eps):
    """flashnn/norm.py:25-33, cast to the input type as the Triton path returns it (:29)."""
    xf = x.float()
    n = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)
    return (n * weight).type_as(x)


def layernorm(x, weight, bias, eps):
    """flashnn/norm.py:82-85."""
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), weight, bias, eps)


def layernorm_dquant(x, weight, bias, eps):
    """flashnn/norm.py:112-119."""
    n = torch.nn.functional.layer_norm(x, (x.shape[-1],), weight, bias, eps)
    mx = torch.max(torch.abs(n), dim=-1, keepdim=True)[0]
    scale = mx / 127.0
    q = torch.clamp(torch.round(n / scale), -128.0, 127.0)
    return q.to(torch.int8), scale.reshape(-1, 1)
