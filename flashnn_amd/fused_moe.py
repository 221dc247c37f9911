"""Mixture-of-experts grouped GEMMs with the reference's launcher signatures: int8 tokens on int8
expert weights (flashnn/triton_kernels/fused_moe_a8w8.py:176-290) and fp16/bf16 tokens on int4 expert
weights (fused_moe_a16w4.py:326-466), exported at flashnn/__init__.py:14-15."""
import torch

from . import _lib


def fused_moe_a8w8_forward(A, B, C, alpha_row_ptr, alpha_col_ptr, topk_weights, topk_ids, sorted_token_ids,
                           expert_ids, num_tokens_post_padded, mul_routed_weight, top_k, BM):
    """C[t] <- scale(A[t // top_k] x B[e]^T) for every routed row t listed in sorted_token_ids.

    A: int8 [M, K] tokens; B: int8 [E, N, K]; C: fp16/bf16 [M, top_k, N], written in place;
    alpha_row_ptr: [M] scales of A's rows; alpha_col_ptr: [E, N] scales of B's rows; topk_weights,
    topk_ids: [M, top_k]; sorted_token_ids: int32 [EM] routed-row ids grouped by expert and padded
    with M*top_k to blocks of BM; expert_ids: int32 [EM / BM]; num_tokens_post_padded: int32 [1];
    BM: the block size the sorted list was aligned to.  Argument meaning and asserts follow the
    reference launcher; unlike it, C may be bfloat16 and the scale types are free.
    """
    assert topk_weights.stride(1) == 1
    assert sorted_token_ids.stride(0) == 1
    assert B.shape[1] % 16 == 0 and B.shape[2] % 16 == 0
    assert A.dtype == torch.int8 and B.dtype == torch.int8, "Matrix A/B must be int8 type"
    assert C.dtype in (torch.float16, torch.bfloat16), "Output type must be float16 or bfloat16"
    assert A.dim() == 2 and B.dim() == 3 and A.shape[1] == B.shape[2], "Matrix B must be transposed"
    assert A.stride(1) == 1 and B.stride(2) == 1 and C.stride(-1) == 1
    for name, t in (("sorted_token_ids", sorted_token_ids), ("expert_ids", expert_ids),
                    ("num_tokens_post_padded", num_tokens_post_padded)):
        assert t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be a contiguous int32 tensor"
    _lib.require_gpu(A, B, C, alpha_row_ptr, alpha_col_ptr, topk_weights, sorted_token_ids, expert_ids,
                     num_tokens_post_padded)
    N, K = B.shape[1], B.shape[2]
    EM, num_valid_tokens = sorted_token_ids.shape[0], topk_ids.numel()
    assert C.numel() == num_valid_tokens * N or C.stride(-2) >= N
    assert alpha_row_ptr.is_contiguous() and alpha_row_ptr.numel() == A.shape[0]
    assert alpha_col_ptr.stride(-1) == 1 and alpha_col_ptr.shape[-1] == N
    assert topk_weights.is_contiguous()
    ldc = C.stride(-2)
    if C.dim() == 3:
        assert C.stride(0) == C.shape[1] * ldc, "C must be addressable as [M * top_k, N] rows"
    lib = _lib.load()
    _lib.check(lib.fnn_fused_moe_a8w8(
        _lib.ptr(C), _lib.ptr(A), _lib.ptr(B), _lib.ptr(alpha_row_ptr), _lib.ptr(alpha_col_ptr),
        _lib.ptr(topk_weights), _lib.ptr(sorted_token_ids), _lib.ptr(expert_ids), _lib.ptr(num_tokens_post_padded),
        N, K, EM, num_valid_tokens, A.stride(0), B.stride(0), B.stride(1), ldc,
        alpha_col_ptr.stride(0) if alpha_col_ptr.dim() == 2 else 0, 1 if mul_routed_weight else 0, int(top_k),
        int(BM), _lib.dtype_code(C.dtype), _lib.dtype_code(alpha_row_ptr.dtype),
        _lib.dtype_code(alpha_col_ptr.dtype), _lib.dtype_code(topk_weights.dtype), _lib.current_stream(A.device)))
    return C


def fused_moe_a16w4_forward(A, B, C, scale_b, zero_points, topk_weights, topk_ids, sorted_token_ids, expert_ids,
                            num_tokens_post_padded, mul_routed_weight, top_k, BM):
    """C[t] <- A[t // top_k] x dequant(B[e])^T for every routed row t listed in sorted_token_ids.

    A: fp16/bf16 [M, K]; B: int8-typed [E, N, K] holding two int4 output channels per byte (low nibble:
    channel 2j); C: [M, top_k, 2N] of A's type, written in place; scale_b / zero_points: [E, 2N] (per
    channel) or [E, 2N, K // block] (per K block), zero_points may be None and may be int8 or floating;
    routing arguments as for fused_moe_a8w8_forward.  Argument meaning and asserts follow the reference
    launcher (fused_moe_a16w4.py:366-383)."""
    assert topk_weights.stride(1) == 1
    assert sorted_token_ids.stride(0) == 1
    assert B.shape[1] % 16 == 0 and B.shape[2] % 16 == 0
    assert B.dtype == torch.int8, "Weight must be int8 type"
    assert A.dtype in (torch.float16, torch.bfloat16) and C.dtype == A.dtype
    assert A.dim() == 2 and B.dim() == 3 and A.shape[1] == B.shape[2], "Matrix B must be transposed"
    assert A.stride(1) == 1 and B.stride(2) == 1 and C.stride(-1) == 1
    for name, t in (("sorted_token_ids", sorted_token_ids), ("expert_ids", expert_ids),
                    ("num_tokens_post_padded", num_tokens_post_padded)):
        assert t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be a contiguous int32 tensor"
    _lib.require_gpu(A, B, C, scale_b, zero_points, topk_weights, sorted_token_ids, expert_ids,
                     num_tokens_post_padded)
    N, K = B.shape[1], B.shape[2]
    EM, num_valid_tokens = sorted_token_ids.shape[0], topk_ids.numel()
    is_perchannel = scale_b.dim() == 2          # (E, 2N)
    assert scale_b.shape[1] == 2 * N and (zero_points is None or zero_points.shape == scale_b.shape)
    group = 0 if is_perchannel else K // scale_b.shape[-1]
    assert topk_weights.is_contiguous()
    ldc = C.stride(-2)
    if C.dim() == 3:
        assert C.stride(0) == C.shape[1] * ldc, "C must be addressable as [M * top_k, 2N] rows"

    def strides(t):
        if t is None:
            return 0, 0, 0
        return t.stride(0), t.stride(1), (0 if t.dim() == 2 else t.stride(2))

    zp_code = 0
    if zero_points is not None:
        zp_code = _lib.FNN_I8 if zero_points.dtype == torch.int8 else _lib.dtype_code(zero_points.dtype)
    lib = _lib.load()
    _lib.check(lib.fnn_fused_moe_a16w4(
        _lib.ptr(C), _lib.ptr(A), _lib.ptr(B), _lib.ptr(scale_b), _lib.ptr(zero_points), _lib.ptr(topk_weights),
        _lib.ptr(sorted_token_ids), _lib.ptr(expert_ids), _lib.ptr(num_tokens_post_padded),
        N, K, EM, num_valid_tokens, A.stride(0), B.stride(0), B.stride(1), ldc, *strides(scale_b),
        *strides(zero_points), group, 1 if mul_routed_weight else 0, int(top_k), int(BM),
        _lib.dtype_code(A.dtype), _lib.dtype_code(scale_b.dtype), zp_code, _lib.dtype_code(topk_weights.dtype),
        _lib.current_stream(A.device)))
    return C
