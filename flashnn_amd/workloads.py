"""Seeded synthetic inputs for the benchmark configurations (CPU tensors; callers move
them to the GPU).  Shapes and distributions follow the configurations the benchmark and
the parity tests are quoted on."""
import math

import torch


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def activations(M, K, dtype, seed=0, outlier_frac=0.0, outlier_gain=20.0):
    """~N(0,1) activations; optionally a fixed random subset of channels scaled up."""
    g = _gen(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    if outlier_frac > 0:
        n_out = math.ceil(outlier_frac * K)
        cols = torch.randperm(K, generator=g)[:n_out]
        x[:, cols] *= outlier_gain
    return x.to(dtype)


def int8_weights(N, K, seed=1):
    """int8 weights uniform in [-127, 127] and per-output-channel fp32 scales U(1e-3, 1e-2)."""
    g = _gen(seed)
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    s = torch.empty(N, dtype=torch.float32).uniform_(1e-3, 1e-2, generator=g)
    return w, s


def int4_group_weights(N, K, group, scale_dtype=torch.float16, seed=2):
    """uint4 weights with per-group scales and uint4 zero points, expressed through the
    operator's signed-nibble layout: returns (packed [N/2,K] int8, scales [K/group,N],
    zero_points [K/group,N] as scale_dtype, u4 [N,K] uint8, zp_u4 [K/group,N] uint8).

    A uint4 value u with zero point z equals the signed nibble (u - 8) with zero point
    (z - 8): (u - 8) - (z - 8) = u - z.  Row j of the packed matrix holds channel 2j in the
    low nibble and channel 2j+1 in the high nibble."""
    g = _gen(seed)
    u = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    zp = torch.randint(0, 16, (K // group, N), generator=g, dtype=torch.uint8)
    s = torch.empty(K // group, N, dtype=torch.float32).uniform_(1e-3, 1e-2, generator=g).to(scale_dtype)
    nib = (u.to(torch.int16) - 8) & 0xF
    packed = (nib[0::2] | (nib[1::2] << 4)).to(torch.uint8).view(torch.int8).contiguous()
    zp_ref = (zp.to(torch.float32) - 8).to(scale_dtype)
    return packed, s, zp_ref, u, zp


def rmsnorm_gamma(K, seed=3):
    g = _gen(seed)
    return torch.empty(K, dtype=torch.float32).uniform_(0.5, 1.5, generator=g)


# (K, N) of the Llama-7B-like linear layers used for the A8W8 prefill configuration
A8W8_PREFILL_SHAPES = {"qkv": (4096, 12288), "o": (4096, 4096), "gate_up": (4096, 22016),
                       "down": (11008, 4096)}
A16W8_DECODE_SHAPES = [(4096, 4096), (4096, 11008), (11008, 4096)]
A16W4_SHAPE = (8192, 28672)


def sharded_model_gemm_shapes():
    """(N, K) of the four linear layers of the sharded decoder models the reference's A8W8 sweep
    walks (benchmark/benchmark_gemm_a8w8_amd.py:19-34): FFN up, FFN gate+down input, attention
    output and QKV projection, for (hidden, intermediate, shards, heads, kv_heads)."""
    shapes = []
    for hidden, inter, tp, heads, kv_heads in [(13312, 71168, 8, 104, 8), (13312, 71168, 4, 104, 4),
                                               (8192, 29568, 4, 64, 8), (8192, 29568, 2, 64, 8),
                                               (3584, 18944, 1, 28, 4)]:
        gqa = heads // kv_heads
        shapes += [(hidden, inter // tp), ((inter // tp) * 2, hidden), (hidden, hidden // tp),
                   ((hidden // tp) + ((hidden // tp) // gqa) * 2, hidden)]
    return shapes


# activation row counts of both reference sweeps (benchmark_gemm_a8w8_amd.py:42,
# benchmark_dynamic_quant.py:14) and the row lengths of the dynamic-quant sweep (:10)
SWEEP_M = [1, 10, 20, 30, 40, 764, 1024, 2048, 4096, 8192]
DYNAMIC_QUANT_SWEEP_K = [1664, 3328, 8896, 13312, 17792, 35584]


def moe_align_block_size(topk_ids, block_size, num_experts):
    """Groups the routed rows by expert the way callers of fused_moe_*_forward prepare them (the
    reference ships no such helper; its launcher's docstring describes the layout,
    flashnn/triton_kernels/fused_moe_a8w8.py:203-207): returns int32 tensors
    (sorted_token_ids [numel + num_experts*(block_size-1)], expert_ids [len(sorted)/block_size],
    num_tokens_post_padded [1]).  Routed row i = position in topk_ids.flatten(); each expert's rows are
    listed in ascending order and padded with numel to a multiple of block_size; the unused tail of
    sorted_token_ids holds numel and the unused tail of expert_ids holds 0."""
    flat = topk_ids.flatten().to(torch.int64)
    numel = flat.numel()
    cap = numel + num_experts * (block_size - 1)
    cap = (cap + block_size - 1) // block_size * block_size
    sorted_ids = torch.full((cap,), numel, dtype=torch.int32)
    expert_ids = torch.zeros(cap // block_size, dtype=torch.int32)
    pos = 0
    for e in range(num_experts):
        rows = torch.nonzero(flat == e).flatten()
        n = rows.numel()
        if n == 0:
            continue
        sorted_ids[pos:pos + n] = rows.to(torch.int32)
        padded = (n + block_size - 1) // block_size * block_size
        expert_ids[pos // block_size:(pos + padded) // block_size] = e
        pos += padded
    return sorted_ids, expert_ids, torch.tensor([pos], dtype=torch.int32)
