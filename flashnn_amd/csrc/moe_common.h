// Gather/scatter description shared by the mixture-of-experts forms of the few-row GEMM kernels.
#pragma once

#include "fnn_common.h"

namespace fnn {

// Mixture-of-experts form of the few-row kernels: the activation rows of a pass are gathered through a
// sorted token list, every block of block_m sorted rows multiplies one expert's weight matrix, and
// the output rows are scattered back by token id (flashnn/triton_kernels/fused_moe_a8w8.py:37-173, fused_moe_a16w4.py:50-206).
struct MoeArgs {
    const int32_t* sorted_ids;   // [EM] token ids (index into the M*top_k routed rows); >= num_valid: padding
    const int32_t* expert_ids;   // [EM / block_m]
    const int32_t* ntpp;         // [1] number of sorted rows in use (a multiple of block_m)
    const void* topk_w;          // [M*top_k] routing weights, or unused
    int topk_w_dtype, mul_w, top_k, block_m, num_valid, EM;
    int64_t stride_be;           // bytes (= elements) between the weight matrices of two experts
    int64_t stride_scale_be;     // elements between the column scales of two experts
    int64_t stride_zp_be;        // ... and between their zero points (weight-only form)
    // weight-only form: element strides of scale[e, n, kblock] and zero_point[e, n, kblock]
    int64_t stride_scale_n, stride_scale_k, stride_zp_n, stride_zp_k;
};

}  // namespace fnn
