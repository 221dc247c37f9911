// Argument block and output modes shared by the A8W8 GEMM kernels.
#pragma once

#include "fnn_common.h"

namespace fnn {

enum { OUT_F16 = 0, OUT_BF16 = 1, OUT_I32 = 2 };

struct A8W8Args {
    const int8_t* a;
    const int8_t* b;
    void* out;
    const void* arow;
    const void* acol;
    int M, N, K;
    int64_t lda, ldb, ldc;
    int out_dtype, arow_dtype, acol_dtype;
    int tiles_m, tiles_n, tiles_per_xcd;
};

// Mixture-of-experts form of the few-row kernel: the activation rows of a pass are gathered through a
// sorted token list, every block of block_m sorted rows multiplies one expert's weight matrix, and
// the output rows are scattered back by token id (flashnn/triton_kernels/fused_moe_a8w8.py:37-173).
struct MoeArgs {
    const int32_t* sorted_ids;   // [EM] token ids (index into the M*top_k routed rows); >= num_valid: padding
    const int32_t* expert_ids;   // [EM / block_m]
    const int32_t* ntpp;         // [1] number of sorted rows in use (a multiple of block_m)
    const void* topk_w;          // [M*top_k] routing weights, or unused
    int topk_w_dtype, mul_w, top_k, block_m, num_valid, EM;
    int64_t stride_be;           // bytes (= elements) between the weight matrices of two experts
    int64_t stride_scale_be;     // elements between the column scales of two experts
};

// gemm_a8w8_skinny.hip: up to 64 activation rows, the weights streamed once; false if the shape
// does not suit it
bool launch_a8w8_skinny(A8W8Args& p, int mode, hipStream_t st);
// the same kernel over gathered rows (p.M is ignored); false if the shape does not suit it
bool launch_a8w8_moe(A8W8Args& p, const MoeArgs& q, int mode, hipStream_t st);

}  // namespace fnn
