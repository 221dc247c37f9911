// Argument block and output modes shared by the A8W8 GEMM kernels.
#pragma once

#include "fnn_common.h"
#include "moe_common.h"

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
    int gn;                 // tile columns per group of the tile numbering
    // K cut into kparts ranges of k_chunk bytes per row (the tiled kernel's split form only)
    int kparts, k_chunk;
    int* ws_count;          // one ticket counter per tile, zero between calls
    int32_t* ws_part;       // kparts slots of tile-rows x tile-columns accumulators per tile
};

// gemm_a8w8_skinny.hip: up to 64 activation rows, the weights streamed once (its panel form also takes up to
// kA8PanelRowsNarrow rows, in passes of 64); false if the shape does not suit it
constexpr int kA8PanelRowsNarrow = 256;
bool launch_a8w8_skinny(A8W8Args& p, int mode, hipStream_t st);
// the same kernel over gathered rows (p.M is ignored); false if the shape does not suit it
bool launch_a8w8_moe(A8W8Args& p, const MoeArgs& q, int mode, hipStream_t st);

}  // namespace fnn
