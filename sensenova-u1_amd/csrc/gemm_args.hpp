// Argument block shared by the dequant-GEMM kernels.
#pragma once

#include "sngguf_common.hpp"

namespace sngguf {

// The M rows are seen through an optional row map as [group 0 | group 1]; group 0 multiplies
// weight set 0 (text rows -> understanding weights), group 1 weight set 1 (image rows ->
// generation weights).  A plain linear is "all rows in group 0, no map".
struct GemmArgs {
    const bf16_t* x;
    bf16_t* y;
    int64_t M, N, K;
    const int32_t* rowmap;  // M entries, grouped order -> row of x / y; NULL = identity
    const int32_t* n0_dev;  // device count of group-0 rows; NULL = use n0
    int64_t n0;
    const uint8_t* q[2];
    const bf16_t* bias[2];
    const bf16_t* residual; // [M][N] added to the rounded projection output (same rows as y), or NULL
    int group_mask;         // bit g: rows of group g are computed by this launch
    // Split of K over workgroups (large-tile kernel only): with ksplit > 1 every output tile is computed by ksplit
    // workgroups, each over its share of the K steps, and written as fp32 partial sums to partial[slice][M][N]
    // (no bias, no residual, nothing written to y); a second kernel adds the slices up.
    float* partial;
    int ksplit;
    // Gated pair (four-wavefront dense kernel only): the N weight rows are blocks of 128 gate rows, each followed by the
    // 128 up rows of the same output columns, and y is [M][gated_cols]: silu(gate) * up, rounded as the decode kernels'
    // gated pair rounds (no bias, no residual, no K split).  0 = a plain projection.
    int64_t gated_cols;
};

}  // namespace sngguf
