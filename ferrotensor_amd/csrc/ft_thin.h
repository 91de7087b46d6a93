// Batched rank-r (thin) products of the LoRA linears; see ft_thin.hip.
#pragma once

#include "ft_common.h"

constexpr int FT_THIN_MAX_BATCH = 8;

struct ft_thin_problem {
    const float* x;   // row-wise: [M, K] (ldx);          col-wise: [M, R] (ldx)
    const float* y;   // row-wise: [K, C] or [C, K] (ldy); col-wise: [M, C] (ldy)
    float* out;       // row-wise: [M, C] (ldo);          col-wise: [R, C] or [C, R] (ldo)
    int M, K, R, C;
    long ldx, ldy, ldo;
    float scale;
    int y_transposed;    // row-wise only
    int out_transposed;  // col-wise only
    long scratch_offset; // filled in by ft_thin_colwise
    int accumulate;      // col-wise only: out += result (gradient accumulation) instead of out = result
};

bool ft_thin_rank_supported(size_t r);
bool ft_thin_rowwise_ok(const ft_thin_problem& p);
bool ft_thin_colwise_ok(const ft_thin_problem& p);
// One launch for up to FT_THIN_MAX_BATCH independent products of equal rank.
int ft_thin_rowwise(ft_context* ctx, const ft_thin_problem* probs, int count);
int ft_thin_colwise(ft_context* ctx, const ft_thin_problem* probs, int count);
