// Argument block and entry points shared by the attention sources
// (ft_attention.hip: general head dims and the 32-row kernels; ft_attention16.hip:
// the 16-row kernels for whole, aligned head dims).
#pragma once

#include "ft_common.h"

constexpr float kAttnMasked = -1.0e30f;   // scores at or below this are treated as -inf
constexpr float kAttnLseEmpty = 3.0e38f;  // log-sum-exp of a row with no visible key

struct AttnArgs {
    const float* q;
    const float* k;
    const float* v;
    const float* out;
    const float* d_out;
    float* o;
    float* dq;
    float* dk;
    float* dv;
    float* stats;
    int B, Sq, Sk, H, Hkv, D;
    int causal, causal_offset;
    float scale;
    // Backward only, head_dim 64: when set, dQ and dK leave the kernels already rotated back
    // through RoPE (the inverse rotation by the (cos, sin) of their token position, table
    // [Sq or Sk][32] float2), which is what RoPENode::backward does to them next.
    const float2* rope;
    // dK/dV with one workgroup per query head instead of per kv head: that head's unscaled sums
    // go to part[2 * g + {0: dK, 1: dV}] (each laid out like dk), and attn_dkdv_combine_kernel
    // adds the group in head order.
    float* part;
    int split_g;
};

constexpr size_t kAttnScratchFloats = (size_t)8 << 20;  // 32 MiB of per-head partial dK/dV

// ft_attention16.hip. `usable`: head dim 64, every tensor 16-byte aligned.
bool ft_attn16_usable(const AttnArgs& a);
// Do the forward / dQ kernels have enough workgroups at this shape to beat the 32-row kernels?
// (The dK/dV kernel always does.)
bool ft_attn16_forward_pays(const ft_context* ctx, const AttnArgs& a);
bool ft_attn16_backward_dq_pays(const ft_context* ctx, const AttnArgs& a);
int ft_attn16_forward(ft_context* ctx, const AttnArgs& a);
int ft_attn16_backward_dq(ft_context* ctx, const AttnArgs& a);
int ft_attn16_backward_dkdv(ft_context* ctx, const AttnArgs& a);

// ft_attention.hip: dk = scale * (sum over the group's heads of part[2g]) rotated back when asked,
// dv = sum of part[2g + 1].
int ft_attn_dkdv_combine(ft_context* ctx, const AttnArgs& a, int DP);
