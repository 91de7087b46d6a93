// Causal / full grouped-query flash attention, forward and backward, on the
// gfx950 f32 matrix cores (v_mfma_f32_32x32x2_f32).
//
// Layout (as the reference): q/out/dO/dq [B,Sq,H,D], k/v/dk/dv [B,Sk,Hkv,D],
// kv head = h / (H/Hkv); query i sits at position i + causal_offset; stats
// [B*H*Sq][2] = (Delta, log-sum-exp) per query row.
//
// All three kernels compute the score block transposed, S^T = K Q^T, so that a
// lane's 16 accumulator registers hold 16 keys of ONE query (column = lane%32).
// That makes the online-softmax statistics per-lane scalars (one cross-half
// shuffle finishes a row reduction), and the accumulator registers are already
// in the operand layout of the next MFMA (P^T as the B operand of O^T = V^T P^T),
// so P never leaves registers. K/V (or Q/dO) tiles of 32 rows are staged in LDS.
#include "ft_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr float kMasked = -1.0e30f;   // scores at or below this are treated as -inf
constexpr float kLseEmpty = 3.0e38f;  // log-sum-exp of a row with no visible key

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
};

#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)

__device__ __forceinline__ floatx16 zero16() {
    floatx16 z;
#pragma unroll
    for (int r = 0; r < 16; r++) z[r] = 0.0f;
    return z;
}

// Four consecutive head-dim values of one row, zero past D or for an invalid row.
__device__ __forceinline__ float4 load_row4(const float* row, int d, int D, bool row_ok) {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!row_ok) return r;
    if (d + 4 <= D && ((((uintptr_t)(row + d)) & 15) == 0)) return *reinterpret_cast<const float4*>(row + d);
    if (d + 0 < D) r.x = row[d + 0];
    if (d + 1 < D) r.y = row[d + 1];
    if (d + 2 < D) r.z = row[d + 2];
    if (d + 3 < D) r.w = row[d + 3];
    return r;
}

// Accumulator register t of a lane in half `half` belongs to row key_of(t, half)
// of the 32-row block (the MFMA output layout), which is also the k index the
// lane must supply when the register is reused as a B operand.
__device__ __forceinline__ int row_of(int t, int half) { return (t / 4) * 8 + half * 4 + (t % 4); }

// Stage a 32 x DP tile (rows r0.., head hh of a [.., S, heads, D] tensor) into
// LDS with row stride DP+4, zero filled outside S or D. NT threads cooperate.
template <int DP, int NT>
__device__ __forceinline__ void stage_tile(float* lds, const float* base, int b, int S, int heads, int hh, int D,
                                           int r0, int tid) {
    constexpr int LD = DP + 4;
    constexpr int V4 = 32 * DP / 4;
    for (int e = tid; e < V4; e += NT) {
        const int r = e / (DP / 4), c = (e % (DP / 4)) * 4;
        const int row = r0 + r;
        const bool ok = row < S;
        const float* src = base + (((long)b * S + (ok ? row : 0)) * heads + hh) * D;
        *reinterpret_cast<float4*>(lds + r * LD + c) = load_row4(src, c, D, ok);
    }
}

// ---------------------------------------------------------------------------
// Forward. Grid (ceil(Sq / (32*NW)), B*H); each wave owns 32 queries.
// ---------------------------------------------------------------------------
template <int DP, int NW>
__global__ __launch_bounds__(NW * 64) void attn_fwd_kernel(AttnArgs p) {
    constexpr int LD = DP + 4;
    constexpr int NF = DP / 32;  // 32-row blocks of the head dim
    constexpr int NS = DP / 8;   // k-steps of 8 over the head dim
    __shared__ __attribute__((aligned(16))) float Ks[32 * LD];
    __shared__ __attribute__((aligned(16))) float Vs[32 * LD];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int l32 = lane % 32, half = lane / 32;
    const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
    const int kvh = h / (p.H / p.Hkv);
    const int q_wg0 = blockIdx.x * (32 * NW);
    const int q0 = q_wg0 + wave * 32;
    const int qi = q0 + l32;
    const bool q_ok = qi < p.Sq;
    const float* qrow = p.q + (((long)b * p.Sq + (q_ok ? qi : 0)) * p.H + h) * p.D;

    float4 qreg[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        float4 t = load_row4(qrow, 8 * s + 4 * half, p.D, q_ok);
        qreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
    }
    floatx16 o[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) o[f] = zero16();
    float m_run = kMasked, l_run = 0.0f;

    // Keys any query of this workgroup can see (uniform: every wave runs the
    // same number of tiles and meets the same barriers).
    int q_last_wg = q_wg0 + 32 * NW - 1;
    if (q_last_wg > p.Sq - 1) q_last_wg = p.Sq - 1;
    int k_end = p.Sk;
    if (p.causal && q_last_wg + p.causal_offset + 1 < k_end) k_end = q_last_wg + p.causal_offset + 1;
    const int q_last_wave = q0 + 31 + p.causal_offset;  // last position this wave can see when causal
    const int q_pos = qi + p.causal_offset;

    for (int kb = 0; kb < k_end; kb += 32) {
        __syncthreads();
        stage_tile<DP, NW * 64>(Ks, p.k, b, p.Sk, p.Hkv, kvh, p.D, kb, tid);
        stage_tile<DP, NW * 64>(Vs, p.v, b, p.Sk, p.Hkv, kvh, p.D, kb, tid);
        __syncthreads();
        if (q0 >= p.Sq || (p.causal && kb > q_last_wave)) continue;  // wave-uniform

        floatx16 s = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            const float4 a = *reinterpret_cast<const float4*>(Ks + l32 * LD + 8 * st + 4 * half);
            s = MFMA(a.x, qreg[st].x, s);
            s = MFMA(a.y, qreg[st].y, s);
            s = MFMA(a.z, qreg[st].z, s);
            s = MFMA(a.w, qreg[st].w, s);
        }
        float tile_max = kMasked;
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int key = kb + row_of(t, half);
            const bool vis = q_ok && key < p.Sk && (!p.causal || key <= q_pos);
            s[t] = vis ? s[t] : kMasked;
            tile_max = fmaxf(tile_max, s[t]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
        const float m_new = fmaxf(m_run, tile_max);
        const float corr = __expf(m_run - m_new);
        float psum = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const float pj = s[t] > kMasked ? __expf(s[t] - m_new) : 0.0f;
            s[t] = pj;
            psum += pj;
        }
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * corr + psum;
        m_run = m_new;
#pragma unroll
        for (int f = 0; f < NF; f++) {
#pragma unroll
            for (int r = 0; r < 16; r++) o[f][r] *= corr;
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const float a = Vs[row_of(t, half) * LD + f * 32 + l32];
                o[f] = MFMA(a, s[t], o[f]);
            }
        }
    }

    if (!q_ok) return;
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    float* orow = p.o + (((long)b * p.Sq + qi) * p.H + h) * p.D;
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
            const int d = f * 32 + r4 * 8 + half * 4;
            if (d + 4 <= p.D && ((((uintptr_t)(orow + d)) & 15) == 0)) {
                *reinterpret_cast<float4*>(orow + d) = make_float4(o[f][r4 * 4 + 0] * inv, o[f][r4 * 4 + 1] * inv,
                                                                   o[f][r4 * 4 + 2] * inv, o[f][r4 * 4 + 3] * inv);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (d + e < p.D) orow[d + e] = o[f][r4 * 4 + e] * inv;
            }
        }
    if (p.stats && half == 0)
        p.stats[2 * (((long)b * p.H + h) * p.Sq + qi) + 1] = l_run > 0.0f ? m_run + __logf(l_run) : kLseEmpty;
}

// ---------------------------------------------------------------------------
// Backward, pass 1: Delta = dO.O (stored in stats slot 0) and
// dQ = scale * sum_j dS_ij K_j with dS = P * (dO.V - Delta), P = exp(S - LSE).
// Same decomposition as the forward.
// ---------------------------------------------------------------------------
template <int DP, int NW>
__global__ __launch_bounds__(NW * 64) void attn_bwd_dq_kernel(AttnArgs p) {
    constexpr int LD = DP + 4;
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    __shared__ __attribute__((aligned(16))) float Ks[32 * LD];
    __shared__ __attribute__((aligned(16))) float Vs[32 * LD];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int l32 = lane % 32, half = lane / 32;
    const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
    const int kvh = h / (p.H / p.Hkv);
    const int q_wg0 = blockIdx.x * (32 * NW);
    const int q0 = q_wg0 + wave * 32;
    const int qi = q0 + l32;
    const bool q_ok = qi < p.Sq;
    const long qoff = (((long)b * p.Sq + (q_ok ? qi : 0)) * p.H + h) * p.D;
    const long srow = ((long)b * p.H + h) * p.Sq + (q_ok ? qi : 0);

    float4 qreg[NS], doreg[NS];
    float delta = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int d = 8 * s + 4 * half;
        const float4 t = load_row4(p.q + qoff, d, p.D, q_ok);
        qreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
        doreg[s] = load_row4(p.d_out + qoff, d, p.D, q_ok);
        const float4 ov = load_row4(p.out + qoff, d, p.D, q_ok);
        delta += doreg[s].x * ov.x + doreg[s].y * ov.y + doreg[s].z * ov.z + doreg[s].w * ov.w;
    }
    delta += __shfl_xor(delta, 32, 64);
    const float lse = q_ok ? p.stats[2 * srow + 1] : kLseEmpty;
    if (q_ok && half == 0) p.stats[2 * srow] = delta;

    floatx16 acc[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) acc[f] = zero16();

    int q_last_wg = q_wg0 + 32 * NW - 1;
    if (q_last_wg > p.Sq - 1) q_last_wg = p.Sq - 1;
    int k_end = p.Sk;
    if (p.causal && q_last_wg + p.causal_offset + 1 < k_end) k_end = q_last_wg + p.causal_offset + 1;
    const int q_last_wave = q0 + 31 + p.causal_offset;
    const int q_pos = qi + p.causal_offset;

    for (int kb = 0; kb < k_end; kb += 32) {
        __syncthreads();
        stage_tile<DP, NW * 64>(Ks, p.k, b, p.Sk, p.Hkv, kvh, p.D, kb, tid);
        stage_tile<DP, NW * 64>(Vs, p.v, b, p.Sk, p.Hkv, kvh, p.D, kb, tid);
        __syncthreads();
        if (q0 >= p.Sq || (p.causal && kb > q_last_wave)) continue;

        floatx16 s = zero16(), dp = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            const float4 a = *reinterpret_cast<const float4*>(Ks + l32 * LD + 8 * st + 4 * half);
            s = MFMA(a.x, qreg[st].x, s);
            s = MFMA(a.y, qreg[st].y, s);
            s = MFMA(a.z, qreg[st].z, s);
            s = MFMA(a.w, qreg[st].w, s);
            const float4 c = *reinterpret_cast<const float4*>(Vs + l32 * LD + 8 * st + 4 * half);
            dp = MFMA(c.x, doreg[st].x, dp);
            dp = MFMA(c.y, doreg[st].y, dp);
            dp = MFMA(c.z, doreg[st].z, dp);
            dp = MFMA(c.w, doreg[st].w, dp);
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int key = kb + row_of(t, half);
            const bool vis = q_ok && key < p.Sk && (!p.causal || key <= q_pos);
            const float pij = vis ? __expf(s[t] - lse) : 0.0f;
            s[t] = pij * (dp[t] - delta);
        }
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const float a = Ks[row_of(t, half) * LD + f * 32 + l32];
                acc[f] = MFMA(a, s[t], acc[f]);
            }
    }

    if (!q_ok) return;
    float* drow = p.dq + qoff;
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
            const int d = f * 32 + r4 * 8 + half * 4;
            if (d + 4 <= p.D && ((((uintptr_t)(drow + d)) & 15) == 0)) {
                *reinterpret_cast<float4*>(drow + d) =
                    make_float4(acc[f][r4 * 4 + 0] * p.scale, acc[f][r4 * 4 + 1] * p.scale,
                                acc[f][r4 * 4 + 2] * p.scale, acc[f][r4 * 4 + 3] * p.scale);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (d + e < p.D) drow[d + e] = acc[f][r4 * 4 + e] * p.scale;
            }
        }
}

// ---------------------------------------------------------------------------
// Backward, pass 2: dK and dV of 32 keys of one (batch, kv head), summed over
// the query heads of the group and over the query blocks that can see them.
// The (head, query block) items are dealt round-robin to the 4 waves, each with
// its own Q / dO staging area; the 4 partial results are added in wave order
// through LDS (no atomics: the result is deterministic).
// Grid (ceil(Sk/32), B*Hkv), 256 threads.
// ---------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_kernel(AttnArgs p) {
    constexpr int LD = DP + 4;
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    constexpr int REGION = 2 * 32 * LD;  // floats per wave: Q tile + dO tile
    static_assert(2 * DP * 33 <= REGION, "reduction buffer must fit the staging area");
    extern __shared__ __attribute__((aligned(16))) float smem[];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int l32 = lane % 32, half = lane / 32;
    const int b = blockIdx.y / p.Hkv, kvh = blockIdx.y % p.Hkv;
    const int G = p.H / p.Hkv;
    const int kb0 = blockIdx.x * 32;
    const int key = kb0 + l32;
    const bool k_ok = key < p.Sk;
    const long koff = (((long)b * p.Sk + (k_ok ? key : 0)) * p.Hkv + kvh) * p.D;
    float* Qs = smem + wave * REGION;
    float* dOs = Qs + 32 * LD;

    float4 kreg[NS], vreg[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int d = 8 * s + 4 * half;
        const float4 t = load_row4(p.k + koff, d, p.D, k_ok);
        kreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
        vreg[s] = load_row4(p.v + koff, d, p.D, k_ok);
    }
    floatx16 dk[NF], dv[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) {
        dk[f] = zero16();
        dv[f] = zero16();
    }

    // Query blocks that can see key block kb0.
    const int nqb = (p.Sq + 31) / 32;
    int qb_start = 0;
    if (p.causal) {
        const int first_q = kb0 - p.causal_offset;  // smallest i with i + offset >= kb0
        qb_start = first_q > 0 ? first_q / 32 : 0;
    }
    const int per_head = nqb > qb_start ? nqb - qb_start : 0;
    const int items = per_head * G;
    const int rounds = (items + 3) / 4;

    for (int it = 0; it < rounds; it++) {
        const int item = it * 4 + wave;
        const bool active = item < items;  // wave-uniform
        const int g = active ? item / per_head : 0;
        const int qb = active ? qb_start + item % per_head : 0;
        const int h = kvh * G + g;
        const int q0 = qb * 32;
        __syncthreads();
        if (active) {
            stage_tile<DP, 64>(Qs, p.q, b, p.Sq, p.H, h, p.D, q0, lane);
            stage_tile<DP, 64>(dOs, p.d_out, b, p.Sq, p.H, h, p.D, q0, lane);
        }
        __syncthreads();
        if (!active) continue;

        float lse[16], dlt[16];
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int qi = q0 + row_of(t, half);
            if (qi < p.Sq) {
                const float2 st = *reinterpret_cast<const float2*>(p.stats + 2 * (((long)b * p.H + h) * p.Sq + qi));
                dlt[t] = st.x;
                lse[t] = st.y;
            } else {
                dlt[t] = 0.0f;
                lse[t] = kLseEmpty;
            }
        }
        floatx16 s = zero16(), dp = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            const float4 a = *reinterpret_cast<const float4*>(Qs + l32 * LD + 8 * st + 4 * half);
            s = MFMA(a.x, kreg[st].x, s);
            s = MFMA(a.y, kreg[st].y, s);
            s = MFMA(a.z, kreg[st].z, s);
            s = MFMA(a.w, kreg[st].w, s);
            const float4 c = *reinterpret_cast<const float4*>(dOs + l32 * LD + 8 * st + 4 * half);
            dp = MFMA(c.x, vreg[st].x, dp);
            dp = MFMA(c.y, vreg[st].y, dp);
            dp = MFMA(c.z, vreg[st].z, dp);
            dp = MFMA(c.w, vreg[st].w, dp);
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int qi = q0 + row_of(t, half);
            const bool vis = k_ok && qi < p.Sq && (!p.causal || key <= qi + p.causal_offset);
            const float pij = vis ? __expf(s[t] - lse[t]) : 0.0f;
            s[t] = pij;                       // P
            dp[t] = pij * (dp[t] - dlt[t]);   // dS
        }
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const int r = row_of(t, half);
                dv[f] = MFMA(dOs[r * LD + f * 32 + l32], s[t], dv[f]);
                dk[f] = MFMA(Qs[r * LD + f * 32 + l32], dp[t], dk[f]);
            }
    }

    // Cross-wave sum. red[wave][which][d][33]
    __syncthreads();
    float* red = smem + wave * REGION;
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int d = f * 32 + row_of(t, half);
            red[d * 33 + l32] = dk[f][t];
            red[DP * 33 + d * 33 + l32] = dv[f][t];
        }
    __syncthreads();
    for (int e = tid; e < 32 * DP; e += 256) {
        const int kk = e / DP, d = e % DP;
        const int krow = kb0 + kk;
        if (krow < p.Sk && d < p.D) {
            float sk = 0.0f, sv = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                sk += smem[w * REGION + d * 33 + kk];
                sv += smem[w * REGION + DP * 33 + d * 33 + kk];
            }
            const long o = (((long)b * p.Sk + krow) * p.Hkv + kvh) * p.D + d;
            p.dk[o] = sk * p.scale;  // dK = scale * sum dS Q (Q is staged unscaled)
            p.dv[o] = sv;
        }
    }
}

template <int DP>
int launch_fwd(ft_context* ctx, const AttnArgs& a) {
    constexpr int NW = 2;
    const dim3 grid(ft_div_up(a.Sq, 32 * NW), (unsigned)(a.B * a.H));
    // flop convention of the reference's benchmarks: causal forward 2*B*H*Sq*Sk*D, full 4*...
    const double fl = (a.causal ? 2.0 : 4.0) * a.B * a.H * (double)a.Sq * a.Sk * a.D;
    const double by = 4.0 * a.B * ((double)a.Sq * a.H * a.D * 2 + (double)a.Sk * a.Hkv * a.D * 2);
    ft_prof_scope prof(ctx, "attn_fwd_kernel", fl, by);
    hipLaunchKernelGGL((attn_fwd_kernel<DP, NW>), grid, dim3(NW * 64), 0, ctx->stream, a);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

template <int DP>
int launch_bwd(ft_context* ctx, const AttnArgs& a) {
    constexpr int NW = 2;
    const dim3 grid(ft_div_up(a.Sq, 32 * NW), (unsigned)(a.B * a.H));
    // backward = 2.5x forward by the reference's convention: 1.5x (3 products) in dQ, 2x (4 products)
    // in dK/dV, minus the shared recomputation -> charged 1.0x and 1.5x.
    const double fl = (a.causal ? 2.0 : 4.0) * a.B * a.H * (double)a.Sq * a.Sk * a.D;
    const double by = 4.0 * a.B * ((double)a.Sq * a.H * a.D * 4 + (double)a.Sk * a.Hkv * a.D * 4);
    {
        ft_prof_scope prof(ctx, "attn_bwd_dq_kernel", 1.0 * fl, by * 0.5);
        hipLaunchKernelGGL((attn_bwd_dq_kernel<DP, NW>), grid, dim3(NW * 64), 0, ctx->stream, a);
    }
    FT_LAUNCH_CHECK();
    constexpr size_t smem = (size_t)4 * 2 * 32 * (DP + 4) * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        FT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dkdv_kernel<DP>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const dim3 grid2(ft_div_up(a.Sk, 32), (unsigned)(a.B * a.Hkv));
    {
        ft_prof_scope prof(ctx, "attn_bwd_dkdv_kernel", 1.5 * fl, by * 0.5);
        hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DP>), grid2, dim3(256), smem, ctx->stream, a);
    }
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int check_common(const char* who, ft_context* ctx, size_t B, size_t Sq, size_t Sk, size_t H, size_t Hkv, size_t D,
                 const ft_attention_options* opts) {
    FT_CHECK_ARG(ctx && opts, "%s: NULL argument", who);
    FT_CHECK_ARG(D >= 1 && D <= 128, "%s: flash attention supports head_dim <= 128, got %zu", who, D);
    FT_CHECK_ARG(Hkv > 0 && H % Hkv == 0, "%s: num_heads (%zu) must be a multiple of num_kv_heads (%zu)", who, H, Hkv);
    FT_CHECK_ARG(opts->window == 0, "%s: sliding windows are not supported", who);
    FT_CHECK_ARG(opts->dropout_prob == 0.0f, "%s: attention dropout is not supported", who);
    FT_CHECK_ARG(B * H < 65536 && B * Hkv < 65536, "%s: batch*heads too large for the launch grid", who);
    FT_CHECK_ARG(Sq < (1u << 24) && Sk < (1u << 24), "%s: sequence too long", who);
    return FT_OK;
}

AttnArgs make_args(size_t B, size_t Sq, size_t Sk, size_t H, size_t Hkv, size_t D, const ft_attention_options* o) {
    AttnArgs a{};
    a.B = (int)B; a.Sq = (int)Sq; a.Sk = (int)Sk; a.H = (int)H; a.Hkv = (int)Hkv; a.D = (int)D;
    a.causal = o->causal ? 1 : 0;
    a.causal_offset = (int)o->causal_offset;
    a.scale = 1.0f / sqrtf((float)D);
    return a;
}

}  // namespace

extern "C" {

int ft_flash_attention_v2_with_stats(ft_context* ctx, const float* q, const float* k, const float* v, float* out,
                                     float* stats, size_t B, size_t Sq, size_t Sk, size_t H, size_t Hkv, size_t D,
                                     const ft_attention_options* opts) {
    FT_TRY(check_common("ft_flash_attention_v2_with_stats", ctx, B, Sq, Sk, H, Hkv, D, opts));
    FT_CHECK_ARG(q && k && v && out, "ft_flash_attention_v2_with_stats: NULL tensor");
    if (B == 0 || Sq == 0 || H == 0) return FT_OK;
    AttnArgs a = make_args(B, Sq, Sk, H, Hkv, D, opts);
    a.q = q; a.k = k; a.v = v; a.o = out; a.stats = stats;
    if (D <= 32) return launch_fwd<32>(ctx, a);
    if (D <= 64) return launch_fwd<64>(ctx, a);
    return launch_fwd<128>(ctx, a);
}

int ft_flash_attention_v2_backward_with_stats(ft_context* ctx, const float* q, const float* k, const float* v,
                                              const float* out, const float* d_out, float* dq, float* dk, float* dv,
                                              float* stats, size_t B, size_t Sq, size_t Sk, size_t H, size_t Hkv,
                                              size_t D, const ft_attention_options* opts) {
    FT_TRY(check_common("ft_flash_attention_v2_backward_with_stats", ctx, B, Sq, Sk, H, Hkv, D, opts));
    FT_CHECK_ARG(q && k && v && out && d_out && dq && dk && dv && stats,
                 "ft_flash_attention_v2_backward_with_stats: NULL tensor");
    if (B == 0 || H == 0) return FT_OK;
    AttnArgs a = make_args(B, Sq, Sk, H, Hkv, D, opts);
    a.q = q; a.k = k; a.v = v; a.out = out; a.d_out = d_out; a.dq = dq; a.dk = dk; a.dv = dv; a.stats = stats;
    if (D <= 32) return launch_bwd<32>(ctx, a);
    if (D <= 64) return launch_bwd<64>(ctx, a);
    return launch_bwd<128>(ctx, a);
}

}  // extern "C"
