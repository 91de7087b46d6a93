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
#include "ft_attention.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr float kMasked = kAttnMasked;
constexpr float kLseEmpty = kAttnLseEmpty;

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

// Operand fetches straight from global memory into MFMA operand registers. The
// tiles are small (32 rows x head_dim), every wave needs its own, and they are
// L2 resident, so there is no LDS staging and no workgroup barrier in the key
// loop: a wave runs free, with the next tile's loads in flight while it
// multiplies the current one.
//   quad: 4 consecutive head-dim values of one row (A operand "row x k" with k
//         along the head dim: lanes 0-31 take quads 8s.., lanes 32-63 8s+4..)
//   one:  a single value (A operand with the head dim as the ROW: lane = d)
template <bool FULL>
__device__ __forceinline__ float4 ld_quad(const float* row, int d, int D) {
    if constexpr (FULL) return *reinterpret_cast<const float4*>(row + d);
    return load_row4(row, d, D, true);
}
template <bool FULL>
__device__ __forceinline__ float ld_one(const float* row, int d, int D) {
    if constexpr (FULL) return row[d];
    return d < D ? row[d] : 0.0f;
}

// Work distribution. Under the causal mask a block's cost grows (or shrinks)
// with its index. The items of a launch are ordered block-major, most expensive
// block index first, over a 1-D grid: the long items start first (the tail of
// the launch is made of short ones), and because consecutive workgroups go
// round-robin to the 8 XCDs, every XCD receives the same mix of block indices
// (a (block, batch*head) grid with 8 blocks would hand XCD c all the blocks
// of index c). `j` counts the block indices in dispatch order.
__device__ __forceinline__ bool attn_work_item(int nblk, int nbh, int& j, int& bh) {
    const int t = (int)blockIdx.x;
    if (t >= nblk * nbh) return false;
    j = t / nbh;
    bh = t % nbh;
    return true;
}
inline unsigned attn_grid(size_t nblk, size_t nbh) { return (unsigned)(nblk * nbh); }

// ---------------------------------------------------------------------------
// Forward. A workgroup owns 32 queries of one (batch, head); its NSPL waves take
// every NSPL-th block of 32 keys and merge their partial softmax states through
// LDS at the end (shorter critical path under the causal mask, and two waves
// per SIMD to overlap one wave's softmax arithmetic with the other's MFMAs).
// One workgroup per (query block, batch*head) item (attn_work_item); within a
// head the last query block, which has the longest key loop, starts first.
// ---------------------------------------------------------------------------
constexpr int kKeySplit = 4;    // forward
constexpr int kKeySplitDq = 2;  // dQ: two waves per SIMD need <= 256 registers per lane

template <int DP, bool FULL>
__global__ __launch_bounds__(kKeySplit * 64) void attn_fwd_kernel(AttnArgs p) {
    constexpr int NF = DP / 32;  // 32-row blocks of the head dim
    constexpr int NS = DP / 8;   // k-steps of 8 over the head dim
    constexpr int NSPL = kKeySplit;
    __shared__ float merge[(NSPL - 1) * 64 * (NF * 16 + 2)];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, l32 = lane % 32, half = lane / 32;
    int blk_j, bh_i;
    const int nqb_grid = (p.Sq + 31) / 32;
    if (!attn_work_item(nqb_grid, p.B * p.H, blk_j, bh_i)) return;
    const int b = bh_i / p.H, h = bh_i % p.H;
    const int kvh = h / (p.H / p.Hkv);
    const int q0 = (nqb_grid - 1 - blk_j) * 32;  // the last query block has the longest key loop: first
    const int qi = q0 + l32;
    const bool q_ok = qi < p.Sq;
    const int qc = q_ok ? qi : p.Sq - 1;
    const float* qrow = p.q + (((long)b * p.Sq + qc) * p.H + h) * p.D;
    const long kst = (long)p.Hkv * p.D;
    const float* kbase = p.k + ((long)b * p.Sk * p.Hkv + kvh) * p.D;
    const float* vbase = p.v + ((long)b * p.Sk * p.Hkv + kvh) * p.D;

    float4 qreg[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const float4 t = ld_quad<FULL>(qrow, 8 * s + 4 * half, p.D);
        qreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
    }
    floatx16 o[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) o[f] = zero16();
    float m_run = kMasked, l_run = 0.0f;

    int k_end = p.Sk;
    if (p.causal && q0 + 31 + p.causal_offset + 1 < k_end) k_end = q0 + 31 + p.causal_offset + 1;
    const int q_pos = qi + p.causal_offset;

    float4 kc[NS], kn[NS];
    float vc[NF][16], vn[NF][16];
    auto load_block = [&](int kb, float4 (&kk)[NS], float (&vv)[NF][16]) {
        int key = kb + l32;
        key = key < p.Sk ? key : p.Sk - 1;
        const float* krow = kbase + key * kst;
#pragma unroll
        for (int s = 0; s < NS; s++) kk[s] = ld_quad<FULL>(krow, 8 * s + 4 * half, p.D);
#pragma unroll
        for (int t = 0; t < 16; t++) {
            int kt = kb + row_of(t, half);
            kt = kt < p.Sk ? kt : p.Sk - 1;
            const float* vrow = vbase + kt * kst;
#pragma unroll
            for (int f = 0; f < NF; f++) vv[f][t] = ld_one<FULL>(vrow, f * 32 + l32, p.D);
        }
    };
    const int kb_first = wave * 32;
    if (kb_first < k_end) load_block(kb_first, kc, vc);
    for (int kb = kb_first; kb < k_end; kb += 32 * NSPL) {
        const bool more = kb + 32 * NSPL < k_end;
        if (more) load_block(kb + 32 * NSPL, kn, vn);

        floatx16 s = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            s = MFMA(kc[st].x, qreg[st].x, s);
            s = MFMA(kc[st].y, qreg[st].y, s);
            s = MFMA(kc[st].z, qreg[st].z, s);
            s = MFMA(kc[st].w, qreg[st].w, s);
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
            for (int t = 0; t < 16; t++) o[f] = MFMA(vc[f][t], s[t], o[f]);
        }
        if (more) {
#pragma unroll
            for (int st = 0; st < NS; st++) kc[st] = kn[st];
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int t = 0; t < 16; t++) vc[f][t] = vn[f][t];
        }
    }

    // Merge the waves' (m, l, O) into wave 0, in wave order.
    if constexpr (NSPL > 1) {
        constexpr int W = NF * 16 + 2;
        if (wave > 0) {
            float* dst = merge + ((wave - 1) * 64 + lane) * W;
            dst[0] = m_run;
            dst[1] = l_run;
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int r = 0; r < 16; r++) dst[2 + f * 16 + r] = o[f][r];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 1; w < NSPL; w++) {
            const float* src = merge + ((w - 1) * 64 + lane) * W;
            const float m_o = src[0], l_o = src[1];
            const float m_new = fmaxf(m_run, m_o);
            const float c0 = __expf(m_run - m_new), c1 = __expf(m_o - m_new);
            l_run = l_run * c0 + l_o * c1;
            m_run = m_new;
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[f][r] = o[f][r] * c0 + src[2 + f * 16 + r] * c1;
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
template <int DP, bool FULL>
__global__ __launch_bounds__(kKeySplitDq * 64) void attn_bwd_dq_kernel(AttnArgs p) {
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    constexpr int NSPL = kKeySplitDq;
    __shared__ float merge[(NSPL - 1) * 64 * NF * 16];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, l32 = lane % 32, half = lane / 32;
    int blk_j, bh_i;
    const int nqb_grid = (p.Sq + 31) / 32;
    if (!attn_work_item(nqb_grid, p.B * p.H, blk_j, bh_i)) return;
    const int b = bh_i / p.H, h = bh_i % p.H;
    const int kvh = h / (p.H / p.Hkv);
    const int q0 = (nqb_grid - 1 - blk_j) * 32;  // the last query block has the longest key loop: first
    const int qi = q0 + l32;
    const bool q_ok = qi < p.Sq;
    const int qc = q_ok ? qi : p.Sq - 1;
    const long qoff = (((long)b * p.Sq + qc) * p.H + h) * p.D;
    const long srow = ((long)b * p.H + h) * p.Sq + qc;
    const long kst = (long)p.Hkv * p.D;
    const float* kbase = p.k + ((long)b * p.Sk * p.Hkv + kvh) * p.D;
    const float* vbase = p.v + ((long)b * p.Sk * p.Hkv + kvh) * p.D;

    float4 qreg[NS], doreg[NS];
    float delta = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int d = 8 * s + 4 * half;
        const float4 t = ld_quad<FULL>(p.q + qoff, d, p.D);
        qreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
        doreg[s] = ld_quad<FULL>(p.d_out + qoff, d, p.D);
        const float4 ov = ld_quad<FULL>(p.out + qoff, d, p.D);
        delta += doreg[s].x * ov.x + doreg[s].y * ov.y + doreg[s].z * ov.z + doreg[s].w * ov.w;
    }
    delta += __shfl_xor(delta, 32, 64);
    const float lse = q_ok ? p.stats[2 * srow + 1] : kLseEmpty;
    if (q_ok && half == 0 && wave == 0) p.stats[2 * srow] = delta;

    floatx16 acc[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) acc[f] = zero16();

    int k_end = p.Sk;
    if (p.causal && q0 + 31 + p.causal_offset + 1 < k_end) k_end = q0 + 31 + p.causal_offset + 1;
    const int q_pos = qi + p.causal_offset;

    float4 kc[NS], vc[NS], kn[NS], vn[NS];
    auto load_quads = [&](int kb, float4 (&kk)[NS], float4 (&vv)[NS]) {
        int key = kb + l32;
        key = key < p.Sk ? key : p.Sk - 1;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            kk[s] = ld_quad<FULL>(kbase + key * kst, 8 * s + 4 * half, p.D);
            vv[s] = ld_quad<FULL>(vbase + key * kst, 8 * s + 4 * half, p.D);
        }
    };
    const int kb_first = wave * 32;
    if (kb_first < k_end) load_quads(kb_first, kc, vc);
    for (int kb = kb_first; kb < k_end; kb += 32 * NSPL) {
        const bool more = kb + 32 * NSPL < k_end;
        // K^T operand of dQ += K^T dS^T for this block: issued now, used last.
        float k1[NF][16];
#pragma unroll
        for (int t = 0; t < 16; t++) {
            int kt = kb + row_of(t, half);
            kt = kt < p.Sk ? kt : p.Sk - 1;
#pragma unroll
            for (int f = 0; f < NF; f++) k1[f][t] = ld_one<FULL>(kbase + kt * kst, f * 32 + l32, p.D);
        }
        if (more) load_quads(kb + 32 * NSPL, kn, vn);

        floatx16 s = zero16(), dp = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            s = MFMA(kc[st].x, qreg[st].x, s);
            s = MFMA(kc[st].y, qreg[st].y, s);
            s = MFMA(kc[st].z, qreg[st].z, s);
            s = MFMA(kc[st].w, qreg[st].w, s);
            dp = MFMA(vc[st].x, doreg[st].x, dp);
            dp = MFMA(vc[st].y, doreg[st].y, dp);
            dp = MFMA(vc[st].z, doreg[st].z, dp);
            dp = MFMA(vc[st].w, doreg[st].w, dp);
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
            for (int t = 0; t < 16; t++) acc[f] = MFMA(k1[f][t], s[t], acc[f]);
        if (more) {
#pragma unroll
            for (int st = 0; st < NS; st++) {
                kc[st] = kn[st];
                vc[st] = vn[st];
            }
        }
    }

    // Sum of the waves' partial dQ, in wave order.
    if constexpr (NSPL > 1) {
        constexpr int W = NF * 16;
        if (wave > 0) {
            float* dst = merge + ((wave - 1) * 64 + lane) * W;
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int r = 0; r < 16; r++) dst[f * 16 + r] = acc[f][r];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 1; w < NSPL; w++) {
            const float* src = merge + ((w - 1) * 64 + lane) * W;
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[f][r] += src[f * 16 + r];
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
// The (head, query block) items are dealt round-robin to the NWV waves of the
// workgroup; the partial results are added in wave order through LDS (no
// atomics: the result is deterministic). One workgroup per (key block, batch*kv
// head) item, key block 0 first (under the causal mask it has the most items).
// ---------------------------------------------------------------------------
// 8 waves for head dims up to 64; 4 for 128 (the reduction buffer must fit LDS).
constexpr int dkdv_waves(int dp) { return dp <= 64 ? 8 : 4; }

template <int DP, bool FULL>
__global__ __launch_bounds__(dkdv_waves(DP) * 64) void attn_bwd_dkdv_kernel(AttnArgs p) {
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    constexpr int NWV = dkdv_waves(DP);
    constexpr int REGION = 2 * DP * 33;  // floats per wave: dK^T and dV^T, [d][33]
    extern __shared__ __attribute__((aligned(16))) float smem[];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int l32 = lane % 32, half = lane / 32;
    int blk_j, bh_i;
    if (!attn_work_item((p.Sk + 31) / 32, p.B * p.Hkv, blk_j, bh_i)) return;
    const int b = bh_i / p.Hkv, kvh = bh_i % p.Hkv;
    const int G = p.H / p.Hkv;
    const int kb0 = blk_j * 32;  // key block 0 has the most items under the causal mask: first
    const int key = kb0 + l32;
    const bool k_ok = key < p.Sk;
    const long koff = (((long)b * p.Sk + (k_ok ? key : p.Sk - 1)) * p.Hkv + kvh) * p.D;
    const long qst = (long)p.H * p.D;

    float4 kreg[NS], vreg[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int d = 8 * s + 4 * half;
        const float4 t = ld_quad<FULL>(p.k + koff, d, p.D);
        kreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
        vreg[s] = ld_quad<FULL>(p.v + koff, d, p.D);
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

    for (int item = wave; item < items; item += NWV) {
        const int g = item / per_head;
        const int q0 = (qb_start + item % per_head) * 32;
        const int h = kvh * G + g;
        const float* qbase = p.q + ((long)b * p.Sq * p.H + h) * p.D;
        const float* dobase = p.d_out + ((long)b * p.Sq * p.H + h) * p.D;
        int qr = q0 + l32;
        qr = qr < p.Sq ? qr : p.Sq - 1;

        floatx16 s = zero16(), dp = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            const float4 a = ld_quad<FULL>(qbase + qr * qst, 8 * st + 4 * half, p.D);
            const float4 c = ld_quad<FULL>(dobase + qr * qst, 8 * st + 4 * half, p.D);
            s = MFMA(a.x, kreg[st].x, s);
            s = MFMA(a.y, kreg[st].y, s);
            s = MFMA(a.z, kreg[st].z, s);
            s = MFMA(a.w, kreg[st].w, s);
            dp = MFMA(c.x, vreg[st].x, dp);
            dp = MFMA(c.y, vreg[st].y, dp);
            dp = MFMA(c.z, vreg[st].z, dp);
            dp = MFMA(c.w, vreg[st].w, dp);
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int qi = q0 + row_of(t, half);
            float lse = kLseEmpty, dlt = 0.0f;
            if (qi < p.Sq) {
                const float2 st2 = *reinterpret_cast<const float2*>(p.stats + 2 * (((long)b * p.H + h) * p.Sq + qi));
                dlt = st2.x;
                lse = st2.y;
            }
            const bool vis = k_ok && qi < p.Sq && (!p.causal || key <= qi + p.causal_offset);
            const float pij = vis ? __expf(s[t] - lse) : 0.0f;
            s[t] = pij;                   // P
            dp[t] = pij * (dp[t] - dlt);  // dS
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            int qt = q0 + row_of(t, half);
            qt = qt < p.Sq ? qt : p.Sq - 1;
#pragma unroll
            for (int f = 0; f < NF; f++) {
                dv[f] = MFMA(ld_one<FULL>(dobase + qt * qst, f * 32 + l32, p.D), s[t], dv[f]);
                dk[f] = MFMA(ld_one<FULL>(qbase + qt * qst, f * 32 + l32, p.D), dp[t], dk[f]);
            }
        }
    }

    // Cross-wave sum: red[wave][which][d][33]
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
    for (int e = tid; e < 32 * DP; e += NWV * 64) {
        const int kk = e / DP, d = e % DP;
        const int krow = kb0 + kk;
        if (krow < p.Sk && d < p.D) {
            float sk = 0.0f, sv = 0.0f;
#pragma unroll
            for (int w = 0; w < NWV; w++) {
                sk += smem[w * REGION + d * 33 + kk];
                sv += smem[w * REGION + DP * 33 + d * 33 + kk];
            }
            const long o = (((long)b * p.Sk + krow) * p.Hkv + kvh) * p.D + d;
            p.dk[o] = sk * p.scale;  // dK = scale * sum dS Q (Q is read unscaled)
            p.dv[o] = sv;
        }
    }
}

// ---------------------------------------------------------------------------
// dK/dV for whole, aligned head dims (D == DP): the same decomposition, with the
// operand traffic arranged for latency. Every tile is read from global memory
// once, as coalesced 16-byte quads: the key block's K and V go to a tile in LDS
// that all waves share; an item's Q and dO quads go to registers (they are the
// A operands of S and dP), and from there into a wave-private LDS tile from
// which the same data is read back transposed (lane = head-dim index) as the A
// operands of dV^T and dK^T. The next item's quads are fetched into the same
// registers while the current item's second half multiplies, so a wave sees one
// global latency per launch, not two per item.
// LDS rows are 16-byte-chunk swizzled (chunk c of row r sits at c ^ (r & 15)):
// quad reads/writes of 16 consecutive rows and transposed reads of 32
// consecutive columns are both conflict-free.
// One workgroup per (key block, batch*kv head) item, key block 0 (the most
// items under the causal mask) first within a head.
// ---------------------------------------------------------------------------
template <int DP>
__device__ __forceinline__ int sw_off(int row, int chunk) {
    constexpr int CH = DP / 4;
    return row * DP + ((chunk ^ (row & (CH < 16 ? CH - 1 : 15))) * 4);
}

template <int DP>
__global__ __launch_bounds__(512) void attn_bwd_dkdv_lds_kernel(AttnArgs p) {
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    constexpr int NWV = 8;
    constexpr int TILE = 32 * DP;
    constexpr int REGION = 2 * DP * 33;                                  // reduction layout: dK^T, dV^T as [d][33]
    constexpr int PRIV = (2 * TILE + 64) > REGION ? (2 * TILE + 64) : REGION;  // Q tile, dO tile, 32 (Delta, LSE)
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* ks = smem;            // K * scale
    float* vs = smem + TILE;
    float* priv = smem + 2 * TILE + (threadIdx.x / 64) * PRIV;
    float* qs = priv;
    float* dos = priv + TILE;
    float* sts = priv + 2 * TILE;

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int l32 = lane % 32, half = lane / 32;
    int blk_j, bh_i;
    if (!attn_work_item((p.Sk + 31) / 32, p.B * (p.split_g ? p.H : p.Hkv), blk_j, bh_i)) return;
    const int Gfull = p.H / p.Hkv;
    const int b = bh_i / (p.split_g ? p.H : p.Hkv);
    const int hsel = bh_i % (p.split_g ? p.H : p.Hkv);
    const int kvh = p.split_g ? hsel / Gfull : hsel;
    const int g0 = p.split_g ? hsel % Gfull : 0;   // first query head of this workgroup within the group
    const int G = p.split_g ? 1 : Gfull;           // and how many it covers
    const int kb0 = blk_j * 32;  // key block 0 has the most items under the causal mask: first
    const int key = kb0 + l32;
    const bool k_ok = key < p.Sk;
    const long qst = (long)p.H * DP;

    // K and V of the key block -> shared LDS tile (rows past Sk are clamped: masked below).
    for (int e = tid; e < 32 * (DP / 4); e += NWV * 64) {
        const int r = e / (DP / 4), c = e % (DP / 4);
        int kr = kb0 + r;
        kr = kr < p.Sk ? kr : p.Sk - 1;
        const long o = (((long)b * p.Sk + kr) * p.Hkv + kvh) * DP + 4 * c;
        const float4 kq = *reinterpret_cast<const float4*>(p.k + o);
        *reinterpret_cast<float4*>(ks + sw_off<DP>(r, c)) =
            make_float4(kq.x * p.scale, kq.y * p.scale, kq.z * p.scale, kq.w * p.scale);
        *reinterpret_cast<float4*>(vs + sw_off<DP>(r, c)) = *reinterpret_cast<const float4*>(p.v + o);
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

    float4 qa[NS], qc[NS];
    float2 st_mine = make_float2(0.0f, kLseEmpty);
    auto fetch = [&](int item) {
        const int g = item / per_head;
        const int q0 = (qb_start + item % per_head) * 32;
        const int h = kvh * Gfull + g0 + g;
        int qr = q0 + l32;
        const bool ok = qr < p.Sq;
        qr = ok ? qr : p.Sq - 1;
        const float* qrow = p.q + ((long)b * p.Sq * p.H + h) * DP + qr * qst;
        const float* dorow = p.d_out + ((long)b * p.Sq * p.H + h) * DP + qr * qst;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            qa[s] = *reinterpret_cast<const float4*>(qrow + 8 * s + 4 * half);
            qc[s] = *reinterpret_cast<const float4*>(dorow + 8 * s + 4 * half);
        }
        const float2 t = *reinterpret_cast<const float2*>(p.stats + 2 * (((long)b * p.H + h) * p.Sq + qr));
        st_mine = ok ? t : make_float2(0.0f, kLseEmpty);
    };
    if (wave < items) fetch(wave);
    __syncthreads();  // K/V tile complete

    for (int item = wave; item < items; item += NWV) {
        const int q0 = (qb_start + item % per_head) * 32;
        // LDS addresses are formed from this per item (not kept in registers across the loop)
        int lq = l32;
        asm volatile("" : "+v"(lq));
        // this item's tiles -> private LDS (for the transposed reads), S and dP from the registers
#pragma unroll
        for (int s = 0; s < NS; s++) {
            *reinterpret_cast<float4*>(qs + sw_off<DP>(lq, 2 * s + half)) = qa[s];
            *reinterpret_cast<float4*>(dos + sw_off<DP>(lq, 2 * s + half)) = qc[s];
        }
        if (half == 0) *reinterpret_cast<float2*>(sts + 2 * lq) = st_mine;
        floatx16 s = zero16(), dp = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            const float4 kq = *reinterpret_cast<const float4*>(ks + sw_off<DP>(lq, 2 * st + half));
            const float4 vq = *reinterpret_cast<const float4*>(vs + sw_off<DP>(lq, 2 * st + half));
            s = MFMA(qa[st].x, kq.x, s);
            s = MFMA(qa[st].y, kq.y, s);
            s = MFMA(qa[st].z, kq.z, s);
            s = MFMA(qa[st].w, kq.w, s);
            dp = MFMA(qc[st].x, vq.x, dp);
            dp = MFMA(qc[st].y, vq.y, dp);
            dp = MFMA(qc[st].z, vq.z, dp);
            dp = MFMA(qc[st].w, vq.w, dp);
            if (st % 2 == 1) __builtin_amdgcn_sched_barrier(0);  // bounds how many LDS quads are live
        }
        __builtin_amdgcn_sched_barrier(0);
        // the next item's quads travel while the rest of this item is computed
        if (item + NWV < items) fetch(item + NWV);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int r = row_of(t, half);
            const int qi = q0 + r;
            const float2 st2 = *reinterpret_cast<const float2*>(sts + 2 * r);
            const bool vis = k_ok && qi < p.Sq && (!p.causal || key <= qi + p.causal_offset);
            const float pij = vis ? __expf(s[t] - st2.y) : 0.0f;
            s[t] = pij;                     // P
            dp[t] = pij * (dp[t] - st2.x);  // dS
        }
        // transposed operands in groups of 4 rows: 4 * 2 * NF LDS reads, then their MFMAs
#pragma unroll
        for (int t4 = 0; t4 < 16; t4 += 4) {
            float ao[4][NF], aq[4][NF];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int r = row_of(t4 + u, half);
#pragma unroll
                for (int f = 0; f < NF; f++) {
                    const int d = f * 32 + lq;
                    ao[u][f] = dos[sw_off<DP>(r, d / 4) + (d & 3)];
                    aq[u][f] = qs[sw_off<DP>(r, d / 4) + (d & 3)];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int f = 0; f < NF; f++) {
                    dv[f] = MFMA(ao[u][f], s[t4 + u], dv[f]);
                    dk[f] = MFMA(aq[u][f], dp[t4 + u], dk[f]);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // Cross-wave sum in wave order: red[wave][which][d][33] over the private regions.
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int d = f * 32 + row_of(t, half);
            priv[d * 33 + l32] = dk[f][t];
            priv[DP * 33 + d * 33 + l32] = dv[f][t];
        }
    __syncthreads();
    const float* red = smem + 2 * TILE;
    for (int e = tid; e < 32 * DP; e += NWV * 64) {
        const int kk = e / DP, d = e % DP;
        const int krow = kb0 + kk;
        if (krow < p.Sk) {
            float sk = 0.0f, sv = 0.0f;
#pragma unroll
            for (int w = 0; w < NWV; w++) {
                sk += red[w * PRIV + d * 33 + kk];
                sv += red[w * PRIV + DP * 33 + d * 33 + kk];
            }
            const long o = (((long)b * p.Sk + krow) * p.Hkv + kvh) * DP + d;
            if (p.split_g) {
                const long n_all = (long)p.B * p.Sk * p.Hkv * DP;
                p.part[(2 * g0) * n_all + o] = sk;
                p.part[(2 * g0 + 1) * n_all + o] = sv;
                continue;
            }
            p.dv[o] = sv;
            if (DP == 64 && p.rope) {
                // dK rotated back: this thread also sums the partner element (d +- 32)
                const int dp = d < 32 ? d + 32 : d - 32;
                float sp = 0.0f;
#pragma unroll
                for (int w = 0; w < NWV; w++) sp += red[w * PRIV + dp * 33 + kk];
                const float2 cs = p.rope[(long)krow * 32 + (d & 31)];
                const float x = sk * p.scale, y = sp * p.scale;
                p.dk[o] = d < 32 ? x * cs.x + y * cs.y : x * cs.x - y * cs.y;
            } else {
                p.dk[o] = sk * p.scale;  // dK = scale * sum dS Q (Q is read unscaled)
            }
        }
    }
}

// dk = scale * sum over the group's query heads of part[2g] (rotated back through RoPE when
// asked), dv = sum of part[2g + 1]; heads added in order. One thread per element.
__global__ __launch_bounds__(256) void attn_dkdv_combine_kernel(AttnArgs p, int DP) {
    const long n_all = (long)p.B * p.Sk * p.Hkv * DP;
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_all) return;
    const int G = p.H / p.Hkv;
    float sk = 0.0f, sv = 0.0f;
    for (int g = 0; g < G; g++) {
        sk += p.part[(2 * g) * n_all + i];
        sv += p.part[(2 * g + 1) * n_all + i];
    }
    p.dv[i] = sv;
    if (DP == 64 && p.rope) {
        const int d = (int)(i % DP);
        const long ip = d < 32 ? i + 32 : i - 32;
        float sp = 0.0f;
        for (int g = 0; g < G; g++) sp += p.part[(2 * g) * n_all + ip];
        const int krow = (int)((i / ((long)p.Hkv * DP)) % p.Sk);
        const float2 cs = p.rope[(long)krow * 32 + (d & 31)];
        const float x = sk * p.scale, y = sp * p.scale;
        p.dk[i] = d < 32 ? x * cs.x + y * cs.y : x * cs.x - y * cs.y;
    } else {
        p.dk[i] = sk * p.scale;
    }
}

// ---------------------------------------------------------------------------
// Forward and dQ for whole, aligned head dims (D == DP), same operand scheme as
// the dK/dV kernel above: a key block's K and V are read from global memory once
// as coalesced quads into registers (the next block's while the current one
// multiplies); the operand that is needed with the head dim as the MFMA row
// (V^T in the forward, K^T for dQ) is written to a wave-private swizzled LDS
// tile and read back transposed.
// ---------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(kKeySplit * 64) void attn_fwd_lds_kernel(AttnArgs p) {
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    constexpr int NSPL = kKeySplit;
    constexpr int TILE = 32 * DP;
    constexpr int MERGE = 64 * (NF * 16 + 2);
    constexpr int PRIV = TILE > MERGE ? TILE : MERGE;
    __shared__ __attribute__((aligned(16))) float lds[NSPL * PRIV];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, l32 = lane % 32, half = lane / 32;
    float* vt = lds + wave * PRIV;
    int blk_j, bh_i;
    const int nqb_grid = (p.Sq + 31) / 32;
    if (!attn_work_item(nqb_grid, p.B * p.H, blk_j, bh_i)) return;
    const int b = bh_i / p.H, h = bh_i % p.H;
    const int kvh = h / (p.H / p.Hkv);
    const int q0 = (nqb_grid - 1 - blk_j) * 32;  // the last query block has the longest key loop: first
    const int qi = q0 + l32;
    const bool q_ok = qi < p.Sq;
    const int qc = q_ok ? qi : p.Sq - 1;
    const float* qrow = p.q + (((long)b * p.Sq + qc) * p.H + h) * DP;
    const long kst = (long)p.Hkv * DP;
    const float* kbase = p.k + ((long)b * p.Sk * p.Hkv + kvh) * DP;
    const float* vbase = p.v + ((long)b * p.Sk * p.Hkv + kvh) * DP;

    float4 qreg[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const float4 t = *reinterpret_cast<const float4*>(qrow + 8 * s + 4 * half);
        qreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
    }
    floatx16 o[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) o[f] = zero16();
    float m_run = kMasked, l_run = 0.0f;

    int k_end = p.Sk;
    if (p.causal && q0 + 31 + p.causal_offset + 1 < k_end) k_end = q0 + 31 + p.causal_offset + 1;
    const int q_pos = qi + p.causal_offset;

    float4 kc[NS], vc[NS];
    auto fetch = [&](int kb) {
        int key = kb + l32;
        key = key < p.Sk ? key : p.Sk - 1;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            kc[s] = *reinterpret_cast<const float4*>(kbase + key * kst + 8 * s + 4 * half);
            vc[s] = *reinterpret_cast<const float4*>(vbase + key * kst + 8 * s + 4 * half);
        }
    };
    const int kb_first = wave * 32;
    if (kb_first < k_end) fetch(kb_first);
    for (int kb = kb_first; kb < k_end; kb += 32 * NSPL) {
#pragma unroll
        for (int s = 0; s < NS; s++)
            *reinterpret_cast<float4*>(vt + sw_off<DP>(l32, 2 * s + half)) =
                make_float4(vc[s].x, vc[s].y, vc[s].z, vc[s].w);
        floatx16 s = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            s = MFMA(kc[st].x, qreg[st].x, s);
            s = MFMA(kc[st].y, qreg[st].y, s);
            s = MFMA(kc[st].z, qreg[st].z, s);
            s = MFMA(kc[st].w, qreg[st].w, s);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kb + 32 * NSPL < k_end) fetch(kb + 32 * NSPL);
        __builtin_amdgcn_sched_barrier(0);
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
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[f][r] *= corr;
#pragma unroll
        for (int t4 = 0; t4 < 16; t4 += 4) {
            float av[4][NF];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int r = row_of(t4 + u, half);
#pragma unroll
                for (int f = 0; f < NF; f++) {
                    const int d = f * 32 + l32;
                    av[u][f] = vt[sw_off<DP>(r, d / 4) + (d & 3)];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int f = 0; f < NF; f++) o[f] = MFMA(av[u][f], s[t4 + u], o[f]);
        }
    }

    // Merge the waves' (m, l, O) into wave 0, in wave order (through the private tiles).
    constexpr int W = NF * 16 + 2;
    if (wave > 0) {
        float* dst = vt + lane * W;
        dst[0] = m_run;
        dst[1] = l_run;
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int r = 0; r < 16; r++) dst[2 + f * 16 + r] = o[f][r];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 1; w < NSPL; w++) {
        const float* src = lds + w * PRIV + lane * W;
        const float m_o = src[0], l_o = src[1];
        const float m_new = fmaxf(m_run, m_o);
        const float c0 = __expf(m_run - m_new), c1 = __expf(m_o - m_new);
        l_run = l_run * c0 + l_o * c1;
        m_run = m_new;
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[f][r] = o[f][r] * c0 + src[2 + f * 16 + r] * c1;
    }

    if (!q_ok) return;
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    float* orow = p.o + (((long)b * p.Sq + qi) * p.H + h) * DP;
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
            const int d = f * 32 + r4 * 8 + half * 4;
            *reinterpret_cast<float4*>(orow + d) = make_float4(o[f][r4 * 4 + 0] * inv, o[f][r4 * 4 + 1] * inv,
                                                               o[f][r4 * 4 + 2] * inv, o[f][r4 * 4 + 3] * inv);
        }
    if (p.stats && half == 0)
        p.stats[2 * (((long)b * p.H + h) * p.Sq + qi) + 1] = l_run > 0.0f ? m_run + __logf(l_run) : kLseEmpty;
}

template <int DP, int NSPL>
__global__ __launch_bounds__(NSPL * 64) void attn_bwd_dq_lds_kernel(AttnArgs p) {
    constexpr int NF = DP / 32;
    constexpr int NS = DP / 8;
    constexpr int TILE = 32 * DP;
    constexpr int MERGE = 64 * NF * 16;
    constexpr int PRIV = TILE > MERGE ? TILE : MERGE;
    __shared__ __attribute__((aligned(16))) float lds[NSPL * PRIV];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, l32 = lane % 32, half = lane / 32;
    float* kt = lds + wave * PRIV;
    int blk_j, bh_i;
    const int nqb_grid = (p.Sq + 31) / 32;
    if (!attn_work_item(nqb_grid, p.B * p.H, blk_j, bh_i)) return;
    const int b = bh_i / p.H, h = bh_i % p.H;
    const int kvh = h / (p.H / p.Hkv);
    const int q0 = (nqb_grid - 1 - blk_j) * 32;  // the last query block has the longest key loop: first
    const int qi = q0 + l32;
    const bool q_ok = qi < p.Sq;
    const int qc = q_ok ? qi : p.Sq - 1;
    const long qoff = (((long)b * p.Sq + qc) * p.H + h) * DP;
    const long srow = ((long)b * p.H + h) * p.Sq + qc;
    const long kst = (long)p.Hkv * DP;
    const float* kbase = p.k + ((long)b * p.Sk * p.Hkv + kvh) * DP;
    const float* vbase = p.v + ((long)b * p.Sk * p.Hkv + kvh) * DP;

    float4 qreg[NS], doreg[NS];
    float delta = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int d = 8 * s + 4 * half;
        const float4 t = *reinterpret_cast<const float4*>(p.q + qoff + d);
        qreg[s] = make_float4(t.x * p.scale, t.y * p.scale, t.z * p.scale, t.w * p.scale);
        doreg[s] = *reinterpret_cast<const float4*>(p.d_out + qoff + d);
        const float4 ov = *reinterpret_cast<const float4*>(p.out + qoff + d);
        delta += doreg[s].x * ov.x + doreg[s].y * ov.y + doreg[s].z * ov.z + doreg[s].w * ov.w;
    }
    delta += __shfl_xor(delta, 32, 64);
    const float lse = q_ok ? p.stats[2 * srow + 1] : kLseEmpty;
    if (q_ok && half == 0 && wave == 0) p.stats[2 * srow] = delta;

    floatx16 acc[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) acc[f] = zero16();

    int k_end = p.Sk;
    if (p.causal && q0 + 31 + p.causal_offset + 1 < k_end) k_end = q0 + 31 + p.causal_offset + 1;
    const int q_pos = qi + p.causal_offset;

    float4 kc[NS], vc[NS];
    auto fetch = [&](int kb) {
        int key = kb + l32;
        key = key < p.Sk ? key : p.Sk - 1;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            kc[s] = *reinterpret_cast<const float4*>(kbase + key * kst + 8 * s + 4 * half);
            vc[s] = *reinterpret_cast<const float4*>(vbase + key * kst + 8 * s + 4 * half);
        }
    };
    const int kb_first = wave * 32;
    if (kb_first < k_end) fetch(kb_first);
    for (int kb = kb_first; kb < k_end; kb += 32 * NSPL) {
#pragma unroll
        for (int s = 0; s < NS; s++) *reinterpret_cast<float4*>(kt + sw_off<DP>(l32, 2 * s + half)) = kc[s];
        floatx16 s = zero16(), dp = zero16();
#pragma unroll
        for (int st = 0; st < NS; st++) {
            s = MFMA(kc[st].x, qreg[st].x, s);
            s = MFMA(kc[st].y, qreg[st].y, s);
            s = MFMA(kc[st].z, qreg[st].z, s);
            s = MFMA(kc[st].w, qreg[st].w, s);
            dp = MFMA(vc[st].x, doreg[st].x, dp);
            dp = MFMA(vc[st].y, doreg[st].y, dp);
            dp = MFMA(vc[st].z, doreg[st].z, dp);
            dp = MFMA(vc[st].w, doreg[st].w, dp);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kb + 32 * NSPL < k_end) fetch(kb + 32 * NSPL);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int key = kb + row_of(t, half);
            const bool vis = q_ok && key < p.Sk && (!p.causal || key <= q_pos);
            const float pij = vis ? __expf(s[t] - lse) : 0.0f;
            s[t] = pij * (dp[t] - delta);
        }
#pragma unroll
        for (int t4 = 0; t4 < 16; t4 += 4) {
            float ak[4][NF];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int r = row_of(t4 + u, half);
#pragma unroll
                for (int f = 0; f < NF; f++) {
                    const int d = f * 32 + l32;
                    ak[u][f] = kt[sw_off<DP>(r, d / 4) + (d & 3)];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int f = 0; f < NF; f++) acc[f] = MFMA(ak[u][f], s[t4 + u], acc[f]);
        }
    }

    // Sum of the waves' partial dQ, in wave order (through the private tiles).
    constexpr int W = NF * 16;
    if (wave > 0) {
        float* dst = kt + lane * W;
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int r = 0; r < 16; r++) dst[f * 16 + r] = acc[f][r];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 1; w < NSPL; w++) {
        const float* src = lds + w * PRIV + lane * W;
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[f][r] += src[f * 16 + r];
    }

    if (!q_ok) return;
    float* drow = p.dq + qoff;
    if constexpr (DP == 64) {
        if (p.rope) {
            // pairs (d, d + 32) are registers r of accumulator blocks 0 and 1 of this lane
            const float2* tb = p.rope + (long)qi * 32;
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const int d = r4 * 8 + half * 4;
                float lo[4], hi[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float2 cs = tb[d + e];
                    const float x1 = acc[0][r4 * 4 + e] * p.scale, x2 = acc[1][r4 * 4 + e] * p.scale;
                    lo[e] = x1 * cs.x + x2 * cs.y;
                    hi[e] = x2 * cs.x - x1 * cs.y;
                }
                *reinterpret_cast<float4*>(drow + d) = make_float4(lo[0], lo[1], lo[2], lo[3]);
                *reinterpret_cast<float4*>(drow + 32 + d) = make_float4(hi[0], hi[1], hi[2], hi[3]);
            }
            return;
        }
    }
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
            const int d = f * 32 + r4 * 8 + half * 4;
            *reinterpret_cast<float4*>(drow + d) =
                make_float4(acc[f][r4 * 4 + 0] * p.scale, acc[f][r4 * 4 + 1] * p.scale, acc[f][r4 * 4 + 2] * p.scale,
                            acc[f][r4 * 4 + 3] * p.scale);
        }
}

// The unguarded vector loads need whole, aligned quads in every row.
bool attn_full(const AttnArgs& a, int DP) {
    auto al = [](const void* q) { return q == nullptr || (((uintptr_t)q) & 15) == 0; };
    // o (forward) and dq / dk / dv (backward) are written as 16-byte groups; NULL in the other pass
    return a.D == DP && al(a.q) && al(a.k) && al(a.v) && al(a.out) && al(a.d_out) && al(a.o) && al(a.dq) && al(a.dk) && al(a.dv);
}

template <int DP>
int launch_fwd(ft_context* ctx, const AttnArgs& a) {
    const dim3 grid(attn_grid(ft_div_up(a.Sq, 32), (size_t)a.B * a.H));
    // flop convention of the reference's benchmarks: causal forward 2*B*H*Sq*Sk*D, full 4*...
    const double fl = (a.causal ? 2.0 : 4.0) * a.B * a.H * (double)a.Sq * a.Sk * a.D;
    const double by = 4.0 * a.B * ((double)a.Sq * a.H * a.D * 2 + (double)a.Sk * a.Hkv * a.D * 2);
    ft_prof_scope prof(ctx, "attn_fwd_kernel", fl, by);
    if constexpr (DP <= 64) {
        if (DP == 64 && ft_attn16_usable(a) && ft_attn16_forward_pays(ctx, a)) return ft_attn16_forward(ctx, a);
        if (attn_full(a, DP)) {
            hipLaunchKernelGGL((attn_fwd_lds_kernel<DP>), grid, dim3(kKeySplit * 64), 0, ctx->stream, a);
            FT_LAUNCH_CHECK();
            return FT_OK;
        }
    }
    if (attn_full(a, DP))
        hipLaunchKernelGGL((attn_fwd_kernel<DP, true>), grid, dim3(kKeySplit * 64), 0, ctx->stream, a);
    else
        hipLaunchKernelGGL((attn_fwd_kernel<DP, false>), grid, dim3(kKeySplit * 64), 0, ctx->stream, a);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

template <int DP>
int launch_bwd(ft_context* ctx, const AttnArgs& a) {
    const dim3 grid(attn_grid(ft_div_up(a.Sq, 32), (size_t)a.B * a.H));
    // backward = 2.5x forward by the reference's convention, charged 1.0x to the dQ pass and 1.5x to dK/dV.
    const double fl = (a.causal ? 2.0 : 4.0) * a.B * a.H * (double)a.Sq * a.Sk * a.D;
    const double by = 4.0 * a.B * ((double)a.Sq * a.H * a.D * 4 + (double)a.Sk * a.Hkv * a.D * 4);
    const bool full = attn_full(a, DP);
    {
        ft_prof_scope prof(ctx, "attn_bwd_dq_kernel", 1.0 * fl, by * 0.5);
        bool done = false;
        if constexpr (DP <= 64) {
            if (full) {
                // Few workgroups (one or two sequences per pass): four waves share a query block's
                // keys instead of two, so the chip is not left to a long serial key loop.
                if (DP == 64 && ft_attn16_usable(a) && ft_attn16_backward_dq_pays(ctx, a)) {
                    FT_TRY(ft_attn16_backward_dq(ctx, a));
                } else if ((size_t)grid.x <= (size_t)ctx->num_cus && a.Sk > 64)
                    hipLaunchKernelGGL((attn_bwd_dq_lds_kernel<DP, 4>), grid, dim3(4 * 64), 0, ctx->stream, a);
                else
                    hipLaunchKernelGGL((attn_bwd_dq_lds_kernel<DP, kKeySplitDq>), grid, dim3(kKeySplitDq * 64), 0,
                                       ctx->stream, a);
                done = true;
            }
        }
        if (done) {
        } else if (full)
            hipLaunchKernelGGL((attn_bwd_dq_kernel<DP, true>), grid, dim3(kKeySplitDq * 64), 0, ctx->stream, a);
        else
            hipLaunchKernelGGL((attn_bwd_dq_kernel<DP, false>), grid, dim3(kKeySplitDq * 64), 0, ctx->stream, a);
    }
    FT_LAUNCH_CHECK();
    if constexpr (DP <= 64) {
        if (full) {
            constexpr int TILE = 32 * DP, REGION = 2 * DP * 33;
            constexpr int PRIV = (2 * TILE + 64) > REGION ? (2 * TILE + 64) : REGION;
            constexpr size_t smem_lds = (size_t)(2 * TILE + 8 * PRIV) * sizeof(float);
            static bool attr_lds = false;
            if (!attr_lds) {
                FT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dkdv_lds_kernel<DP>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_lds));
                attr_lds = true;
            }
            const size_t items = ft_div_up(a.Sk, 32) * (size_t)a.B * a.Hkv;
            const size_t G = (size_t)a.H / a.Hkv;
            const size_t n_all = (size_t)a.B * a.Sk * a.Hkv * DP;
            ft_prof_scope prof(ctx, "attn_bwd_dkdv_kernel", 1.5 * fl, by * 0.5);
            if (DP == 64 && ft_attn16_usable(a)) return ft_attn16_backward_dkdv(ctx, a);
            // Few items (one or two sequences per pass) and a GQA group to share them out:
            // one workgroup per query head, then the ordered sum over the group.
            if (G > 1 && items * 2 <= (size_t)ctx->num_cus && 2 * G * n_all <= kAttnScratchFloats) {
                if (!ctx->attn_scratch) {
                    FT_HIP(hipSetDevice(ctx->device));
                    FT_HIP(hipMalloc((void**)&ctx->attn_scratch, kAttnScratchFloats * sizeof(float)));
                }
                AttnArgs s = a;
                s.part = ctx->attn_scratch;
                s.split_g = 1;
                const dim3 grid_s(attn_grid(ft_div_up(a.Sk, 32), (size_t)a.B * a.H));
                hipLaunchKernelGGL((attn_bwd_dkdv_lds_kernel<DP>), grid_s, dim3(512), smem_lds, ctx->stream, s);
                FT_LAUNCH_CHECK();
                hipLaunchKernelGGL(attn_dkdv_combine_kernel, dim3(ft_div_up(n_all, 256)), dim3(256), 0, ctx->stream, s, DP);
                FT_LAUNCH_CHECK();
                return FT_OK;
            }
            const dim3 grid3(attn_grid(ft_div_up(a.Sk, 32), (size_t)a.B * a.Hkv));
            hipLaunchKernelGGL((attn_bwd_dkdv_lds_kernel<DP>), grid3, dim3(512), smem_lds, ctx->stream, a);
            FT_LAUNCH_CHECK();
            return FT_OK;
        }
    }
    constexpr size_t smem = (size_t)dkdv_waves(DP) * 2 * DP * 33 * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        FT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dkdv_kernel<DP, true>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        FT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dkdv_kernel<DP, false>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const dim3 grid2(attn_grid(ft_div_up(a.Sk, 32), (size_t)a.B * a.Hkv));
    {
        ft_prof_scope prof(ctx, "attn_bwd_dkdv_kernel", 1.5 * fl, by * 0.5);
        if (full)
            hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DP, true>), grid2, dim3(dkdv_waves(DP) * 64), smem, ctx->stream, a);
        else
            hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DP, false>), grid2, dim3(dkdv_waves(DP) * 64), smem, ctx->stream, a);
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
    FT_CHECK_ARG(B * H * ((Sq + 31) / 32 + (Sk + 31) / 32) < (1u << 30), "%s: too many blocks for one launch", who);
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

int ft_attn_dkdv_combine(ft_context* ctx, const AttnArgs& a, int DP) {
    const size_t n_all = (size_t)a.B * a.Sk * a.Hkv * DP;
    hipLaunchKernelGGL(attn_dkdv_combine_kernel, dim3(ft_div_up(n_all, 256)), dim3(256), 0, ctx->stream, a, DP);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

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

// Can the backward kernels rotate dQ and dK back through RoPE themselves (self-attention over
// whole rows from position 0, head_dim 64, aligned tensors)?
bool ft_internal_attention_rope_fusable(const float* q, const float* k, const float* v, const float* out,
                                        const float* d_out, size_t Sq, size_t Sk, size_t D) {
    AttnArgs a{};
    a.D = (int)D;
    a.q = q; a.k = k; a.v = v; a.out = out; a.d_out = d_out;
    return D == 64 && Sq == Sk && attn_full(a, 64);
}

// ft_flash_attention_v2_backward_with_stats followed by the inverse RoPE of dq and dk (positions
// 0..S-1, table from ft_internal_rope_table), in the same two launches.
int ft_internal_attention_backward_rope(ft_context* ctx, const float* q, const float* k, const float* v,
                                        const float* out, const float* d_out, float* dq, float* dk, float* dv,
                                        float* stats, size_t B, size_t S, size_t H, size_t Hkv,
                                        const ft_attention_options* opts, const float* rope_table) {
    FT_TRY(check_common("attention backward", ctx, B, S, S, H, Hkv, 64, opts));
    FT_CHECK_ARG(q && k && v && out && d_out && dq && dk && dv && stats && rope_table, "attention backward: NULL tensor");
    FT_CHECK_ARG(ft_internal_attention_rope_fusable(q, k, v, out, d_out, S, S, 64), "attention backward: not fusable");
    if (B == 0 || H == 0) return FT_OK;
    AttnArgs a = make_args(B, S, S, H, Hkv, 64, opts);
    a.q = q; a.k = k; a.v = v; a.out = out; a.d_out = d_out; a.dq = dq; a.dk = dk; a.dv = dv; a.stats = stats;
    a.rope = reinterpret_cast<const float2*>(rope_table);
    return launch_bwd<64>(ctx, a);
}
