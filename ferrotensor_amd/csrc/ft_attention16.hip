// Causal / full grouped-query flash attention for whole, 16-byte aligned head dims
// (32 and 64), built from 16-row wave tiles of v_mfma_f32_16x16x4_f32.
//
// Layout as in ft_attention.hip: q/out/dO/dq [B,Sq,H,D], k/v/dk/dv [B,Sk,Hkv,D],
// stats [B*H*Sq][2] = (Delta, log-sum-exp).
//
// A wave owns 16 rows (queries in the forward and dQ kernels, keys in the dK/dV
// kernel) and keeps what belongs to them in registers; the other side streams
// through LDS. Scores are computed transposed (S^T = K Q^T for a query wave), so
// a lane's accumulator registers are keys of ONE query: softmax statistics are
// per-lane scalars plus two cross-lane steps, and the probabilities are already
// the B operand of the next product. The 16x16x4 shape keeps a wave at about a
// hundred registers (four waves per SIMD) and cuts the causal triangle in 16-row
// steps.
//
// Operand layouts of v_mfma_f32_16x16x4_f32 (lane = l16 + 16 * g):
//   A[m][k]: lane (m = l16, k = g);  B[k][n]: lane (n = l16, k = g);
//   D[m][n]: lane (n = l16), register r holds row m = 4 g + r.
// A 16-byte LDS read of four consecutive head-dim values feeds four MFMAs: the
// contraction index (or output row) of MFMA e is permuted accordingly, the same
// way on both operands.
#include "ft_attention.h"

#include <type_traits>

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

constexpr int KT = 64;  // keys per shared K/V tile (forward, dQ)
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float log2_fast(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ floatx4 zero4() { return floatx4{0.0f, 0.0f, 0.0f, 0.0f}; }

// A query's (or key's) 16 values sit in the four lanes l16, l16 + 16, l16 + 32, l16 + 48: the two
// gfx950 lane swaps bring them together without a trip through LDS. v_permlane32_swap exchanges the
// upper 32 lanes of its first operand with the lower 32 of its second, v_permlane16_swap the odd
// 16-lane rows of the first with the even rows of the second; called on (x, x) the two results
// hold a lane's own value and its partner's.
__device__ __forceinline__ float group_max(float x) {
    auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
// Sum in a fixed order: (g0 + g1) + (g2 + g3) in every lane.
__device__ __forceinline__ float group_sum(float x) {
    auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(b[0]) + __uint_as_float(b[1]);
    auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(a[0]) + __uint_as_float(a[1]);
}
// The value held by the lane 32 away.
__device__ __forceinline__ float other_half(float x) {
    auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float lo = __uint_as_float(a[0]), hi = __uint_as_float(a[1]);
    // after the swap a[0] = (x.lo, x.lo) and a[1] = (x.hi, x.hi): lanes below 32 want x.hi
    return (threadIdx.x & 32) ? lo : hi;
}

// EV consecutive floats from LDS (EV * 4 bytes aligned).
template <int EV>
__device__ __forceinline__ void lds_vec(const float* src, float (&v)[EV]) {
    if constexpr (EV == 4) {
        const float4 t = *reinterpret_cast<const float4*>(src);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else if constexpr (EV == 2) {
        const float2 t = *reinterpret_cast<const float2*>(src);
        v[0] = t.x; v[1] = t.y;
    } else {
#pragma unroll
        for (int e = 0; e < EV; e++) v[e] = src[e];
    }
}
template <int EV>
__device__ __forceinline__ void store_vec(float* dst, const float (&v)[EV]) {
    if constexpr (EV == 4) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    } else if constexpr (EV == 2) {
        *reinterpret_cast<float2*>(dst) = make_float2(v[0], v[1]);
    } else {
#pragma unroll
        for (int e = 0; e < EV; e++) dst[e] = v[e];
    }
}

// Writes of a wave to its own LDS tile become visible to its later reads.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LDS tiles are rows of 64 floats (16 chunks of 16 bytes) with the chunk index XOR-swizzled by
// the row. gfx950 serves a 16-byte-per-lane LDS access 16 lanes at a time, and the 16 are not
// neighbours: lanes 0-3, 12-15, 20-23, 24-27 go together (measured), i.e. half of one 16-lane row
// and the other half of the next. Both access shapes used here must spread such a group over all
// 64 banks: "column" reads (lane l16 takes row l16, all four rows of lanes one chunk each) and
// "row" reads (the 16 lanes of a lane row take the 16 chunks of one tile row, each lane row its own
// tile row 4 apart). f(r) = r ^ ((r & 4) << 1) does that for both; plain padding cannot.
__device__ __forceinline__ int sw(int row, int chunk) {
    const int r = row & 15;
    return row * 64 + (((chunk ^ r ^ ((r & 4) << 1)) & 15) << 2);
}

// ---------------------------------------------------------------------------
// Work decomposition of the forward and dQ kernels. A head's queries are cut in
// tiles of TQ = 16 * NG rows; a workgroup takes the tile pair (nT - 1 - i, i) of
// one (batch, head): under the causal mask every pair is the same amount of work,
// and both tiles walk the same K/V tiles (64 keys, staged once in LDS for all
// waves, double buffered). Sixteen query rows belong to TWO waves, one per half of
// every K/V tile (keys 0-31 and 32-63 of the tile), so the longest chain of
// dependent work is half a row block's keys; the halves meet once, through LDS,
// after the last tile. Wave order: key half, then tile of the pair, then row
// block; the row blocks of the early tile are taken in reverse, so that the four
// waves on a SIMD (waves w, w + 4, ...) add up to the same key count everywhere.
// ---------------------------------------------------------------------------
constexpr int D64 = 64;
constexpr int TILE = KT * D64;   // floats of one K or V tile in LDS
constexpr int HALF = 32 * D64;   // floats of one key half of a tile

template <int NG>
struct QueryWave {
    static constexpr int TQ = 16 * NG;
    int b, h, kvh;
    int kh;        // key half of every tile this wave multiplies
    int w2;        // index among the waves of its half
    int q0w;       // first query row of this wave
    int q;         // this lane's query row (may be >= Sq)
    int qc;        // clamped to a valid row
    bool q_ok;
    int kend_w;    // one past the last key any row of this wave may see (0: nothing to do)
    int kfull_w;   // keys below this are visible to every row of the wave
    int nkt;       // K/V tiles the workgroup walks

    __device__ __forceinline__ void init(const AttnArgs& p, int wave, int l16) {
        const int nbh = p.B * p.H;
        const int nT = (p.Sq + TQ - 1) / TQ;
        const int pi = blockIdx.x / nbh, bh = blockIdx.x % nbh;
        b = bh / p.H;
        h = bh % p.H;
        kvh = h / (p.H / p.Hkv);
        const int JA = nT - 1 - pi, JB = pi;
        kh = wave / (2 * NG);
        w2 = wave % (2 * NG);
        const int grp = w2 / NG, wr = w2 % NG;
        const bool active = grp == 0 || JB != JA;
        const int J = grp == 0 ? JA : JB;
        const int rb = grp == 0 ? wr : NG - 1 - wr;
        q0w = J * TQ + 16 * rb;
        q = q0w + l16;
        q_ok = active && q < p.Sq;
        qc = q < p.Sq ? q : p.Sq - 1;
        const int qlast_w = q0w + 15 < p.Sq ? q0w + 15 : p.Sq - 1;
        kend_w = (active && q0w < p.Sq) ? key_end(p, qlast_w) : 0;
        kfull_w = p.causal ? q0w + p.causal_offset + 1 : p.Sk;
        if (kfull_w > p.Sk) kfull_w = p.Sk;
        const int qlast_wg = ((JA + 1) * TQ < p.Sq ? (JA + 1) * TQ : p.Sq) - 1;
        nkt = (key_end(p, qlast_wg) + KT - 1) / KT;
    }
    static __device__ __forceinline__ int key_end(const AttnArgs& p, int qlast) {
        int e = p.Sk;
        if (p.causal) {
            const int c = qlast + p.causal_offset + 1;
            e = c < e ? c : e;
        }
        return e < 0 ? 0 : e;
    }
    // 16-key sub-blocks of this wave's half of the tile at key kb that some row can see (0..2)
    __device__ __forceinline__ int visible_subblocks(int kb) const {
        int n = (kend_w - kb + 15) / 16 - 2 * kh;
        n = n < 2 ? n : 2;
        return n > 0 ? n : 0;
    }
    // is every key of this wave's half of that tile visible to every row?
    __device__ __forceinline__ bool half_unmasked(int kb) const { return kb + 32 * (kh + 1) <= kfull_w; }
};

// The K/V tile of 64 keys: global -> registers (the next tile's while the current one multiplies)
// -> LDS. Defines kv_fetch(t) and kv_store(stage) over the local arrays kpre, vpre.
#define FT_ATTN16_KV_LOADER(p, w, tid, smem)                                                         \
    constexpr int LPT = KT * 16 / NT;                                                                \
    static_assert(KT * 16 % NT == 0, "a K/V tile must divide evenly over the workgroup");            \
    float4 kpre[LPT], vpre[LPT];                                                                     \
    auto kv_fetch = [&](int t) {                                                                     \
        _Pragma("unroll") for (int u = 0; u < LPT; u++) {                                            \
            const int e = tid + NT * u;                                                              \
            const int r = e / 16, c = e % 16;                                                        \
            int key = t * KT + r;                                                                    \
            key = key < p.Sk ? key : p.Sk - 1;                                                       \
            const long o = (((long)w.b * p.Sk + key) * p.Hkv + w.kvh) * D64 + 4 * c;                 \
            kpre[u] = *reinterpret_cast<const float4*>(p.k + o);                                     \
            vpre[u] = *reinterpret_cast<const float4*>(p.v + o);                                     \
        }                                                                                            \
    };                                                                                               \
    auto kv_store = [&](int stage) {                                                                 \
        float* ks_ = smem + stage * 2 * TILE;                                                        \
        _Pragma("unroll") for (int u = 0; u < LPT; u++) {                                            \
            const int e = tid + NT * u;                                                              \
            const int r = e / 16, c = e % 16;                                                        \
            *reinterpret_cast<float4*>(ks_ + sw(r, c)) =                                             \
                make_float4(kpre[u].x, kpre[u].y, kpre[u].z, kpre[u].w);                             \
            *reinterpret_cast<float4*>(ks_ + TILE + sw(r, c)) =                                      \
                make_float4(vpre[u].x, vpre[u].y, vpre[u].z, vpre[u].w);                             \
        }                                                                                            \
    }

template <int NG>
__global__ __launch_bounds__(4 * NG * 64) void attn16_fwd_kernel(AttnArgs p) {
    constexpr int NT = 4 * NG * 64;
    extern __shared__ __attribute__((aligned(16))) float smem[];  // [2 stages][K tile, V tile]
    const int tid = threadIdx.x, lane = tid % 64, l16 = lane % 16, g = lane / 16;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);  // wave-uniform: the tile bookkeeping stays in SGPRs

    QueryWave<NG> w;
    w.init(p, wave, l16);
    FT_ATTN16_KV_LOADER(p, w, tid, smem);
    if (w.nkt > 0) kv_fetch(0);

    // this lane's swizzled offsets into a tile: "column" reads (row l16 of a sub-block, chunk
    // 4 blk + g) and "row" reads (row 4 g + i, chunk l16), both within the wave's key half
    int off_col[4], off_row[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        off_col[j] = sw(l16, 4 * j + g) + w.kh * HALF;
        off_row[j] = sw(4 * g + j, l16) + w.kh * HALF;
    }

    // scores are kept in base 2: log2(e) / sqrt(D) goes into Q
    const float qscale = p.scale * kLog2e;
    const float* qrow = p.q + (((long)w.b * p.Sq + w.qc) * p.H + w.h) * D64;
    float4 qf[4];
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
        const float4 t = *reinterpret_cast<const float4*>(qrow + 16 * blk + 4 * g);
        qf[blk] = make_float4(t.x * qscale, t.y * qscale, t.z * qscale, t.w * qscale);
    }
    floatx4 o[4];
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = zero4();
    float m_run = kAttnMasked, l_lane = 0.0f;
    // the last key this lane's query may see
    const int key_lim = (p.causal && w.q + p.causal_offset < p.Sk - 1) ? w.q + p.causal_offset : p.Sk - 1;

    if (w.nkt > 0) kv_store(0);
    __syncthreads();

    // This wave's half of one K/V tile against its 16 queries: NSB visible 16-key sub-blocks, MASK
    // when some key of them is hidden from some query (the diagonal, the end of the keys).
    auto tile = [&](auto nsb_tag, auto mask_tag, const float* ks, const float* vs, int kb) {
        constexpr int NSB = decltype(nsb_tag)::value;
        constexpr bool MASK = decltype(mask_tag)::value;
        floatx4 s[NSB];
#pragma unroll
        for (int u = 0; u < NSB; u++) s[u] = zero4();
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {
            float4 kq[NSB];
#pragma unroll
            for (int u = 0; u < NSB; u++) kq[u] = *reinterpret_cast<const float4*>(ks + off_col[blk] + u * 16 * D64);
#pragma unroll
            for (int u = 0; u < NSB; u++) s[u] = MFMA16(kq[u].x, qf[blk].x, s[u]);
#pragma unroll
            for (int u = 0; u < NSB; u++) s[u] = MFMA16(kq[u].y, qf[blk].y, s[u]);
#pragma unroll
            for (int u = 0; u < NSB; u++) s[u] = MFMA16(kq[u].z, qf[blk].z, s[u]);
#pragma unroll
            for (int u = 0; u < NSB; u++) s[u] = MFMA16(kq[u].w, qf[blk].w, s[u]);
        }
        float tmax = kAttnMasked;
#pragma unroll
        for (int u = 0; u < NSB; u++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if constexpr (MASK) {
                    const int key = kb + 32 * w.kh + 16 * u + 4 * g + i;
                    s[u][i] = key <= key_lim ? s[u][i] : kAttnMasked;
                }
                tmax = fmaxf(tmax, s[u][i]);
            }
        tmax = group_max(tmax);
        const float m_new = fmaxf(m_run, tmax);
        const float corr = exp2_fast(m_run - m_new);
        float psum = 0.0f;
#pragma unroll
        for (int u = 0; u < NSB; u++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float pj = exp2_fast(s[u][i] - m_new);
                if constexpr (MASK) pj = s[u][i] > kAttnMasked ? pj : 0.0f;
                s[u][i] = pj;
                psum += pj;
            }
        l_lane = l_lane * corr + psum;  // this lane's keys only; the lanes of a query meet at the end
        m_run = m_new;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] *= corr;
#pragma unroll
        for (int u = 0; u < NSB; u++) {
            float4 vv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) vv[i] = *reinterpret_cast<const float4*>(vs + off_row[i] + u * 16 * D64);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                o[0] = MFMA16(vv[i].x, s[u][i], o[0]);
                o[1] = MFMA16(vv[i].y, s[u][i], o[1]);
                o[2] = MFMA16(vv[i].z, s[u][i], o[2]);
                o[3] = MFMA16(vv[i].w, s[u][i], o[3]);
            }
        }
    };
    using std::integral_constant;

    for (int t = 0; t < w.nkt; t++) {
        const bool more = t + 1 < w.nkt;
        if (more) kv_fetch(t + 1);
        const float* ks = smem + (t & 1) * 2 * TILE;
        const float* vs = ks + TILE;
        const int kb = t * KT;
        const int nsb = w.visible_subblocks(kb);
        if (nsb > 0) {
            if (w.half_unmasked(kb))
                tile(integral_constant<int, 2>{}, std::false_type{}, ks, vs, kb);
            else if (nsb == 2)
                tile(integral_constant<int, 2>{}, std::true_type{}, ks, vs, kb);
            else
                tile(integral_constant<int, 1>{}, std::true_type{}, ks, vs, kb);
        }
        if (more) kv_store((t + 1) & 1);
        __syncthreads();
    }

    // The two key halves of a row block meet: the second half's (m, l, O) go through LDS (the
    // K/V stages are free now), lane for lane, and the first half finishes the softmax.
    float* mrg = smem + (w.w2 * 18) * 64 + lane;
    if (w.kh == 1) {
        mrg[0] = m_run;
        mrg[64] = l_lane;
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int r = 0; r < 4; r++) mrg[(2 + 4 * e + r) * 64] = o[e][r];
    }
    __syncthreads();
    if (w.kh == 1) return;
    {
        const float m_o = mrg[0], l_o = mrg[64];
        const float m_new = fmaxf(m_run, m_o);
        const float c0 = exp2_fast(m_run - m_new), c1 = exp2_fast(m_o - m_new);
        l_lane = l_lane * c0 + l_o * c1;
        m_run = m_new;
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int r = 0; r < 4; r++) o[e][r] = o[e][r] * c0 + mrg[(2 + 4 * e + r) * 64] * c1;
    }
    const float l_run = group_sum(l_lane);
    if (!w.q_ok) return;
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    // register r of accumulator e is head-dim index 4 * (4 g + r) + e
    float* orow = p.o + (((long)w.b * p.Sq + w.q) * p.H + w.h) * D64;
#pragma unroll
    for (int r = 0; r < 4; r++)
        *reinterpret_cast<float4*>(orow + 4 * (4 * g + r)) =
            make_float4(o[0][r] * inv, o[1][r] * inv, o[2][r] * inv, o[3][r] * inv);
    if (p.stats && g == 0)
        p.stats[2 * (((long)w.b * p.H + w.h) * p.Sq + w.q) + 1] =
            l_run > 0.0f ? (m_run + log2_fast(l_run)) * kLn2 : kAttnLseEmpty;
}

// ---------------------------------------------------------------------------
// Backward, pass 1: Delta = dO.O (stats slot 0) and dQ = scale * sum_j dS_ij K_j,
// dS = P (dO.V - Delta), P = exp(S - LSE). Same decomposition as the forward; the
// two key halves of a row block add their partial dQ through LDS at the end.
// ---------------------------------------------------------------------------
template <int NG>
__global__ __launch_bounds__(4 * NG * 64) void attn16_dq_kernel(AttnArgs p) {
    constexpr int NT = 4 * NG * 64;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, lane = tid % 64, l16 = lane % 16, g = lane / 16;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);

    QueryWave<NG> w;
    w.init(p, wave, l16);
    FT_ATTN16_KV_LOADER(p, w, tid, smem);
    if (w.nkt > 0) kv_fetch(0);

    int off_col[4], off_row[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        off_col[j] = sw(l16, 4 * j + g) + w.kh * HALF;
        off_row[j] = sw(4 * g + j, l16) + w.kh * HALF;
    }

    const float qscale = p.scale * kLog2e;
    const long qoff = (((long)w.b * p.Sq + w.qc) * p.H + w.h) * D64;
    const long srow = ((long)w.b * p.H + w.h) * p.Sq + w.qc;
    float4 qf[4], dof[4];
    float delta = 0.0f;
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
        const int d = 16 * blk + 4 * g;
        const float4 t = *reinterpret_cast<const float4*>(p.q + qoff + d);
        qf[blk] = make_float4(t.x * qscale, t.y * qscale, t.z * qscale, t.w * qscale);
        dof[blk] = *reinterpret_cast<const float4*>(p.d_out + qoff + d);
        const float4 ov = *reinterpret_cast<const float4*>(p.out + qoff + d);
        delta += dof[blk].x * ov.x + dof[blk].y * ov.y + dof[blk].z * ov.z + dof[blk].w * ov.w;
    }
    delta = group_sum(delta);
    const float lse2 = (w.q_ok ? p.stats[2 * srow + 1] : kAttnLseEmpty) * kLog2e;
    if (w.q_ok && g == 0 && w.kh == 0) p.stats[2 * srow] = delta;

    floatx4 acc[4];
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] = zero4();
    // the last key this lane's query may see
    const int key_lim = (p.causal && w.q + p.causal_offset < p.Sk - 1) ? w.q + p.causal_offset : p.Sk - 1;

    if (w.nkt > 0) kv_store(0);
    __syncthreads();

    auto tile = [&](auto nsb_tag, auto mask_tag, const float* ks, const float* vs, int kb) {
        constexpr int NSB = decltype(nsb_tag)::value;
        constexpr bool MASK = decltype(mask_tag)::value;
        floatx4 s[NSB], dp[NSB];
#pragma unroll
        for (int u = 0; u < NSB; u++) {
            s[u] = zero4();
            dp[u] = zero4();
        }
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {
            float4 kq[NSB], vq[NSB];
#pragma unroll
            for (int u = 0; u < NSB; u++) {
                kq[u] = *reinterpret_cast<const float4*>(ks + off_col[blk] + u * 16 * D64);
                vq[u] = *reinterpret_cast<const float4*>(vs + off_col[blk] + u * 16 * D64);
            }
#pragma unroll
            for (int u = 0; u < NSB; u++) {
                s[u] = MFMA16(kq[u].x, qf[blk].x, s[u]);
                dp[u] = MFMA16(vq[u].x, dof[blk].x, dp[u]);
            }
#pragma unroll
            for (int u = 0; u < NSB; u++) {
                s[u] = MFMA16(kq[u].y, qf[blk].y, s[u]);
                dp[u] = MFMA16(vq[u].y, dof[blk].y, dp[u]);
            }
#pragma unroll
            for (int u = 0; u < NSB; u++) {
                s[u] = MFMA16(kq[u].z, qf[blk].z, s[u]);
                dp[u] = MFMA16(vq[u].z, dof[blk].z, dp[u]);
            }
#pragma unroll
            for (int u = 0; u < NSB; u++) {
                s[u] = MFMA16(kq[u].w, qf[blk].w, s[u]);
                dp[u] = MFMA16(vq[u].w, dof[blk].w, dp[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < NSB; u++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float pij = exp2_fast(s[u][i] - lse2);
                if constexpr (MASK) {
                    const int key = kb + 32 * w.kh + 16 * u + 4 * g + i;
                    pij = key <= key_lim ? pij : 0.0f;
                }
                s[u][i] = pij * (dp[u][i] - delta);  // dS
            }
#pragma unroll
        for (int u = 0; u < NSB; u++) {
            float4 kk[4];
#pragma unroll
            for (int i = 0; i < 4; i++) kk[i] = *reinterpret_cast<const float4*>(ks + off_row[i] + u * 16 * D64);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                acc[0] = MFMA16(kk[i].x, s[u][i], acc[0]);
                acc[1] = MFMA16(kk[i].y, s[u][i], acc[1]);
                acc[2] = MFMA16(kk[i].z, s[u][i], acc[2]);
                acc[3] = MFMA16(kk[i].w, s[u][i], acc[3]);
            }
        }
    };
    using std::integral_constant;

    for (int t = 0; t < w.nkt; t++) {
        const bool more = t + 1 < w.nkt;
        if (more) kv_fetch(t + 1);
        const float* ks = smem + (t & 1) * 2 * TILE;
        const float* vs = ks + TILE;
        const int kb = t * KT;
        const int nsb = w.visible_subblocks(kb);
        if (nsb > 0) {
            if (w.half_unmasked(kb))
                tile(integral_constant<int, 2>{}, std::false_type{}, ks, vs, kb);
            else if (nsb == 2)
                tile(integral_constant<int, 2>{}, std::true_type{}, ks, vs, kb);
            else
                tile(integral_constant<int, 1>{}, std::true_type{}, ks, vs, kb);
        }
        if (more) kv_store((t + 1) & 1);
        __syncthreads();
    }

    // the second key half's partial dQ joins the first's, lane for lane
    float* mrg = smem + (w.w2 * 16) * 64 + lane;
    if (w.kh == 1) {
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int r = 0; r < 4; r++) mrg[(4 * e + r) * 64] = acc[e][r];
    }
    __syncthreads();
    if (w.kh == 1) return;
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[e][r] += mrg[(4 * e + r) * 64];

    // K in LDS carries no scale (only Q does, for the scores): dQ = scale * dS K.
    // Register r of accumulator e is head-dim index 4 * (4 g + r) + e.
    float* drow = p.dq + qoff;
    if (p.rope) {
        // the partner of head-dim index d (d +- 32) sits in lane g ^ 2 at the same register
        const float2* tb = p.rope + (long)w.qc * 32;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float own = acc[e][r] * p.scale;
                const float other = other_half(own);
                const float2 cs = tb[(16 * g + 4 * r + e) & 31];
                v[e] = g < 2 ? own * cs.x + other * cs.y : own * cs.x - other * cs.y;
            }
            if (w.q_ok) *reinterpret_cast<float4*>(drow + 16 * g + 4 * r) = make_float4(v[0], v[1], v[2], v[3]);
        }
        return;
    }
    if (!w.q_ok) return;
#pragma unroll
    for (int r = 0; r < 4; r++)
        *reinterpret_cast<float4*>(drow + 4 * (4 * g + r)) =
            make_float4(acc[0][r] * p.scale, acc[1][r] * p.scale, acc[2][r] * p.scale, acc[3][r] * p.scale);
}

// ---------------------------------------------------------------------------
// Backward, pass 2: dK and dV of 16 keys of one (batch, kv head), summed over the
// query heads of the group and over the 16-query blocks that can see them. The
// key block (K pre-scaled for the base-2 scores, V) sits in LDS for all eight
// waves; the (head, query block) items are dealt round-robin to the waves, which
// run without a barrier until the end: an item's Q and dO rows come from global
// memory as 16-byte quads straight into the A operands of S = Q K^T and
// dP = dO V^T (the next item's while the current one multiplies), pass through a
// wave-private LDS tile, and are read back with the head dim as the row for
// dV^T += dO^T P and dK^T += Q^T dS. The waves' partial sums are added in wave
// order through LDS (no atomics). One workgroup per (key block, batch * kv head),
// key block 0 (the most items under the causal mask) first.
// ---------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(512, 4) void attn16_dkdv_kernel(AttnArgs p) {
    constexpr int NB = DP / 16, EV = DP / 16, PITCH = DP, NW = 8, C4 = DP / 4;
    constexpr int BLK = 16 * PITCH;
    extern __shared__ __attribute__((aligned(16))) float smem[];  // K block, V block, 8 x (Q tile, dO tile)
    const int tid = threadIdx.x, lane = tid % 64, l16 = lane % 16, g = lane / 16;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);  // wave-uniform: keeps the tile bookkeeping in SGPRs
    float* ks = smem;
    float* vs = smem + BLK;
    float* qs = smem + 2 * BLK + wave * 2 * BLK;
    float* dos = qs + BLK;

    const int nhu = p.B * (p.split_g ? p.H : p.Hkv);
    const int kbi = blockIdx.x / nhu, bh = blockIdx.x % nhu;
    const int Gfull = p.H / p.Hkv;
    const int b = bh / (p.split_g ? p.H : p.Hkv);
    const int hsel = bh % (p.split_g ? p.H : p.Hkv);
    const int kvh = p.split_g ? hsel / Gfull : hsel;
    const int g0 = p.split_g ? hsel % Gfull : 0;  // first query head of this workgroup within the group
    const int G = p.split_g ? 1 : Gfull;          // and how many it covers
    const int kb0 = kbi * 16;
    const int key = kb0 + l16;
    const int key_m = key < p.Sk ? key : 0x7fffffff;  // a key past the end is visible to nobody

    const float kscale = p.scale * kLog2e;
    for (int e = tid; e < 2 * 16 * C4; e += NW * 64) {
        const int which = e / (16 * C4), r = (e / C4) % 16, c = e % C4;
        int kr = kb0 + r;
        kr = kr < p.Sk ? kr : p.Sk - 1;
        const long o = (((long)b * p.Sk + kr) * p.Hkv + kvh) * DP + 4 * c;
        if (which == 0) {
            const float4 t = *reinterpret_cast<const float4*>(p.k + o);
            *reinterpret_cast<float4*>(ks + sw(r, c)) =
                make_float4(t.x * kscale, t.y * kscale, t.z * kscale, t.w * kscale);
        } else {
            *reinterpret_cast<float4*>(vs + sw(r, c)) = *reinterpret_cast<const float4*>(p.v + o);
        }
    }

    // 16-query blocks that can see this key block
    const int nqb = (p.Sq + 15) / 16;
    int qb_start = 0;
    if (p.causal) {
        const int first_q = kb0 - p.causal_offset;  // smallest i with i + offset >= kb0
        qb_start = first_q > 0 ? first_q / 16 : 0;
    }
    const int per_head = nqb > qb_start ? nqb - qb_start : 0;
    const int items = per_head * G;

    float4 qa[NB], da[NB];
    float2 st[4];
    auto fetch = [&](int item) {
        const int gi = item / per_head;
        const int q0 = (qb_start + item % per_head) * 16;
        const int h = kvh * Gfull + g0 + gi;
        int qr = q0 + l16;
        qr = qr < p.Sq ? qr : p.Sq - 1;
        const long ro = (((long)b * p.Sq + qr) * p.H + h) * DP;
#pragma unroll
        for (int blk = 0; blk < NB; blk++) {
            qa[blk] = *reinterpret_cast<const float4*>(p.q + ro + 16 * blk + 4 * g);
            da[blk] = *reinterpret_cast<const float4*>(p.d_out + ro + 16 * blk + 4 * g);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int qi = q0 + 4 * g + i;
            qi = qi < p.Sq ? qi : p.Sq - 1;
            st[i] = *reinterpret_cast<const float2*>(p.stats + 2 * (((long)b * p.H + h) * p.Sq + qi));
        }
    };
    if (wave < items) fetch(wave);
    __syncthreads();  // K/V block complete

    floatx4 dk[EV], dv[EV];
#pragma unroll
    for (int e = 0; e < EV; e++) {
        dk[e] = zero4();
        dv[e] = zero4();
    }

    for (int item = wave; item < items; item += NW) {
        const int q0 = (qb_start + item % per_head) * 16;
        // this item's rows -> the wave's LDS tile (for the transposed reads further down)
#pragma unroll
        for (int blk = 0; blk < NB; blk++) {
            *reinterpret_cast<float4*>(qs + sw(l16, 4 * blk + g)) = qa[blk];
            *reinterpret_cast<float4*>(dos + sw(l16, 4 * blk + g)) = da[blk];
        }
        floatx4 s = zero4(), dp = zero4();
#pragma unroll
        for (int blk = 0; blk < NB; blk++) {
            const float4 kq = *reinterpret_cast<const float4*>(ks + sw(l16, 4 * blk + g));
            const float4 vq = *reinterpret_cast<const float4*>(vs + sw(l16, 4 * blk + g));
            s = MFMA16(qa[blk].x, kq.x, s);
            dp = MFMA16(da[blk].x, vq.x, dp);
            s = MFMA16(qa[blk].y, kq.y, s);
            dp = MFMA16(da[blk].y, vq.y, dp);
            s = MFMA16(qa[blk].z, kq.z, s);
            dp = MFMA16(da[blk].z, vq.z, dp);
            s = MFMA16(qa[blk].w, kq.w, s);
            dp = MFMA16(da[blk].w, vq.w, dp);
        }
        // register i of this lane is query q0 + 4 g + i against key `key`
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // visible: a real key, a real query, and not above the diagonal; written without
            // short-circuit operators so that it stays a select (exp2(-inf) = 0)
            const int qi = q0 + 4 * g + i;
            const int lim = qi < p.Sq ? (p.causal ? qi + p.causal_offset : 0x7ffffffe) : -1;
            const float pij = exp2_fast(key_m <= lim ? s[i] - st[i].y * kLog2e : -INFINITY);
            s[i] = pij;                        // P
            dp[i] = pij * (dp[i] - st[i].x);   // dS
        }
        // the next item's rows travel while the rest of this one is computed
        fetch(item + NW < items ? item + NW : item);  // (the last item is fetched again: no branch, no copies)
        wave_lds_fence();
        float ao[4][EV], aq[4][EV];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lds_vec<EV>(dos + sw(4 * g + i, l16), ao[i]);
            lds_vec<EV>(qs + sw(4 * g + i, l16), aq[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int e = 0; e < EV; e++) {
                dv[e] = MFMA16(ao[i][e], s[i], dv[e]);
                dk[e] = MFMA16(aq[i][e], dp[i], dk[e]);
            }
        wave_lds_fence();  // the tile is rewritten by the next item
    }

    // Cross-wave sum in wave order. A wave's tile pair takes its partial dK (Q tile) and dV (dO tile)
    // as [key][head dim]; register r of accumulator e is head-dim index EV * (4 g + r) + e.
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float a[EV], c[EV];
#pragma unroll
        for (int e = 0; e < EV; e++) {
            a[e] = dk[e][r];
            c[e] = dv[e][r];
        }
        store_vec<EV>(qs + sw(l16, 4 * g + r), a);
        store_vec<EV>(dos + sw(l16, 4 * g + r), c);
    }
    __syncthreads();
    const float* red = smem + 2 * BLK;
    for (int e = tid; e < 2 * 16 * C4; e += NW * 64) {
        const int which = e / (16 * C4), kk = (e / C4) % 16, c = e % C4;
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int wv = 0; wv < NW; wv++) {
            const float4 t = *reinterpret_cast<const float4*>(red + (wv * 2 + which) * BLK + sw(kk, c));
            sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
        }
        const int krow = kb0 + kk;
        const long o = (((long)b * p.Sk + krow) * p.Hkv + kvh) * DP + 4 * c;
        if (p.split_g) {
            if (krow < p.Sk) {
                const long n_all = (long)p.B * p.Sk * p.Hkv * DP;
                *reinterpret_cast<float4*>(p.part + (2 * g0 + which) * n_all + o) = sum;
            }
            continue;
        }
        if (which == 1) {
            if (krow < p.Sk) *reinterpret_cast<float4*>(p.dv + o) = sum;
            continue;
        }
        // dK = scale * sum dS Q (Q is read unscaled)
        sum.x *= p.scale; sum.y *= p.scale; sum.z *= p.scale; sum.w *= p.scale;
        if (DP == 64 && p.rope) {
            // rotated back: the partner chunk (head-dim index +- 32) is held by lane ^ 8 of this wave
            float4 oth;
            oth.x = __shfl_xor(sum.x, 8, 64);
            oth.y = __shfl_xor(sum.y, 8, 64);
            oth.z = __shfl_xor(sum.z, 8, 64);
            oth.w = __shfl_xor(sum.w, 8, 64);
            const int kc = krow < p.Sk ? krow : p.Sk - 1;
            const float2* tb = p.rope + (long)kc * 32 + ((4 * c) & 31);
            const float2 c0 = tb[0], c1 = tb[1], c2 = tb[2], c3 = tb[3];
            const float sg = c < 8 ? 1.0f : -1.0f;
            sum = make_float4(sum.x * c0.x + sg * oth.x * c0.y, sum.y * c1.x + sg * oth.y * c1.y,
                              sum.z * c2.x + sg * oth.z * c2.y, sum.w * c3.x + sg * oth.w * c3.y);
        }
        if (krow < p.Sk) *reinterpret_cast<float4*>(p.dk + o) = sum;
    }
}

template <typename K>
int set_smem(K kernel, size_t bytes) {
    FT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)bytes));
    return FT_OK;
}

template <int NG>
int launch_query_kernels(ft_context* ctx, const AttnArgs& a, bool backward) {
    constexpr int TQ = 16 * NG;
    constexpr size_t smem = (size_t)2 * 2 * TILE * sizeof(float);
    static bool attr = false;
    if (!attr) {
        FT_TRY(set_smem(&attn16_fwd_kernel<NG>, smem));
        FT_TRY(set_smem(&attn16_dq_kernel<NG>, smem));
        attr = true;
    }
    const size_t nT = ft_div_up(a.Sq, TQ);
    const dim3 grid((unsigned)(((nT + 1) / 2) * (size_t)a.B * a.H));
    if (backward)
        hipLaunchKernelGGL((attn16_dq_kernel<NG>), grid, dim3(4 * NG * 64), smem, ctx->stream, a);
    else
        hipLaunchKernelGGL((attn16_fwd_kernel<NG>), grid, dim3(4 * NG * 64), smem, ctx->stream, a);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// Which tile height the forward (backward = false) or dQ kernel should run with at this shape:
// 4 (64-row tiles, 16 waves), 2 (32-row tiles, 8 waves) or 0 (too few workgroups for either: the
// caller keeps the 32-row kernels that split the keys of a query block over waves). Thresholds
// from timings at 1-32 sequences of 15 and 9 heads x 256 tokens and at 1024 tokens.
int query_tile_groups(const ft_context* ctx, const AttnArgs& a, bool backward) {
    const size_t wgs64 = (ft_div_up(a.Sq, 64) + 1) / 2 * (size_t)a.B * a.H;
    const size_t cus = (size_t)ctx->num_cus;
    if (backward) {
        if (wgs64 * 5 >= cus * 4) return 4;
        // the 8-wave dQ kernel holds one workgroup per CU: it pays while one round covers the launch
        if (wgs64 * 4 >= cus && ((ft_div_up(a.Sq, 32) + 1) / 2) * (size_t)a.B * a.H <= cus) return 2;
        return 0;
    }
    if (wgs64 * 2 >= cus) return 4;
    if (wgs64 * 4 >= cus) return 2;
    return 0;
}

template <int DP>
int launch_dkdv(ft_context* ctx, const AttnArgs& a) {
    constexpr size_t smem = (size_t)(2 + 8 * 2) * 16 * DP * sizeof(float);
    static bool attr = false;
    if (!attr) {
        FT_TRY(set_smem(&attn16_dkdv_kernel<DP>, smem));
        attr = true;
    }
    const size_t nkb = ft_div_up(a.Sk, 16);
    const size_t G = (size_t)a.H / a.Hkv;
    const size_t n_all = (size_t)a.B * a.Sk * a.Hkv * DP;
    // Few (key block, kv head) units and a GQA group to share them out: one workgroup per query
    // head, then the ordered sum over the group.
    if (G > 1 && nkb * a.B * a.Hkv < 2 * (size_t)ctx->num_cus && 2 * G * n_all <= kAttnScratchFloats) {
        if (!ctx->attn_scratch) {
            FT_HIP(hipSetDevice(ctx->device));
            FT_HIP(hipMalloc((void**)&ctx->attn_scratch, kAttnScratchFloats * sizeof(float)));
        }
        AttnArgs s = a;
        s.part = ctx->attn_scratch;
        s.split_g = 1;
        hipLaunchKernelGGL((attn16_dkdv_kernel<DP>), dim3((unsigned)(nkb * a.B * a.H)), dim3(512), smem, ctx->stream, s);
        FT_LAUNCH_CHECK();
        return ft_attn_dkdv_combine(ctx, s, DP);
    }
    hipLaunchKernelGGL((attn16_dkdv_kernel<DP>), dim3((unsigned)(nkb * a.B * a.Hkv)), dim3(512), smem, ctx->stream, a);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

}  // namespace

bool ft_attn16_usable(const AttnArgs& a) {
    auto al = [](const void* q) { return q == nullptr || (((uintptr_t)q) & 15) == 0; };
    return a.D == 64 && a.Sq > 0 && a.Sk > 0 && al(a.q) && al(a.k) && al(a.v) && al(a.out) && al(a.d_out) &&
           al(a.o) && al(a.dq) && al(a.dk) && al(a.dv) && (((uintptr_t)a.stats) & 7) == 0;
}

bool ft_attn16_forward_pays(const ft_context* ctx, const AttnArgs& a) { return query_tile_groups(ctx, a, false) != 0; }
bool ft_attn16_backward_dq_pays(const ft_context* ctx, const AttnArgs& a) { return query_tile_groups(ctx, a, true) != 0; }

int ft_attn16_forward(ft_context* ctx, const AttnArgs& a) {
    return query_tile_groups(ctx, a, false) == 2 ? launch_query_kernels<2>(ctx, a, false)
                                                 : launch_query_kernels<4>(ctx, a, false);
}

int ft_attn16_backward_dq(ft_context* ctx, const AttnArgs& a) {
    return query_tile_groups(ctx, a, true) == 2 ? launch_query_kernels<2>(ctx, a, true)
                                                : launch_query_kernels<4>(ctx, a, true);
}

int ft_attn16_backward_dkdv(ft_context* ctx, const AttnArgs& a) { return launch_dkdv<64>(ctx, a); }
