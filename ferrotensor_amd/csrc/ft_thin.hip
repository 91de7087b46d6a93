// The rank-r products around a LoRA linear (r = 4, 8 or 16): bandwidth-bound
// work with almost no flops: fully coalesced 16-byte loads, the small
// contraction on the matrix unit, several independent products per launch.
//
//   row-wise   out[M, C] = scale * X[M, K] @ Y        (x@A,  dT = dY@B^T)
//              16 rows per workgroup, K split over its 4 waves, 16x16x4 MFMA
//              (the matrix unit does the K reduction, no cross-lane shuffles).
//   col-wise   out[R, C] = X[M, R]^T @ Y[M, C]        (dA = x^T@dT, dB = T^T@dY)
//              64 columns of X per workgroup, the M rows cut into slices and
//              contracted by the same MFMA; a second kernel adds the slices
//              in order (deterministic, no atomics).
#include "ft_common.h"
#include "ft_thin.h"

namespace {

constexpr int kWave = 64;

struct ThinBatch {
    ft_thin_problem p[FT_THIN_MAX_BATCH];
    int count;
};

// ---- row-wise ---------------------------------------------------------------
// grid (ceil(M / 16), count); 512 threads = 8 waves. A workgroup owns 16 rows;
// each wave takes an eighth of K through v_mfma_f32_16x16x4_f32 (X rows are the
// A operand, Y columns the B operand, columns >= C fed with zeros), and the eight
// partial 16x16 tiles are added in wave order through LDS. A wave issues the
// loads of 8 iterations (128 k) together: at K around 1000 that is all of them,
// so the launch costs one memory round trip. Every lane reads X in
// 16-byte pieces: lane (row = l % 16, q = l / 16) takes k = 16*it + 4*q .. +3,
// so MFMA e of an iteration contracts k = 16*it + 4*q + e.
typedef float thin_f4 __attribute__((ext_vector_type(4)));

// 16 bytes from device memory (16-byte aligned).
__device__ __forceinline__ float4 load_f4(const ft_global_f* q) {
    const thin_f4 v = *reinterpret_cast<const __attribute__((address_space(1))) thin_f4*>(q);
    return make_float4(v.x, v.y, v.z, v.w);
}

constexpr int kRowWaves = 8;

template <int C, bool YT>
__global__ __launch_bounds__(kRowWaves * 64) void thin_rowwise_kernel(ThinBatch b) {
    // The problem's entry of the argument block, read once (all reads, then all pins: one round trip).
    const ft_thin_problem& pk = b.p[blockIdx.y];
    struct {
        const ft_global_f* x;
        const ft_global_f* y;
        ft_global_f* out;
        int M, K;
        long ldx, ldy, ldo;
        float scale;
    } p;
    {
        const float* rx = pk.x;
        const float* ry = pk.y;
        float* ro = pk.out;
        const int rM = pk.M, rK = pk.K;
        const long rldx = pk.ldx, rldy = pk.ldy, rldo = pk.ldo;
        const float rs = pk.scale;
        p.x = (const ft_global_f*)ft_pinned(rx);
        p.y = (const ft_global_f*)ft_pinned(ry);
        p.out = (ft_global_f*)ft_pinned(ro);
        p.M = ft_pinned(rM);
        p.K = ft_pinned(rK);
        p.ldx = ft_pinned(rldx);
        p.ldy = ft_pinned(rldy);
        p.ldo = ft_pinned(rldo);
        p.scale = ft_pinned(rs);
    }
    const int row0 = blockIdx.x * 16;
    if (row0 >= p.M) return;
    __shared__ float red[kRowWaves][16][17];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int li = lane % 16, q = lane / 16;
    const int row = row0 + li < p.M ? row0 + li : p.M - 1;  // clamped rows are computed and dropped
    const ft_global_f* xr = p.x + (long)row * p.ldx + 4 * q;
    const bool col_live = li < C;
    // K is a multiple of 4; the parts are multiples of 16, so a 4-run of k is all in or all out.
    const int part = ((p.K + 16 * kRowWaves - 1) / (16 * kRowWaves)) * 16;
    const int k_begin = wave * part;
    const int k_end = k_begin + part < p.K ? k_begin + part : p.K;
    thin_f4 acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int U = 8;  // iterations whose loads are issued together
    for (int k0 = k_begin; k0 < k_end; k0 += 16 * U) {
        float4 xa[U];
        float yb[U][4];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + 16 * u + 4 * q;
            const bool in = k < k_end;
            xa[u] = in ? load_f4(xr + k0 + 16 * u) : make_float4(0.f, 0.f, 0.f, 0.f);
            if constexpr (YT) {
                const float4 t = (in && col_live) ? load_f4(p.y + (long)li * p.ldy + k) : make_float4(0.f, 0.f, 0.f, 0.f);
                yb[u][0] = t.x, yb[u][1] = t.y, yb[u][2] = t.z, yb[u][3] = t.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) yb[u][e] = (in && col_live) ? p.y[(long)(k + e) * C + li] : 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[u].x, yb[u][0], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[u].y, yb[u][1], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[u].z, yb[u][2], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[u].w, yb[u][3], acc, 0, 0, 0);
        }
    }
    // accumulator register r holds row 4*q + r, column li
#pragma unroll
    for (int r = 0; r < 4; r++) red[wave][4 * q + r][li] = acc[r];
    __syncthreads();
    const int orow = threadIdx.x / 16, ocol = threadIdx.x % 16;
    if (threadIdx.x < 256 && ocol < C && row0 + orow < p.M) {
        float v = red[0][orow][ocol];
#pragma unroll
        for (int w = 1; w < kRowWaves; w++) v += red[w][orow][ocol];
        p.out[(long)(row0 + orow) * p.ldo + ocol] = v * p.scale;
    }
}

// ---- col-wise ---------------------------------------------------------------
// out_i[R, C] = X[M, R]^T @ Y_i[M, C] for up to three Y_i that share X (the dA of q/k/v all
// contract the same norm output with their own dT): X is read once for all of them.
//
// The contraction over the M rows runs on the matrix unit: v_mfma_f32_16x16x4_f32 with the
// factor columns as the 16 output rows (virtual column v = i * C + c of product i; 16 per "set",
// up to 3 sets, unused ones fed zeros), 4 rows of M as k, and 16 columns of X as output columns.
// A lane (j = lane % 16, kq = lane / 16) fetches X[m0 + kq][n0 + 4j .. 4j+3] as one 16-byte load:
// a wave load covers four 256-byte row segments, and component e of the quad feeds MFMA e, whose
// tile therefore holds the columns n0 + 4j + e. One load instruction pays for 4 * sets MFMAs and a
// wave keeps eight of them in flight.
//
// grid (column tiles of 64 over all problems of the batch, M slices); 256 threads = 4 waves that
// split the slice's rows; their tiles are added in wave order through LDS and the workgroup
// writes one partial tile: partial[((slice * R) + n) * VC + v] at p.scratch_offset, VC = ny * C.
// thin_colwise_finish_kernel adds the slices in order (deterministic, no atomics).
struct ColProblem {
    const float* x;
    const float* y[3];
    float* out[3];
    int M, R, C, ny;
    long ldx, ldy, ldo;
    float scale;
    int out_transposed, accumulate;
    long scratch_offset;
    int tile_begin;   // index of this problem's first column tile in grid.x
    int slices;       // M slices of this problem (<= gridDim.y)
};

struct ColBatch {
    ColProblem p[FT_THIN_MAX_BATCH];
    int count;
    int rows_per_wg;    // multiple of 4 * kColWaves
    int rows_per_wave;  // rows_per_wg / kColWaves
};

constexpr int kColWaves = 4;
constexpr int kColUnroll = 8;   // 4-row groups whose loads are issued together

// The loads of one batch: kColUnroll groups of 4 rows from m0 (rows >= m_end read as zeros).
template <int NSET>
__device__ __forceinline__ void col_load(const float* xp, long ldx, const float* const (&yp)[NSET], long ldy, int nsets,
                                         int m0, int m_end, int kq, bool live, float4 (&xv)[kColUnroll],
                                         float (&yv)[kColUnroll][NSET]) {
#pragma unroll
    for (int u = 0; u < kColUnroll; u++) {
        const int m = m0 + 4 * u + kq;
        const bool in = m < m_end;
        xv[u] = (in && live) ? *reinterpret_cast<const float4*>(xp + (long)m * ldx) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int s = 0; s < NSET; s++) {
            yv[u][s] = 0.0f;
            if (s < nsets) yv[u][s] = (in && yp[s]) ? yp[s][(long)m * ldy] : 0.0f;
        }
    }
}

template <int NSET>
__device__ __forceinline__ void col_mfma(thin_f4 (&acc)[NSET][4], int nsets, const float4 (&xv)[kColUnroll],
                                         const float (&yv)[kColUnroll][NSET]) {
#pragma unroll
    for (int u = 0; u < kColUnroll; u++)
#pragma unroll
        for (int s = 0; s < NSET; s++) {
            if (s >= nsets) continue;
            acc[s][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(yv[u][s], xv[u].x, acc[s][0], 0, 0, 0);
            acc[s][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(yv[u][s], xv[u].y, acc[s][1], 0, 0, 0);
            acc[s][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(yv[u][s], xv[u].z, acc[s][2], 0, 0, 0);
            acc[s][3] = __builtin_amdgcn_mfma_f32_16x16x4f32(yv[u][s], xv[u].w, acc[s][3], 0, 0, 0);
        }
}

template <int NSET>
__global__ __launch_bounds__(kColWaves * 64) void thin_colwise_mfma_kernel(ColBatch b, float* __restrict__ scratch) {
    int pi = 0;
#pragma unroll
    for (int i = 1; i < FT_THIN_MAX_BATCH; i++)
        if (i < b.count && (int)blockIdx.x >= b.p[i].tile_begin) pi = i;
    const ColProblem& p = b.p[pi];
    const int wg_begin = blockIdx.y * b.rows_per_wg;
    if (wg_begin >= p.M) return;   // uniform: this problem has fewer slices than the grid
    __shared__ float red[kColWaves - 1][NSET * 16][kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int j = lane % 16, kq = lane / 16;
    const int n = ((int)blockIdx.x - p.tile_begin) * 64 + 4 * j;
    const bool live = n < p.R;   // R is a multiple of 4 (checked on the host)
    const int wg_end = wg_begin + b.rows_per_wg < p.M ? wg_begin + b.rows_per_wg : p.M;
    const int m_begin = wg_begin + wave * b.rows_per_wave;
    const int m_end = m_begin + b.rows_per_wave < wg_end ? m_begin + b.rows_per_wave : wg_end;
    // Where this lane's A operand (a factor column) of every set comes from.
    const float* yp[NSET];
#pragma unroll
    for (int s = 0; s < NSET; s++) {
        const int v = 16 * s + j;
        const int yi = v / p.C, c = v % p.C;
        const float* base = yi == 0 ? p.y[0] : (yi == 1 ? p.y[1] : p.y[2]);
        yp[s] = yi < p.ny ? base + c : nullptr;
    }
    // Sets this problem fills (wave-uniform): a launch is compiled for the largest of its batch.
    const int nsets = (p.ny * p.C + 15) / 16;
    thin_f4 acc[NSET][4];
#pragma unroll
    for (int s = 0; s < NSET; s++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[s][e] = thin_f4{0.f, 0.f, 0.f, 0.f};
    const float* xp = p.x + n;
    // (Requesting the next batch of loads before multiplying the current one was measured: no gain.)
    float4 xa[kColUnroll];
    float ya[kColUnroll][NSET];
    for (int m0 = m_begin; m0 < m_end; m0 += 4 * kColUnroll) {
        col_load<NSET>(xp, p.ldx, yp, p.ldy, nsets, m0, m_end, kq, live, xa, ya);
        col_mfma<NSET>(acc, nsets, xa, ya);
    }
    // acc[s][e][r] = sum over this wave's rows for virtual column 16s + 4kq + r, X column n + e
    if (wave > 0) {
#pragma unroll
        for (int s = 0; s < NSET; s++)
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) red[wave - 1][(s * 4 + e) * 4 + r][lane] = acc[s][e][r];
    }
    __syncthreads();
    if (wave == 0 && live) {
        const int VC = p.ny * p.C;
        float* dst = scratch + p.scratch_offset + ((long)blockIdx.y * p.R + n) * VC;
#pragma unroll
        for (int s = 0; s < NSET; s++) {
            const int v = 16 * s + 4 * kq;
            if (v >= VC) continue;   // VC is a multiple of 4: a quad of virtual columns is all in or all out
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float t = acc[s][e][r];
#pragma unroll
                    for (int w = 0; w < kColWaves - 1; w++) t += red[w][(s * 4 + e) * 4 + r][lane];
                    o[r] = t;
                }
                *reinterpret_cast<float4*>(dst + (long)e * VC + v) = make_float4(o[0], o[1], o[2], o[3]);
            }
        }
    }
}

// out_i[n][c] (or out_i[c][n] when transposed) = scale * sum over slices, in slice order.
__global__ __launch_bounds__(256) void thin_colwise_finish_kernel(ColBatch b, const float* __restrict__ scratch) {
    const ColProblem& p = b.p[blockIdx.y];
    const int e = blockIdx.x * 256 + threadIdx.x;
    const int VC = p.ny * p.C;
    const int total = p.R * VC;
    if (e >= total) return;
    const float* src = scratch + p.scratch_offset + e;
    float v = 0.0f;
    int s = 0;
    for (; s + 8 <= p.slices; s += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = src[(long)(s + u) * total];
#pragma unroll
        for (int u = 0; u < 8; u++) v += t[u];
    }
    for (; s < p.slices; s++) v += src[(long)s * total];
    const int n = e / VC, vc = e % VC;
    const int yi = vc / p.C, c = vc % p.C;
    float* out = yi == 0 ? p.out[0] : (yi == 1 ? p.out[1] : p.out[2]);
    float* o = p.out_transposed ? out + (long)c * p.ldo + n : out + (long)n * p.ldo + c;
    *o = p.accumulate ? *o + v * p.scale : v * p.scale;
}

bool aligned16(const void* q) { return (((uintptr_t)q) & 15) == 0; }

constexpr size_t kScratchFloats = (size_t)8 << 20;  // 32 MiB of partial sums

int ensure_scratch(ft_context* ctx) {
    if (ctx->thin_scratch) return FT_OK;
    FT_HIP(hipSetDevice(ctx->device));
    FT_HIP(hipMalloc((void**)&ctx->thin_scratch, kScratchFloats * sizeof(float)));
    return FT_OK;
}

}  // namespace

bool ft_thin_rank_supported(size_t r) { return r == 4 || r == 8 || r == 16; }

bool ft_thin_rowwise_ok(const ft_thin_problem& p) {
    return ft_thin_rank_supported((size_t)p.C) && p.K % 4 == 0 && p.ldx % 4 == 0 && aligned16(p.x) && aligned16(p.y) &&
           (!p.y_transposed || p.ldy % 4 == 0) && (p.y_transposed || p.ldy == p.C);
}

bool ft_thin_colwise_ok(const ft_thin_problem& p) {
    return ft_thin_rank_supported((size_t)p.C) && p.R % 4 == 0 && p.ldx % 4 == 0 && aligned16(p.x);
}

int ft_thin_rowwise(ft_context* ctx, const ft_thin_problem* probs, int count) {
    FT_CHECK_ARG(ctx && probs && count >= 1 && count <= FT_THIN_MAX_BATCH, "thin rowwise: bad batch");
    ThinBatch b{};
    b.count = count;
    int mmax = 0;
    double bytes = 0.0;
    for (int i = 0; i < count; i++) {
        const ft_thin_problem& p = probs[i];
        FT_CHECK_ARG(ft_thin_rowwise_ok(p), "thin rowwise: problem %d is not aligned for the vector kernel", i);
        FT_CHECK_ARG(p.C == probs[0].C && p.y_transposed == probs[0].y_transposed,
                     "thin rowwise: a batch must share rank and orientation");
        b.p[i] = p;
        if (p.M > mmax) mmax = p.M;
        bytes += 4.0 * ((double)p.M * p.K + (double)p.K * p.C + (double)p.M * p.C);
    }
    if (mmax == 0) return FT_OK;
    const dim3 grid(ft_div_up(mmax, 16), (unsigned)count);
    ft_prof_scope prof(ctx, probs[0].y_transposed ? "thin_rowwise_kernel<YT>" : "thin_rowwise_kernel", 0.0, bytes);
#define FT_ROW(CC)                                                                                              \
    do {                                                                                                        \
        if (probs[0].y_transposed)                                                                              \
            hipLaunchKernelGGL((thin_rowwise_kernel<CC, true>), grid, dim3(kRowWaves * 64), 0, ctx->stream, b); \
        else                                                                                                    \
            hipLaunchKernelGGL((thin_rowwise_kernel<CC, false>), grid, dim3(kRowWaves * 64), 0, ctx->stream, b); \
    } while (0)
    if (probs[0].C == 4) FT_ROW(4);
    else if (probs[0].C == 8) FT_ROW(8);
    else FT_ROW(16);
#undef FT_ROW
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_thin_colwise(ft_context* ctx, const ft_thin_problem* probs, int count) {
    FT_CHECK_ARG(ctx && probs && count >= 1 && count <= FT_THIN_MAX_BATCH, "thin colwise: bad batch");
    FT_TRY(ensure_scratch(ctx));
    ColBatch b{};
    int mmax = 0, vcmax = 0;
    double bytes = 0.0;
    for (int i = 0; i < count; i++) {
        const ft_thin_problem& q = probs[i];
        FT_CHECK_ARG(ft_thin_colwise_ok(q), "thin colwise: problem %d is not aligned for the vector kernel", i);
        FT_CHECK_ARG(q.C == probs[0].C, "thin colwise: a batch must share the rank");
        if (q.R == 0) continue;   // an empty result; M == 0 gives zero slices: the finish kernel writes zeros
        // Products that contract the same X (same rows, width and layout) share one problem.
        int at = -1;
        for (int k = 0; k < b.count && at < 0; k++) {
            const ColProblem& c = b.p[k];
            if (c.x == q.x && c.M == q.M && c.R == q.R && c.ldx == q.ldx && c.ldy == q.ldy && c.ldo == q.ldo &&
                c.scale == q.scale && c.out_transposed == q.out_transposed && c.accumulate == q.accumulate &&
                c.ny < 3)
                at = k;
        }
        if (at < 0) {
            at = b.count++;
            ColProblem& c = b.p[at];
            c.x = q.x;
            c.M = q.M, c.R = q.R, c.C = q.C, c.ny = 0;
            c.ldx = q.ldx, c.ldy = q.ldy, c.ldo = q.ldo;
            c.scale = q.scale;
            c.out_transposed = q.out_transposed, c.accumulate = q.accumulate;
            bytes += 4.0 * (double)q.M * q.R;
        }
        ColProblem& c = b.p[at];
        c.y[c.ny] = q.y;
        c.out[c.ny] = q.out;
        c.ny++;
        bytes += 4.0 * ((double)q.M * q.C + (double)q.R * q.C);
        if (q.M > mmax) mmax = q.M;
        if (c.ny * c.C > vcmax) vcmax = c.ny * c.C;
    }
    if (b.count == 0) return FT_OK;
    int tiles = 0;
    for (int i = 0; i < b.count; i++) {
        b.p[i].tile_begin = tiles;
        tiles += (b.p[i].R + 63) / 64;
    }
    // Rows per workgroup: enough workgroups to put several on every CU, few enough slices that the
    // partial tiles stay a few percent of the input traffic; whole batches of loads per wave.
    const int quantum = 4 * kColUnroll * kColWaves;   // 128 rows: one batch of loads per wave
    const int want_wgs = 2 * ctx->num_cus;   // measured: 1x and 4x are both slower at the 360M shapes
    int slices = want_wgs / tiles;
    if (slices < 1) slices = 1;
    // rounded up to whole batches, so that the last slice is never a sliver of rows
    int rows_per_wg = ((mmax + slices - 1) / slices + quantum - 1) / quantum * quantum;
    if (rows_per_wg < quantum) rows_per_wg = quantum;
    b.rows_per_wg = rows_per_wg;
    b.rows_per_wave = rows_per_wg / kColWaves;
    size_t off = 0;
    int smax = 1;
    for (int i = 0; i < b.count; i++) {
        ColProblem& c = b.p[i];
        c.slices = (c.M + rows_per_wg - 1) / rows_per_wg;
        if (c.slices > smax) smax = c.slices;
        c.scratch_offset = (long)off;
        off += (size_t)c.slices * c.R * c.ny * c.C;
    }
    if (off > kScratchFloats) {
        // The partial tiles of the batch do not fit the buffer: one product at a time (launches of one
        // stream run in order, so they may share it).
        FT_CHECK_ARG(count > 1, "thin colwise: %zu partial sums of one product exceed the scratch buffer", off);
        for (int i = 0; i < count; i++) FT_TRY(ft_thin_colwise(ctx, probs + i, 1));
        return FT_OK;
    }
    const int nset = (vcmax + 15) / 16;
    const dim3 grid((unsigned)tiles, (unsigned)smax);
    size_t fmax = 0;
    for (int i = 0; i < b.count; i++) {
        const size_t t = (size_t)b.p[i].R * b.p[i].ny * b.p[i].C;
        if (t > fmax) fmax = t;
    }
    const dim3 fgrid(ft_div_up(fmax, 256), (unsigned)b.count);
    ft_prof_scope prof(ctx, "thin_colwise+finish", 0.0, bytes);
    if (nset == 1)
        hipLaunchKernelGGL((thin_colwise_mfma_kernel<1>), grid, dim3(kColWaves * 64), 0, ctx->stream, b,
                           ctx->thin_scratch);
    else if (nset == 2)
        hipLaunchKernelGGL((thin_colwise_mfma_kernel<2>), grid, dim3(kColWaves * 64), 0, ctx->stream, b,
                           ctx->thin_scratch);
    else
        hipLaunchKernelGGL((thin_colwise_mfma_kernel<3>), grid, dim3(kColWaves * 64), 0, ctx->stream, b,
                           ctx->thin_scratch);
    FT_LAUNCH_CHECK();
    hipLaunchKernelGGL(thin_colwise_finish_kernel, fgrid, dim3(256), 0, ctx->stream, b, ctx->thin_scratch);
    FT_LAUNCH_CHECK();
    return FT_OK;
}
