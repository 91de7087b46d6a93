// The rank-r products around a LoRA linear (r = 4, 8 or 16): bandwidth-bound
// work with almost no flops, so they run on the vector ALUs with fully
// coalesced loads, and several independent products go into one launch.
//
//   row-wise   out[M, C] = scale * X[M, K] @ Y        (x@A,  dT = dY@B^T)
//              16 rows per workgroup, K split over its 4 waves, 16x16x4 MFMA
//              (the matrix unit does the K reduction, no cross-lane shuffles).
//   col-wise   out[R, C] = X[M, R]^T @ Y[M, C]        (dA = x^T@dT, dB = T^T@dY)
//              each thread owns 4 columns of X, the M rows are cut into
//              slices; a second kernel adds the slices in order (deterministic,
//              no atomics).
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

constexpr int kRowWaves = 8;

template <int C, bool YT>
__global__ __launch_bounds__(kRowWaves * 64) void thin_rowwise_kernel(ThinBatch b) {
    const ft_thin_problem& p = b.p[blockIdx.y];
    const int row0 = blockIdx.x * 16;
    if (row0 >= p.M) return;
    __shared__ float red[kRowWaves][16][17];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int li = lane % 16, q = lane / 16;
    const int row = row0 + li < p.M ? row0 + li : p.M - 1;  // clamped rows are computed and dropped
    const float* xr = p.x + (long)row * p.ldx + 4 * q;
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
            xa[u] = in ? *reinterpret_cast<const float4*>(xr + k0 + 16 * u) : make_float4(0.f, 0.f, 0.f, 0.f);
            if constexpr (YT) {
                const float4 t = (in && col_live) ? *reinterpret_cast<const float4*>(p.y + (long)li * p.ldy + k)
                                                  : make_float4(0.f, 0.f, 0.f, 0.f);
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
// grid (ceil(Rmax / 256), count, slices); 256 threads = 4 waves. Every thread owns
// 4 columns of X (a wave 256 of them); the rows of a slice are dealt to the four
// waves in contiguous quarters and the four partial results are added in wave
// order through LDS. partial[((slice * R) + n) * C + j] at p.scratch_offset.
template <int C>
__global__ __launch_bounds__(256) void thin_colwise_kernel(ThinBatch b, float* __restrict__ scratch, int slices) {
    const ft_thin_problem& p = b.p[blockIdx.y];
    if ((int)blockIdx.x * 256 >= p.R) return;  // whole workgroup past this problem's width
    __shared__ float red[3][4 * C][kWave + 1];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int n = (blockIdx.x * 64 + lane) * 4;
    const bool live = n < p.R;  // R is a multiple of 4 (checked on the host)
    const int per = (p.M + slices - 1) / slices;
    const int s_begin = blockIdx.z * per;
    const int s_end = s_begin + per < p.M ? s_begin + per : p.M;
    const int quarter = (per + 3) / 4;
    const int m_begin = s_begin + wave * quarter;
    const int m_end = m_begin + quarter < s_end ? m_begin + quarter : s_end;
    float acc[4][C];
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
        for (int j = 0; j < C; j++) acc[e][j] = 0.0f;
    if (live) {
        const float* xp = p.x + n;
#pragma unroll 8
        for (int m = m_begin; m < m_end; m++) {
            const float4 xv = *reinterpret_cast<const float4*>(xp + (long)m * p.ldx);
            const float* yr = p.y + (long)m * p.ldy;  // uniform across the wave
#pragma unroll
            for (int j = 0; j < C; j++) {
                const float yv = yr[j];
                acc[0][j] += xv.x * yv;
                acc[1][j] += xv.y * yv;
                acc[2][j] += xv.z * yv;
                acc[3][j] += xv.w * yv;
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < C; j++) red[wave - 1][e * C + j][lane] = acc[e][j];
    }
    __syncthreads();
    if (wave == 0 && live) {
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < C; j++)
                acc[e][j] = ((acc[e][j] + red[0][e * C + j][lane]) + red[1][e * C + j][lane]) + red[2][e * C + j][lane];
        float* dst = scratch + p.scratch_offset + ((long)blockIdx.z * p.R + n) * C;
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < C; j += 4)
                *reinterpret_cast<float4*>(dst + e * C + j) =
                    make_float4(acc[e][j], acc[e][j + 1], acc[e][j + 2], acc[e][j + 3]);
    }
}

// out[n][j] (or out[j][n] when transposed) = scale * sum over slices, in slice order.
__global__ __launch_bounds__(256) void thin_finish_kernel(ThinBatch b, const float* __restrict__ scratch, int slices) {
    const ft_thin_problem& p = b.p[blockIdx.y];
    const int e = blockIdx.x * 256 + threadIdx.x;
    const int total = p.R * p.C;
    if (e >= total) return;
    const float* src = scratch + p.scratch_offset + e;
    float v = 0.0f;
    int s = 0;
    for (; s + 8 <= slices; s += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = src[(long)(s + u) * total];
#pragma unroll
        for (int u = 0; u < 8; u++) v += t[u];
    }
    for (; s < slices; s++) v += src[(long)s * total];
    const int n = e / p.C, j = e % p.C;
    float* o = p.out_transposed ? p.out + (long)j * p.ldo + n : p.out + (long)n * p.ldo + j;
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
    // The partial-sum buffer is shared: a call on the main stream must not overtake one on the side stream.
    if (ctx->side_active < 0) FT_TRY(ft_side_join(ctx, 0));
    ThinBatch b{};
    b.count = count;
    int rmax = 0, mmax = 0;
    double bytes = 0.0;
    for (int i = 0; i < count; i++) {
        FT_CHECK_ARG(ft_thin_colwise_ok(probs[i]), "thin colwise: problem %d is not aligned for the vector kernel", i);
        FT_CHECK_ARG(probs[i].C == probs[0].C, "thin colwise: a batch must share the rank");
        if (probs[i].R > rmax) rmax = probs[i].R;
        if (probs[i].M > mmax) mmax = probs[i].M;
    }
    if (rmax == 0) return FT_OK;
    // Rows per slice: enough slices to fill the chip, few enough that the
    // partial sums stay a fraction of the input traffic.
    int slices = mmax / 128;
    if (slices > 16) slices = 16;
    if (slices < 1) slices = 1;
    // A batch whose partial sums do not fit the scratch buffer goes out in pieces (the launches of
    // one stream run in order, so the pieces may share the buffer).
    {
        size_t need = 0;
        int fit = 0;
        while (fit < count && need + (size_t)slices * probs[fit].R * probs[fit].C <= kScratchFloats) {
            need += (size_t)slices * probs[fit].R * probs[fit].C;
            fit++;
        }
        FT_CHECK_ARG(fit >= 1, "thin colwise: %zu partial sums of one product exceed the scratch buffer",
                     (size_t)slices * probs[0].R * probs[0].C);
        if (fit < count) {
            FT_TRY(ft_thin_colwise(ctx, probs, fit));
            return ft_thin_colwise(ctx, probs + fit, count - fit);
        }
    }
    size_t off = 0;
    for (int i = 0; i < count; i++) {
        b.p[i] = probs[i];
        b.p[i].scratch_offset = (long)off;
        off += (size_t)slices * probs[i].R * probs[i].C;
        bytes += 4.0 * ((double)probs[i].M * probs[i].R + (double)probs[i].M * probs[i].C +
                        (double)probs[i].R * probs[i].C);
    }
    FT_CHECK_ARG(off <= kScratchFloats, "thin colwise: %zu partial sums exceed the scratch buffer", off);
    const dim3 grid(ft_div_up(rmax, 256), (unsigned)count, (unsigned)slices);
    const dim3 fgrid(ft_div_up((size_t)rmax * probs[0].C, 256), (unsigned)count);
    ft_prof_scope prof(ctx, "thin_colwise+finish", 0.0, bytes);
    if (probs[0].C == 4)
        hipLaunchKernelGGL((thin_colwise_kernel<4>), grid, dim3(256), 0, ctx->stream, b, ctx->thin_scratch, slices);
    else if (probs[0].C == 8)
        hipLaunchKernelGGL((thin_colwise_kernel<8>), grid, dim3(256), 0, ctx->stream, b, ctx->thin_scratch, slices);
    else
        hipLaunchKernelGGL((thin_colwise_kernel<16>), grid, dim3(256), 0, ctx->stream, b, ctx->thin_scratch, slices);
    FT_LAUNCH_CHECK();
    hipLaunchKernelGGL(thin_finish_kernel, fgrid, dim3(256), 0, ctx->stream, b, ctx->thin_scratch, slices);
    FT_LAUNCH_CHECK();
    return FT_OK;
}
