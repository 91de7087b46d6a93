// The rank-r products around a LoRA linear (r = 4, 8 or 16): bandwidth-bound
// work with almost no flops, so they run on the vector ALUs with fully
// coalesced loads, and several independent products go into one launch.
//
//   row-wise   out[M, C] = scale * X[M, K] @ Y        (x@A,  dT = dY@B^T)
//              two rows per wave, lanes stride over K, butterfly reduction.
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
// grid (ceil(M / 8), count); 256 threads = 4 waves x 2 rows.
template <int C, bool YT>
__global__ __launch_bounds__(256) void thin_rowwise_kernel(ThinBatch b) {
    const ft_thin_problem& p = b.p[blockIdx.y];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int row0 = (blockIdx.x * 4 + wave) * 2;
    if (row0 >= p.M) return;  // wave-uniform
    const bool two = row0 + 1 < p.M;
    const float* x0 = p.x + (long)row0 * p.ldx;
    const float* x1 = p.x + (long)(two ? row0 + 1 : row0) * p.ldx;
    float acc0[C], acc1[C];
#pragma unroll
    for (int j = 0; j < C; j++) acc0[j] = acc1[j] = 0.0f;

    const int K4 = p.K / 4;  // K is a multiple of 4 (checked on the host)
    for (int q = lane; q < K4; q += kWave) {
        const int k = q * 4;
        const float4 a0 = *reinterpret_cast<const float4*>(x0 + k);
        const float4 a1 = *reinterpret_cast<const float4*>(x1 + k);
        if constexpr (!YT) {
            // Y[k..k+3][0..C-1] is one contiguous run of 4*C floats.
            const float4* y4 = reinterpret_cast<const float4*>(p.y + (long)k * C);
            float yv[4 * C];
#pragma unroll
            for (int e = 0; e < C; e++) {
                const float4 t = y4[e];
                yv[4 * e + 0] = t.x;
                yv[4 * e + 1] = t.y;
                yv[4 * e + 2] = t.z;
                yv[4 * e + 3] = t.w;
            }
#pragma unroll
            for (int j = 0; j < C; j++) {
                acc0[j] += a0.x * yv[j] + a0.y * yv[C + j] + a0.z * yv[2 * C + j] + a0.w * yv[3 * C + j];
                acc1[j] += a1.x * yv[j] + a1.y * yv[C + j] + a1.z * yv[2 * C + j] + a1.w * yv[3 * C + j];
            }
        } else {
            // Y is stored [C, K]: row j holds the k run.
#pragma unroll
            for (int j = 0; j < C; j++) {
                const float4 t = *reinterpret_cast<const float4*>(p.y + (long)j * p.ldy + k);
                acc0[j] += a0.x * t.x + a0.y * t.y + a0.z * t.z + a0.w * t.w;
                acc1[j] += a1.x * t.x + a1.y * t.y + a1.z * t.z + a1.w * t.w;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < C; j++) {
#pragma unroll
        for (int o = kWave / 2; o > 0; o >>= 1) {
            acc0[j] += __shfl_xor(acc0[j], o, kWave);
            acc1[j] += __shfl_xor(acc1[j], o, kWave);
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int j = 0; j < C; j++) {
            p.out[(long)row0 * p.ldo + j] = acc0[j] * p.scale;
            if (two) p.out[(long)(row0 + 1) * p.ldo + j] = acc1[j] * p.scale;
        }
    }
}

// ---- col-wise ---------------------------------------------------------------
// grid (ceil(Rmax / 256), count, slices); 64 threads, each owning 4 columns.
// partial[((slice * R) + n) * C + j] at p.scratch_offset.
template <int C>
__global__ __launch_bounds__(64) void thin_colwise_kernel(ThinBatch b, float* __restrict__ scratch, int slices) {
    const ft_thin_problem& p = b.p[blockIdx.y];
    const int n = (blockIdx.x * 64 + threadIdx.x) * 4;
    if (blockIdx.x * 256 >= p.R) return;  // whole workgroup past this problem's width
    const bool live = n < p.R;            // R is a multiple of 4 (checked on the host)
    const int per = (p.M + slices - 1) / slices;
    const int m_begin = blockIdx.z * per;
    const int m_end = m_begin + per < p.M ? m_begin + per : p.M;
    float acc[4][C];
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
        for (int j = 0; j < C; j++) acc[e][j] = 0.0f;
    if (live) {
        const float* xp = p.x + n;
#pragma unroll 4
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
    for (int s = 0; s < slices; s++) v += src[(long)s * total];
    const int n = e / p.C, j = e % p.C;
    if (p.out_transposed)
        p.out[(long)j * p.ldo + n] = v * p.scale;
    else
        p.out[(long)n * p.ldo + j] = v * p.scale;
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
    const dim3 grid(ft_div_up(mmax, 8), (unsigned)count);
    ft_prof_scope prof(ctx, probs[0].y_transposed ? "thin_rowwise_kernel<YT>" : "thin_rowwise_kernel", 0.0, bytes);
#define FT_ROW(CC)                                                                                              \
    do {                                                                                                        \
        if (probs[0].y_transposed)                                                                              \
            hipLaunchKernelGGL((thin_rowwise_kernel<CC, true>), grid, dim3(256), 0, ctx->stream, b);           \
        else                                                                                                    \
            hipLaunchKernelGGL((thin_rowwise_kernel<CC, false>), grid, dim3(256), 0, ctx->stream, b);          \
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
    int slices = mmax / 64;
    if (slices > 32) slices = 32;
    if (slices < 1) slices = 1;
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
        hipLaunchKernelGGL((thin_colwise_kernel<4>), grid, dim3(64), 0, ctx->stream, b, ctx->thin_scratch, slices);
    else if (probs[0].C == 8)
        hipLaunchKernelGGL((thin_colwise_kernel<8>), grid, dim3(64), 0, ctx->stream, b, ctx->thin_scratch, slices);
    else
        hipLaunchKernelGGL((thin_colwise_kernel<16>), grid, dim3(64), 0, ctx->stream, b, ctx->thin_scratch, slices);
    FT_LAUNCH_CHECK();
    hipLaunchKernelGGL(thin_finish_kernel, fgrid, dim3(256), 0, ctx->stream, b, ctx->thin_scratch, slices);
    FT_LAUNCH_CHECK();
    return FT_OK;
}
