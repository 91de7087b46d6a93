// Bandwidth-bound kernels of the LoRA step for gfx950: RMSNorm forward and
// backward, RoPE, SiLU-gate, adds and scales, masked softmax-cross-entropy,
// gradient-norm partials, AdamW, embedding gather. Each is written to touch
// every array once (float4 accesses, one row or chunk per workgroup, 64-lane
// wave reductions), so HBM traffic equals the algorithmic byte count.
#include "ft_common.h"

#include <algorithm>

#include <atomic>
#include <mutex>

namespace {

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Block-wide sum / max over NT threads (NT a multiple of 64, <= 1024). Every
// thread gets the result. `red` holds NT/64 floats.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x / kWave, l = threadIdx.x % kWave;
    __syncthreads();
    if (l == 0) red[w] = v;
    __syncthreads();
    float t = (l < NT / kWave) ? red[l] : 0.0f;
    return wave_sum(t);
}
template <int NT>
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int w = threadIdx.x / kWave, l = threadIdx.x % kWave;
    __syncthreads();
    if (l == 0) red[w] = v;
    __syncthreads();
    float t = (l < NT / kWave) ? red[l] : -3.4e38f;
    return wave_max(t);
}

__host__ __device__ inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// ---------------------------------------------------------------------------
// Elementwise
// ---------------------------------------------------------------------------

enum class Ew { Add, AddBackward, SiluGate, SiluGateBackward, Scale, Accumulate, Zero };

struct EwArgs {
    const float* a;
    const float* b;
    const float* c;
    float* o0;
    float* o1;
    size_t n;
    float s;
};

template <Ew OP>
__device__ __forceinline__ void ew_apply(const EwArgs& p, size_t i) {
    if constexpr (OP == Ew::Add) {
        p.o0[i] = p.a[i] + p.b[i];
    } else if constexpr (OP == Ew::AddBackward) {
        const float g = p.a[i];
        p.o0[i] = g;
        p.o1[i] = g;
    } else if constexpr (OP == Ew::SiluGate) {
        const float x = p.a[i];
        const float silu = x * (1.0f / (1.0f + __expf(-x)));
        p.o0[i] = silu * p.b[i];
    } else if constexpr (OP == Ew::SiluGateBackward) {
        const float x = p.a[i], y = p.b[i], g = p.c[i];
        const float s = 1.0f / (1.0f + __expf(-x));
        p.o1[i] = g * (x * s);
        p.o0[i] = g * y * (s * (1.0f + x * (1.0f - s)));
    } else if constexpr (OP == Ew::Scale) {
        p.o0[i] = p.o0[i] * p.s;
    } else if constexpr (OP == Ew::Accumulate) {
        p.o0[i] = p.o0[i] + p.a[i];
    } else {
        p.o0[i] = 0.0f;
    }
}

template <Ew OP>
__device__ __forceinline__ void ew_apply4(const EwArgs& p, size_t i4) {
    const float4* a = reinterpret_cast<const float4*>(p.a);
    const float4* b = reinterpret_cast<const float4*>(p.b);
    const float4* c = reinterpret_cast<const float4*>(p.c);
    float4* o0 = reinterpret_cast<float4*>(p.o0);
    float4* o1 = reinterpret_cast<float4*>(p.o1);
    if constexpr (OP == Ew::Add) {
        const float4 x = a[i4], y = b[i4];
        o0[i4] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    } else if constexpr (OP == Ew::AddBackward) {
        const float4 g = a[i4];
        o0[i4] = g;
        o1[i4] = g;
    } else if constexpr (OP == Ew::SiluGate) {
        const float4 x = a[i4], y = b[i4];
        float4 r;
        r.x = x.x * (1.0f / (1.0f + __expf(-x.x))) * y.x;
        r.y = x.y * (1.0f / (1.0f + __expf(-x.y))) * y.y;
        r.z = x.z * (1.0f / (1.0f + __expf(-x.z))) * y.z;
        r.w = x.w * (1.0f / (1.0f + __expf(-x.w))) * y.w;
        o0[i4] = r;
    } else if constexpr (OP == Ew::SiluGateBackward) {
        const float4 x = a[i4], y = b[i4], g = c[i4];
        float4 ga, gb;
#define FT_SGB(f)                                              \
    {                                                          \
        const float s = 1.0f / (1.0f + __expf(-x.f));          \
        gb.f = g.f * (x.f * s);                                \
        ga.f = g.f * y.f * (s * (1.0f + x.f * (1.0f - s)));    \
    }
        FT_SGB(x) FT_SGB(y) FT_SGB(z) FT_SGB(w)
#undef FT_SGB
        o0[i4] = ga;
        o1[i4] = gb;
    } else if constexpr (OP == Ew::Scale) {
        float4 x = o0[i4];
        x.x *= p.s; x.y *= p.s; x.z *= p.s; x.w *= p.s;
        o0[i4] = x;
    } else if constexpr (OP == Ew::Accumulate) {
        float4 x = o0[i4];
        const float4 y = a[i4];
        x.x += y.x; x.y += y.y; x.z += y.z; x.w += y.w;
        o0[i4] = x;
    } else {
        o0[i4] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

template <Ew OP, bool VEC>
__global__ __launch_bounds__(256) void ew_kernel(EwArgs p) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC) {
        const size_t n4 = p.n / 4;
        for (; i < n4; i += stride) ew_apply4<OP>(p, i);
        // tail (n % 4 elements) by the first threads
        const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (t < p.n - n4 * 4) ew_apply<OP>(p, n4 * 4 + t);
    } else {
        for (; i < p.n; i += stride) ew_apply<OP>(p, i);
    }
}

template <Ew OP>
int ew_launch(ft_context* ctx, EwArgs p) {
    if (p.n == 0) return FT_OK;
    const bool vec = aligned16(p.a) && aligned16(p.b) && aligned16(p.c) && aligned16(p.o0) && aligned16(p.o1);
    const size_t work = vec ? (p.n + 3) / 4 : p.n;
    size_t blocks = (work + 255) / 256;
    const size_t cap = (size_t)ctx->num_cus * 16;
    if (blocks > cap) blocks = cap;
    static const char* const names[] = {"ew_kernel<Add>", "ew_kernel<AddBackward>", "ew_kernel<SiluGate>",
                                        "ew_kernel<SiluGateBackward>", "ew_kernel<Scale>", "ew_kernel<Accumulate>",
                                        "ew_kernel<Zero>"};
    static const double arrays[] = {3, 3, 3, 5, 2, 3, 1};
    ft_prof_scope prof(ctx, names[(int)OP], 0.0, 4.0 * arrays[(int)OP] * (double)p.n);
    if (vec)
        hipLaunchKernelGGL((ew_kernel<OP, true>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, p);
    else
        hipLaunchKernelGGL((ew_kernel<OP, false>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, p);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// ---------------------------------------------------------------------------
// Embedding gather: one wave per token row.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void embedding_kernel(const float* __restrict__ table, size_t vocab,
                                                        size_t hidden, const uint32_t* __restrict__ ids,
                                                        size_t n, float* __restrict__ out) {
    const size_t row = (size_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (row >= n) return;
    const int lane = threadIdx.x % kWave;
    const uint32_t id = ids[row];
    float* o = out + row * hidden;
    if ((size_t)id < vocab) {
        const float* src = table + (size_t)id * hidden;
        if ((hidden & 3) == 0 && aligned16(table) && aligned16(out)) {
            const float4* s4 = reinterpret_cast<const float4*>(src);
            float4* o4 = reinterpret_cast<float4*>(o);
            for (size_t i = lane; i < hidden / 4; i += kWave) o4[i] = s4[i];
        } else {
            for (size_t i = lane; i < hidden; i += kWave) o[i] = src[i];
        }
    } else {
        for (size_t i = lane; i < hidden; i += kWave) o[i] = 0.0f;
    }
}

// ---------------------------------------------------------------------------
// RMSNorm. One 256-thread workgroup per row; the second sweep over the row
// re-reads what the first sweep just pulled into cache.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void rms_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                       float* __restrict__ out, size_t rows, size_t size,
                                                       float eps, int vec) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float* xr = x + row * size;
    float* orow = out + row * size;
    float ss = 0.0f;
    if (vec) {
        const float4* x4 = reinterpret_cast<const float4*>(xr);
        for (size_t i = threadIdx.x; i < size / 4; i += 256) {
            const float4 v = x4[i];
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    } else {
        for (size_t i = threadIdx.x; i < size; i += 256) ss += xr[i] * xr[i];
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)size + eps);
    if (vec) {
        const float4* x4 = reinterpret_cast<const float4*>(xr);
        const float4* w4 = reinterpret_cast<const float4*>(w);
        float4* o4 = reinterpret_cast<float4*>(orow);
        for (size_t i = threadIdx.x; i < size / 4; i += 256) {
            const float4 v = x4[i], g = w4[i];
            o4[i] = make_float4(v.x * inv * g.x, v.y * inv * g.y, v.z * inv * g.z, v.w * inv * g.w);
        }
    } else {
        for (size_t i = threadIdx.x; i < size; i += 256) orow[i] = xr[i] * inv * w[i];
    }
}

// Backward for ROWS_PER_WG consecutive rows per workgroup. gx as in the
// reference; when gw_partial != nullptr each workgroup also writes its rows'
// contribution sum g*x*inv per feature to gw_partial[blockIdx.x * size + i].
template <int ROWS_PER_WG>
__global__ __launch_bounds__(256) void rms_norm_backward_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ g,
    float* __restrict__ gx, float* __restrict__ gw_partial, size_t rows, size_t size, float eps) {
    __shared__ float red[4];
    const size_t row0 = (size_t)blockIdx.x * ROWS_PER_WG;
    // Columns this thread owns: threadIdx.x + 256*j. Up to 8 partial sums stay
    // in registers; wider rows fall back to read-modify-write on the partial row.
    constexpr int MAXC = 8;
    float gwacc[MAXC];
#pragma unroll
    for (int j = 0; j < MAXC; j++) gwacc[j] = 0.0f;
    const bool wide = size > (size_t)256 * MAXC;
    if (gw_partial && wide)
        for (size_t i = threadIdx.x; i < size; i += 256) gw_partial[(size_t)blockIdx.x * size + i] = 0.0f;
    for (int rr = 0; rr < ROWS_PER_WG; rr++) {
        const size_t row = row0 + rr;
        if (row >= rows) break;  // uniform
        const float* xr = x + row * size;
        const float* gr = g + row * size;
        float ss = 0.0f, gwx = 0.0f;
        for (size_t i = threadIdx.x; i < size; i += 256) {
            const float xv = xr[i];
            ss += xv * xv;
            gwx += gr[i] * w[i] * xv;
        }
        ss = block_sum<256>(ss, red);
        gwx = block_sum<256>(gwx, red);
        const float inv = 1.0f / sqrtf(ss / (float)size + eps);
        const float coef = gwx * inv * inv * inv / (float)size;
        int j = 0;
        for (size_t i = threadIdx.x; i < size; i += 256, j++) {
            const float xv = xr[i], gv = gr[i];
            gx[row * size + i] = gv * w[i] * inv - xv * coef;
            if (gw_partial) {
                if (!wide) {
                    // j < MAXC by construction; the unrolled select keeps gwacc in registers.
#pragma unroll
                    for (int q = 0; q < MAXC; q++)
                        if (q == j) gwacc[q] += gv * xv * inv;
                } else {
                    gw_partial[(size_t)blockIdx.x * size + i] += gv * xv * inv;
                }
            }
        }
    }
    if (gw_partial && !wide) {
        int j = 0;
        for (size_t i = threadIdx.x; i < size; i += 256, j++) {
            float v = 0.0f;
#pragma unroll
            for (int q = 0; q < MAXC; q++)
                if (q == j) v = gwacc[q];
            gw_partial[(size_t)blockIdx.x * size + i] = v;
        }
    }
}

// gw[i] = sum over partial rows, in ascending order (deterministic).
__global__ __launch_bounds__(256) void column_sum_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                         size_t parts, size_t size) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= size) return;
    float acc = 0.0f;
    for (size_t p = 0; p < parts; p++) acc += partial[p * size + i];
    out[i] = acc;
}

// ---------------------------------------------------------------------------
// RMSNorm, one wave per row: the row (up to 64*4*NV floats) lives in registers
// between the reduction and the output, so every array is touched once and no
// workgroup barrier is needed. 4 rows per 256-thread workgroup.
// ---------------------------------------------------------------------------
// A lane's NV float4 of one row of a deferred split-K sum: (add +) share 0 + share 1 + ... in that
// order (the order of splitk_reduce_kernel). The loads of up to U shares are issued together, so a row
// costs splits / U memory round trips instead of one per share.
template <int NV>
__device__ __forceinline__ void sum_shares_row(const ft_deferred_sum& d, size_t row_off, int lane, int n4,
                                               float4 (&v)[NV]) {
    constexpr int U = NV <= 4 ? 4 : 2;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        v[j] = (d.add && i < n4) ? reinterpret_cast<const float4*>(d.add + row_off)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int s0 = 0; s0 < d.splits; s0 += U) {
        float4 t[U][NV];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int sc = s0 + u < d.splits ? s0 + u : d.splits - 1;  // a share past the end re-reads the last one
            const float4* src = reinterpret_cast<const float4*>(d.partial + (size_t)sc * d.stride + row_off);
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int i = lane + j * kWave;
                t[u][j] = src[i < n4 ? i : 0];
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (s0 + u < d.splits) {  // uniform
#pragma unroll
                for (int j = 0; j < NV; j++) {
                    v[j].x += t[u][j].x;
                    v[j].y += t[u][j].y;
                    v[j].z += t[u][j].z;
                    v[j].w += t[u][j].w;
                }
            }
        }
    }
}

// A lane's NV float4 of row `row` of a product whose last tiles are still K shares (tail split): elements
// of whole tiles come from d.out; an element of tail tile u is (add +) share 0 + share 1 + ... in that
// order (the order of the GEMM's own reduce kernel). is_tail[j] says which of the lane's float4 were
// summed here. A wave whose row block holds no tail tile issues no extra load. No load sits under a
// lane-dependent branch (the compiler waits for every earlier load in front of such a load: one round
// trip per load instead of one per batch): lanes outside the tail tiles read share addresses of tile 0
// and drop the values.
template <int NV>
__device__ __forceinline__ void sum_tail_row(const ft_deferred_sum& d, int row, int lane, int n4, float4 (&v)[NV],
                                             bool (&is_tail)[NV]) {
    constexpr int U = 4;
    const size_t row_off = (size_t)row * 4 * n4;
    const int tm = row >> 6;
    const int shares = 1 << d.tail_shift;
    const int last = (d.tiles_n - 1) / d.panel;
    const float* src[NV];
    bool any = false;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        const int ii = i < n4 ? i : 0;
        const int tn = ii >> 4;  // 16 float4 per 64-column tile
        const int pnl = tn / d.panel;
        const int width = pnl == last ? d.tiles_n - last * d.panel : d.panel;
        const int pos = pnl * d.tiles_m * d.panel + tm * width + (tn - pnl * d.panel);
        is_tail[j] = i < n4 && pos >= d.tail_first;
        any = any || is_tail[j];
        src[j] = d.partial + ((size_t)(is_tail[j] ? pos - d.tail_first : 0) << d.tail_shift) * 4096 + (row & 63) * 64 +
                 (ii & 15) * 4;
        const float* base = (is_tail[j] && d.add) ? d.add : d.out;
        const float4 t = reinterpret_cast<const float4*>(base + row_off)[ii];
        const bool zero = i >= n4 || (is_tail[j] && !d.add);
        v[j] = make_float4(zero ? 0.f : t.x, zero ? 0.f : t.y, zero ? 0.f : t.z, zero ? 0.f : t.w);
    }
    if (__ballot(any) == 0) return;  // wave-uniform
    // Four shares' loads at a time, in straight-line code (a share past the end re-reads the last one and
    // is not added); a tail tile has at most eight shares.
    auto batch = [&](int s0) {
        float4 t[U][NV];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int sc = s0 + u < shares ? s0 + u : shares - 1;
#pragma unroll
            for (int j = 0; j < NV; j++) t[u][j] = *reinterpret_cast<const float4*>(src[j] + (size_t)sc * 4096);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const bool take = is_tail[j] && s0 + u < shares;
                v[j].x = take ? v[j].x + t[u][j].x : v[j].x;
                v[j].y = take ? v[j].y + t[u][j].y : v[j].y;
                v[j].z = take ? v[j].z + t[u][j].z : v[j].z;
                v[j].w = take ? v[j].w + t[u][j].w : v[j].w;
            }
        }
    };
    batch(0);
    if (shares > U) batch(U);
}

// SUM: 0 = x is complete; 1 = x is the K shares of the GEMM that produced it; 2 = x is complete except for
// the tail tiles of that GEMM (ft_deferred_sum). In both deferred forms the summed elements are written to
// x_out (which is the product's output buffer).
template <int NV, int SUM = 0>
__global__ __launch_bounds__(256) void rms_norm_wave_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            float* __restrict__ out, int rows, int size, float eps,
                                                            ft_deferred_sum sum, float* __restrict__ x_out) {
    const int row = blockIdx.x * 4 + threadIdx.x / kWave;
    if (row >= rows) return;
    const int lane = threadIdx.x % kWave;
    const int n4 = size / 4;
    const float4* x4 = reinterpret_cast<const float4*>(x + (size_t)row * size);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    float4 v[NV], wv[NV];
    float ss = 0.0f;
    bool is_tail[NV];
    // Every load of the lane is issued before the first wait, none under a lane-dependent branch (a lane
    // past the row's end re-reads element 0 and drops it): one memory round trip for the row.
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        wv[j] = w4[i < n4 ? i : 0];
    }
    if constexpr (SUM == 1) {
        // x is still the K shares of the GEMM that produced it: added here (residual first, then share
        // after share) and written out once.
        sum_shares_row<NV>(sum, (size_t)row * size, lane, n4, v);
    } else if constexpr (SUM == 2) {
        sum_tail_row<NV>(sum, row, lane, n4, v, is_tail);
    } else {
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + j * kWave;
            v[j] = x4[i < n4 ? i : 0];
        }
    }
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        if constexpr (SUM == 1) {
            if (i < n4) reinterpret_cast<float4*>(x_out + (size_t)row * size)[i] = v[j];
        } else if constexpr (SUM == 2) {
            if (is_tail[j]) reinterpret_cast<float4*>(x_out + (size_t)row * size)[i] = v[j];
        }
        if (i >= n4) v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)size + eps);
    float4* o4 = reinterpret_cast<float4*>(out + (size_t)row * size);
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        if (i < n4) {
            const float4 g = wv[j];
            o4[i] = make_float4(v[j].x * inv * g.x, v[j].y * inv * g.y, v[j].z * inv * g.z, v[j].w * inv * g.w);
        }
    }
}

// gx = g*w*inv - x*coef (+ add): the input gradient of RMSNorm, optionally
// summed with the gradient arriving over the residual connection.
// SUM as in rms_norm_wave_kernel, for g (nothing is written back: this kernel is g's only reader).
template <int NV, int SUM = 0>
__global__ __launch_bounds__(256) void rms_norm_backward_wave_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ g, const float* add,
    float* gx, int rows, int size, float eps, ft_deferred_sum sum) {
    const int row = blockIdx.x * 4 + threadIdx.x / kWave;
    if (row >= rows) return;
    const int lane = threadIdx.x % kWave;
    const int n4 = size / 4;
    const float4* x4 = reinterpret_cast<const float4*>(x + (size_t)row * size);
    const float4* g4 = reinterpret_cast<const float4*>(g + (size_t)row * size);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    // (without a residual gradient the slot re-reads x and the value is dropped)
    const float4* a4 = add ? reinterpret_cast<const float4*>(add + (size_t)row * size) : x4;
    float4 xv[NV], gv[NV], wv[NV], av[NV];
    float ss = 0.0f, gwx = 0.0f;
    // Every load of the lane is issued before the first wait, none under a lane-dependent branch (a lane
    // past the row's end re-reads element 0 and drops it): one memory round trip for x, w, g and the
    // residual gradient together.
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        const int ii = i < n4 ? i : 0;
        xv[j] = x4[ii];
        wv[j] = w4[ii];
        av[j] = a4[ii];
        if constexpr (SUM == 0) gv[j] = g4[ii];
    }
    if constexpr (SUM == 1) sum_shares_row<NV>(sum, (size_t)row * size, lane, n4, gv);  // g arrives as K shares
    if constexpr (SUM == 2) {
        bool is_tail[NV];
        sum_tail_row<NV>(sum, row, lane, n4, gv, is_tail);
    }
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        if (i < n4) {
            gv[j] = make_float4(gv[j].x * wv[j].x, gv[j].y * wv[j].y, gv[j].z * wv[j].z, gv[j].w * wv[j].w);  // g*w
        } else {
            xv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            gv[j] = xv[j];
        }
        ss += xv[j].x * xv[j].x + xv[j].y * xv[j].y + xv[j].z * xv[j].z + xv[j].w * xv[j].w;
        gwx += gv[j].x * xv[j].x + gv[j].y * xv[j].y + gv[j].z * xv[j].z + gv[j].w * xv[j].w;
    }
    ss = wave_sum(ss);
    gwx = wave_sum(gwx);
    const float inv = 1.0f / sqrtf(ss / (float)size + eps);
    const float coef = gwx * inv * inv * inv / (float)size;
    float4* o4 = reinterpret_cast<float4*>(gx + (size_t)row * size);
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        if (i < n4) {
            float4 r = make_float4(gv[j].x * inv - xv[j].x * coef, gv[j].y * inv - xv[j].y * coef,
                                   gv[j].z * inv - xv[j].z * coef, gv[j].w * inv - xv[j].w * coef);
            if (add) r = make_float4(av[j].x + r.x, av[j].y + r.y, av[j].z + r.z, av[j].w + r.w);
            o4[i] = r;
        }
    }
}

// The same with the norm-weight gradient: waves stride over the rows, each lane
// adds g*x*inv of its columns in registers, the four waves of a workgroup are
// combined through LDS in wave order and the workgroup writes one partial row;
// column_sum_sliced_kernel adds the partial rows in a fixed order.
template <int NV>
__global__ __launch_bounds__(256) void rms_norm_backward_gw_wave_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ g, float* __restrict__ gx,
    float* __restrict__ gw_partial, int rows, int size, float eps) {
    extern __shared__ float4 gw_lds[];  // [3][size / 4]
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int n4 = size / 4;
    const float4* w4 = reinterpret_cast<const float4*>(w);
    float4 wv[NV], acc[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + j * kWave;
        wv[j] = i < n4 ? w4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
        const float4* x4 = reinterpret_cast<const float4*>(x + (size_t)row * size);
        const float4* g4 = reinterpret_cast<const float4*>(g + (size_t)row * size);
        float4 xv[NV], gv[NV];
        float ss = 0.0f, gwx = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + j * kWave;
            if (i < n4) {
                xv[j] = x4[i];
                gv[j] = g4[i];
            } else {
                xv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                gv[j] = xv[j];
            }
            ss += xv[j].x * xv[j].x + xv[j].y * xv[j].y + xv[j].z * xv[j].z + xv[j].w * xv[j].w;
            gwx += gv[j].x * wv[j].x * xv[j].x + gv[j].y * wv[j].y * xv[j].y + gv[j].z * wv[j].z * xv[j].z +
                   gv[j].w * wv[j].w * xv[j].w;
        }
        ss = wave_sum(ss);
        gwx = wave_sum(gwx);
        const float inv = 1.0f / sqrtf(ss / (float)size + eps);
        const float coef = gwx * inv * inv * inv / (float)size;
        float4* o4 = reinterpret_cast<float4*>(gx + (size_t)row * size);
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + j * kWave;
            if (i < n4)
                o4[i] = make_float4(gv[j].x * wv[j].x * inv - xv[j].x * coef, gv[j].y * wv[j].y * inv - xv[j].y * coef,
                                    gv[j].z * wv[j].z * inv - xv[j].z * coef, gv[j].w * wv[j].w * inv - xv[j].w * coef);
            acc[j].x += gv[j].x * xv[j].x * inv;
            acc[j].y += gv[j].y * xv[j].y * inv;
            acc[j].z += gv[j].z * xv[j].z * inv;
            acc[j].w += gv[j].w * xv[j].w * inv;
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + j * kWave;
            if (i < n4) gw_lds[(wave - 1) * n4 + i] = acc[j];
        }
    }
    __syncthreads();
    if (wave == 0) {
        float4* p4 = reinterpret_cast<float4*>(gw_partial + (size_t)blockIdx.x * size);
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + j * kWave;
            if (i < n4) {
                float4 s = acc[j];
                for (int k = 0; k < 3; k++) {
                    const float4 o = gw_lds[k * n4 + i];
                    s = make_float4(s.x + o.x, s.y + o.y, s.z + o.z, s.w + o.w);
                }
                p4[i] = s;
            }
        }
    }
}

// out[i] = sum of partial[p * size + i] over p: 16 columns per workgroup, the
// partial rows dealt to 16 slices that are added in slice order (deterministic).
__global__ __launch_bounds__(256) void column_sum_sliced_kernel(const float* __restrict__ partial,
                                                                float* __restrict__ out, int parts, int size) {
    __shared__ float red[16][16];
    const int c = threadIdx.x % 16, slice = threadIdx.x / 16;
    const int col = blockIdx.x * 16 + c;
    float acc = 0.0f;
    if (col < size) {
#pragma unroll 8
        for (int p = slice; p < parts; p += 16) acc += partial[(size_t)p * size + col];
    }
    red[slice][c] = acc;
    __syncthreads();
    if (slice == 0 && col < size) {
        float s = red[0][c];
#pragma unroll
        for (int k = 1; k < 16; k++) s += red[k][c];
        out[col] = s;
    }
}

// ---------------------------------------------------------------------------
// RoPE through a (cos, sin) table: the angles of a step depend only on
// (position, i), so they are computed once (exactly as rope_kernel computes
// them) and the rotation itself becomes a pure streaming pass. One launch
// rotates two tensors (q and k).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rope_table_kernel(float2* __restrict__ table, unsigned seq, unsigned head_dim,
                                                         unsigned pos0, float theta) {
    const unsigned half = head_dim / 2;
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= seq * half) return;
    const unsigned t = idx / half, i = idx % half;
    const float pos = (float)(pos0 + t);
    const float freq_exp = -2.0f * (float)i / (float)head_dim;
    const float angle = pos * powf(theta, freq_exp);
    float s, c;
    sincosf(angle, &s, &c);
    table[idx] = make_float2(c, s);
}

struct RopeJob {
    const float* src;
    float* dst;
    unsigned heads;      // head vectors per token
    size_t quads;        // tokens * heads * head_dim / 8 (4 pairs per thread)
};

__global__ __launch_bounds__(256) void rope_apply_kernel(RopeJob j0, RopeJob j1, const float2* __restrict__ table,
                                                         unsigned seq, unsigned head_dim, float dir) {
    const RopeJob& j = blockIdx.y == 0 ? j0 : j1;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= j.quads) return;
    const unsigned half = head_dim / 2, qpv = half / 4;   // quads per head vector
    const size_t vec = idx / qpv;
    const unsigned i = (unsigned)(idx % qpv) * 4;
    const unsigned t = (unsigned)((vec / j.heads) % seq);
    const float2* tb = table + (size_t)t * half + i;
    const float4 v1 = *reinterpret_cast<const float4*>(j.src + vec * head_dim + i);
    const float4 v2 = *reinterpret_cast<const float4*>(j.src + vec * head_dim + i + half);
    const float2 c0 = tb[0], c1 = tb[1], c2 = tb[2], c3 = tb[3];
    float4 o1, o2;
    o1.x = v1.x * c0.x - v2.x * (dir * c0.y);  o2.x = v1.x * (dir * c0.y) + v2.x * c0.x;
    o1.y = v1.y * c1.x - v2.y * (dir * c1.y);  o2.y = v1.y * (dir * c1.y) + v2.y * c1.x;
    o1.z = v1.z * c2.x - v2.z * (dir * c2.y);  o2.z = v1.z * (dir * c2.y) + v2.z * c2.x;
    o1.w = v1.w * c3.x - v2.w * (dir * c3.y);  o2.w = v1.w * (dir * c3.y) + v2.w * c3.x;
    *reinterpret_cast<float4*>(j.dst + vec * head_dim + i) = o1;
    *reinterpret_cast<float4*>(j.dst + vec * head_dim + i + half) = o2;
}

// ---------------------------------------------------------------------------
// RoPE (rotate-half). One thread per (token, head, i < head_dim/2) pair.
// Angles in f32 exactly as pos * powf(theta, -2i/head_dim), precise sin/cos.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void rope_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                   size_t pairs, unsigned head_dim, unsigned seq,
                                                   unsigned pos0, unsigned heads, float theta, float dir) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= pairs) return;
    const unsigned half = head_dim / 2;
    const size_t vec = idx / half;              // head-vector index
    const unsigned i = (unsigned)(idx % half);
    const float pos = (float)(pos0 + (unsigned)((vec / heads) % seq));
    const float freq_exp = -2.0f * (float)i / (float)head_dim;
    const float angle = dir * pos * powf(theta, freq_exp);
    float s, c;
    sincosf(angle, &s, &c);
    const size_t i1 = vec * head_dim + i, i2 = i1 + half;
    const float v1 = src[i1], v2 = src[i2];
    dst[i1] = v1 * c - v2 * s;
    dst[i2] = v1 * s + v2 * c;
}

// ---------------------------------------------------------------------------
// Masked softmax-cross-entropy. One 1024-thread workgroup per row. grad may
// alias logits (no __restrict__ on either), so the target logit is loaded
// before the barrier that precedes the gradient stores. A row of up
// to 1024*4*CACHE floats is held in registers between the reduction and the
// gradient write, so logits are read once and the gradient written once.
// ---------------------------------------------------------------------------

constexpr int kCeThreads = 1024;

template <int CACHE>  // float4 per thread kept in registers (0 = stream from memory)
__global__ __launch_bounds__(kCeThreads) void masked_ce_kernel(
    const float* logits, const uint32_t* __restrict__ targets, const float* __restrict__ weights,
    float* grad, float* __restrict__ row_loss, size_t rows, size_t vocab, float grad_scale) {
    __shared__ float red[kCeThreads / kWave];
    const size_t row = blockIdx.x;
    const float* x = logits + row * vocab;
    float* gr = grad + row * vocab;
    const uint32_t tgt = targets[row];
    const size_t n4 = vocab / 4;
    if (tgt == FT_MASKED_CE_SKIP) {
        float4* g4 = reinterpret_cast<float4*>(gr);
        for (size_t i = threadIdx.x; i < n4; i += kCeThreads) g4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (size_t i = n4 * 4 + threadIdx.x; i < vocab; i += kCeThreads) gr[i] = 0.0f;
        if (threadIdx.x == 0) row_loss[row] = 0.0f;
        return;
    }
    const float4* x4 = reinterpret_cast<const float4*>(x);
    float4 cache[CACHE > 0 ? CACHE : 1];
    float m = -3.4e38f;
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int j = 0; j < CACHE; j++) {
            const size_t i = threadIdx.x + (size_t)j * kCeThreads;
            if (i < n4) {
                cache[j] = x4[i];
                m = fmaxf(m, fmaxf(fmaxf(cache[j].x, cache[j].y), fmaxf(cache[j].z, cache[j].w)));
            }
        }
    } else {
        for (size_t i = threadIdx.x; i < n4; i += kCeThreads) {
            const float4 v = x4[i];
            m = fmaxf(m, fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)));
        }
    }
    for (size_t i = n4 * 4 + threadIdx.x; i < vocab; i += kCeThreads) m = fmaxf(m, x[i]);
    m = block_max<kCeThreads>(m, red);
    float se = 0.0f;
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int j = 0; j < CACHE; j++) {
            const size_t i = threadIdx.x + (size_t)j * kCeThreads;
            if (i < n4) se += expf(cache[j].x - m) + expf(cache[j].y - m) + expf(cache[j].z - m) + expf(cache[j].w - m);
        }
    } else {
        for (size_t i = threadIdx.x; i < n4; i += kCeThreads) {
            const float4 v = x4[i];
            se += expf(v.x - m) + expf(v.y - m) + expf(v.z - m) + expf(v.w - m);
        }
    }
    for (size_t i = n4 * 4 + threadIdx.x; i < vocab; i += kCeThreads) se += expf(x[i] - m);
    se = block_sum<kCeThreads>(se, red);
    const float log_z = m + logf(se);
    const float w = weights[row];
    // The target logit is read before any thread overwrites it (grad may alias logits).
    const float x_t = x[tgt];
    __syncthreads();
    float4* g4 = reinterpret_cast<float4*>(gr);
    auto one = [&](float xv, size_t i) {
        float gv = expf(xv - log_z) * w;
        if (i == (size_t)tgt) gv -= w;
        return gv * grad_scale;
    };
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int j = 0; j < CACHE; j++) {
            const size_t i = threadIdx.x + (size_t)j * kCeThreads;
            if (i < n4) {
                const float4 v = cache[j];
                g4[i] = make_float4(one(v.x, 4 * i), one(v.y, 4 * i + 1), one(v.z, 4 * i + 2), one(v.w, 4 * i + 3));
            }
        }
    } else {
        for (size_t i = threadIdx.x; i < n4; i += kCeThreads) {
            const float4 v = x4[i];
            g4[i] = make_float4(one(v.x, 4 * i), one(v.y, 4 * i + 1), one(v.z, 4 * i + 2), one(v.w, 4 * i + 3));
        }
    }
    for (size_t i = n4 * 4 + threadIdx.x; i < vocab; i += kCeThreads) gr[i] = one(x[i], i);
    if (threadIdx.x == 0) row_loss[row] = log_z - x_t;
}

// Scalar variant for rows that are not 16-byte aligned (vocab % 4 != 0).
__global__ __launch_bounds__(256) void masked_ce_scalar_kernel(
    const float* logits, const uint32_t* __restrict__ targets, const float* __restrict__ weights,
    float* grad, float* __restrict__ row_loss, size_t rows, size_t vocab, float grad_scale) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float* x = logits + row * vocab;
    float* gr = grad + row * vocab;
    const uint32_t tgt = targets[row];
    if (tgt == FT_MASKED_CE_SKIP) {
        for (size_t i = threadIdx.x; i < vocab; i += 256) gr[i] = 0.0f;
        if (threadIdx.x == 0) row_loss[row] = 0.0f;
        return;
    }
    float m = -3.4e38f;
    for (size_t i = threadIdx.x; i < vocab; i += 256) m = fmaxf(m, x[i]);
    m = block_max<256>(m, red);
    float se = 0.0f;
    for (size_t i = threadIdx.x; i < vocab; i += 256) se += expf(x[i] - m);
    se = block_sum<256>(se, red);
    const float log_z = m + logf(se);
    const float w = weights[row];
    const float x_t = x[tgt];
    __syncthreads();
    for (size_t i = threadIdx.x; i < vocab; i += 256) {
        float gv = expf(x[i] - log_z) * w;
        if (i == (size_t)tgt) gv -= w;
        gr[i] = gv * grad_scale;
    }
    if (threadIdx.x == 0) row_loss[row] = log_z - x_t;
}

// ---------------------------------------------------------------------------
// Sum of squares per 4096-element chunk; AdamW.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void sum_squares_kernel(const float* __restrict__ x, size_t n,
                                                          float* __restrict__ out, size_t offset) {
    __shared__ float red[4];
    const size_t start = (size_t)blockIdx.x * FT_SUM_SQUARES_CHUNK;
    const size_t end = start + FT_SUM_SQUARES_CHUNK < n ? start + FT_SUM_SQUARES_CHUNK : n;
    float acc = 0.0f;
    for (size_t i = start + threadIdx.x; i < end; i += 256) {
        const float v = x[i];
        acc += v * v;
    }
    acc = block_sum<256>(acc, red);
    if (threadIdx.x == 0) out[offset + blockIdx.x] = acc;
}

__device__ __forceinline__ void adamw_one(float& w, float g, float& m, float& v, const ft_adam_params& p,
                                          float bc1, float bc2) {
    m = m * p.beta1 + (1.0f - p.beta1) * g;
    v = v * p.beta2 + (1.0f - p.beta2) * g * g;
    const float m_hat = m / bc1;
    const float v_hat = v / bc2;
    w = w - p.lr * (m_hat / (sqrtf(v_hat) + p.eps) + p.weight_decay * w);
}

// Four parameters per thread (16-byte accesses); n4 = number of whole float4 groups.
__global__ __launch_bounds__(256) void adamw_vec4_kernel(float4* __restrict__ w, const float4* __restrict__ g,
                                                         float4* __restrict__ m, float4* __restrict__ v, size_t n4,
                                                         ft_adam_params p, float grad_scale) {
    const float bc1 = 1.0f - powf(p.beta1, p.t);
    const float bc2 = 1.0f - powf(p.beta2, p.t);
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        float4 wi = w[i], mi = m[i], vi = v[i];
        const float4 gi = g[i];
        adamw_one(wi.x, gi.x * grad_scale, mi.x, vi.x, p, bc1, bc2);
        adamw_one(wi.y, gi.y * grad_scale, mi.y, vi.y, p, bc1, bc2);
        adamw_one(wi.z, gi.z * grad_scale, mi.z, vi.z, p, bc1, bc2);
        adamw_one(wi.w, gi.w * grad_scale, mi.w, vi.w, p, bc1, bc2);
        w[i] = wi;
        m[i] = mi;
        v[i] = vi;
    }
}

__global__ __launch_bounds__(256) void adamw_kernel(float* __restrict__ w, const float* __restrict__ g,
                                                    float* __restrict__ m, float* __restrict__ v, size_t n,
                                                    ft_adam_params p, float grad_scale) {
    const float bc1 = 1.0f - powf(p.beta1, p.t);
    const float bc2 = 1.0f - powf(p.beta2, p.t);
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        float wi = w[i], mi = m[i], vi = v[i];
        adamw_one(wi, g[i] * grad_scale, mi, vi, p, bc1, bc2);
        w[i] = wi;
        m[i] = mi;
        v[i] = vi;
    }
}

}  // namespace

// A segment of the multi-tensor AdamW / gradient-norm launch: one
// FT_SUM_SQUARES_CHUNK-sized piece of one tensor.
struct ft_segment {
    float* w;
    float* g;
    float* m;
    float* v;
    uint32_t n;  // elements in this piece (<= 4096)
};

namespace {

// Step control block in device memory, written by the norm kernel and read by
// the AdamW kernel so that no host round trip sits between them.
struct StepControl {
    float grad_norm;
    float clip_scale;
    int apply;       // 0 when the norm is not finite: the update is skipped
};

__global__ __launch_bounds__(256) void multi_sum_squares_kernel(const ft_segment* __restrict__ segs,
                                                                float* __restrict__ partials) {
    __shared__ float red[4];
    const ft_segment s = segs[blockIdx.x];
    float acc = 0.0f;
    for (uint32_t i = threadIdx.x; i < s.n; i += 256) {
        const float v = s.g[i];
        acc += v * v;
    }
    acc = block_sum<256>(acc, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = acc;
}

// Adds the partials in f64 in index order (the reference adds them on the host
// in f64, trainer/src/lib.rs:528-533), then derives the clip scale
// max / (norm + 1e-6) when norm > max (trainer/src/lib.rs:336-343).
__global__ __launch_bounds__(256) void grad_norm_finish_kernel(const float* __restrict__ partials, size_t count,
                                                               float max_norm, float* out /* StepControl */) {
    __shared__ double red[256];
    // Fixed assignment of contiguous ranges to threads keeps the result
    // independent of scheduling.
    const size_t per = (count + 255) / 256;
    const size_t b = threadIdx.x * per;
    const size_t e = b + per < count ? b + per : count;
    double acc = 0.0;
    for (size_t i = b; i < e; i++) acc += (double)partials[i];
    red[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < 256; i++) t += red[i];
        const float norm = (float)sqrt(t);
        StepControl* c = reinterpret_cast<StepControl*>(out);
        c->grad_norm = norm;
        const bool finite = isfinite(norm);
        c->apply = finite ? 1 : 0;
        c->clip_scale = (finite && max_norm > 0.0f && norm > max_norm) ? max_norm / (norm + 1e-6f) : 1.0f;
    }
}

__global__ __launch_bounds__(256) void multi_adamw_kernel(const ft_segment* __restrict__ segs, ft_adam_params p,
                                                          float grad_scale, const float* control) {
    float scale = grad_scale;
    if (control) {
        const StepControl* c = reinterpret_cast<const StepControl*>(control);
        if (!c->apply) return;
        scale *= c->clip_scale;
    }
    const ft_segment s = segs[blockIdx.x];
    const float bc1 = 1.0f - powf(p.beta1, p.t);
    const float bc2 = 1.0f - powf(p.beta2, p.t);
    for (uint32_t i = threadIdx.x; i < s.n; i += 256) {
        float wi = s.w[i], mi = s.m[i], vi = s.v[i];
        // The clip scale of the reference's clip_grad_by_norm pass is applied on
        // the fly; the stored gradient stays unclipped.
        adamw_one(wi, s.g[i] * scale, mi, vi, p, bc1, bc2);
        s.w[i] = wi;
        s.m[i] = mi;
        s.v[i] = vi;
    }
}

// y[row, col] += bias[col]: the projection bias of `Linear::project_2d` (graph/src/lib.rs:128-139), which the
// reference writes as ones[rows, 1] @ bias[1, out] added to the product.
__global__ void __launch_bounds__(256) row_bias_add_kernel(float* __restrict__ y, const float* __restrict__ bias,
                                                           size_t rows, int cols) {
    const size_t n = rows * (size_t)cols;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        y[i] += bias[i % (size_t)cols];
}

// out[col] (+)= sum over rows of g[row, col]: ones^T @ g, the bias gradient. One workgroup per 64 columns,
// four row lanes per column summed in a fixed order, so the result does not depend on the launch.
__global__ void __launch_bounds__(256) col_sum_kernel(const float* __restrict__ g, float* __restrict__ out,
                                                      size_t rows, int cols, int accumulate) {
    __shared__ float part[4][64];
    const int c = blockIdx.x * 64 + (threadIdx.x & 63);
    const int lane_row = threadIdx.x >> 6;
    float acc = 0.0f;
    if (c < cols)
        for (size_t r = lane_row; r < rows; r += 4) acc += g[r * (size_t)cols + c];
    part[lane_row][threadIdx.x & 63] = acc;
    __syncthreads();
    if (lane_row == 0 && c < cols) {
        const float s = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
        out[c] = accumulate ? out[c] + s : s;
    }
}

}  // namespace

// Internal entry points used by the step driver (ft_step.cpp).
// gx = rms_norm_backward(x, w, g) (+ add); add may be NULL or alias gx. No weight gradient.
int ft_internal_rms_norm_backward_add(ft_context* ctx, const float* x, const float* w, const float* g,
                                      const float* add, float* gx, size_t rows, size_t size, float eps) {
    FT_CHECK_ARG(ctx && x && w && g && gx, "rms_norm_backward: NULL argument");
    FT_CHECK_ARG(size > 0, "rms_norm_backward: size is 0");
    if (rows == 0) return FT_OK;
    const bool vec = (size % 4 == 0) && aligned16(x) && aligned16(w) && aligned16(g) && aligned16(gx) &&
                     aligned16(add) && size <= 2048 && rows < (1u << 30);
    if (!vec) {
        FT_TRY(ft_rms_norm_backward(ctx, x, w, g, gx, nullptr, rows, size, eps));
        if (add) return ft_add(ctx, add, gx, gx, rows * size);
        return FT_OK;
    }
    ft_prof_scope prof(ctx, "rms_norm_backward_kernel", 0.0, (add ? 16.0 : 12.0) * (double)rows * size);
    const dim3 grid(ft_div_up(rows, 4));
    if (size <= 1024)
        hipLaunchKernelGGL((rms_norm_backward_wave_kernel<4>), grid, dim3(256), 0, ctx->stream, x, w, g, add, gx,
                           (int)rows, (int)size, eps, ft_deferred_sum{});
    else
        hipLaunchKernelGGL((rms_norm_backward_wave_kernel<8>), grid, dim3(256), 0, ctx->stream, x, w, g, add, gx,
                           (int)rows, (int)size, eps, ft_deferred_sum{});
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// Can a norm kernel add the K shares of a [rows, size] product itself?
bool ft_internal_norm_can_sum(size_t rows, size_t size) { return size % 4 == 0 && size <= 2048 && rows < (1u << 30); }

// Do the tail tiles `d` describes belong to a dense [rows, size] product in 64 x 64 tiles?
static bool tail_sum_fits(const ft_deferred_sum* d, size_t rows, size_t size) {
    return d->out && aligned16(d->out) && d->panel >= 1 && d->tail_shift <= 3 &&
           (size_t)d->tiles_m == ft_div_up(rows, 64) && (size_t)d->tiles_n == ft_div_up(size, 64) &&
           d->tail_first >= 0 && d->tail_first < d->tiles_m * d->tiles_n;
}

// x_out = the deferred sum `d` ([rows, size]); out = rms_norm(x_out) * w. One pass: the shares are read
// where the plain kernel reads x.
int ft_internal_rms_norm_sum(ft_context* ctx, const ft_deferred_sum* d, float* x_out, const float* w, float* out,
                             size_t rows, size_t size, float eps) {
    FT_CHECK_ARG(ctx && d && d->partial && d->pending() && x_out && w && out, "rms_norm_sum: bad argument");
    FT_CHECK_ARG(ft_internal_norm_can_sum(rows, size) && aligned16(d->partial) && aligned16(d->add) && d->stride % 4 == 0 &&
                     aligned16(x_out) && aligned16(w) && aligned16(out),
                 "rms_norm_sum: shape or alignment outside the fused kernel's");
    const bool tail = d->tail_shift > 0;
    if (tail) FT_CHECK_ARG(tail_sum_fits(d, rows, size) && d->out == x_out, "rms_norm_sum: tail tiles of another product");
    if (rows == 0) return FT_OK;
    ft_prof_scope prof(ctx, "rms_norm_kernel", 0.0, (12.0 + 4.0 * d->splits + (d->add ? 4.0 : 0.0)) * (double)rows * size);
    const dim3 grid(ft_div_up(rows, 4));
    if (tail && size <= 1024)
        hipLaunchKernelGGL((rms_norm_wave_kernel<4, 2>), grid, dim3(256), 0, ctx->stream, x_out, w, out, (int)rows,
                           (int)size, eps, *d, x_out);
    else if (tail)
        hipLaunchKernelGGL((rms_norm_wave_kernel<8, 2>), grid, dim3(256), 0, ctx->stream, x_out, w, out, (int)rows,
                           (int)size, eps, *d, x_out);
    else if (size <= 1024)
        hipLaunchKernelGGL((rms_norm_wave_kernel<4, 1>), grid, dim3(256), 0, ctx->stream, x_out, w, out, (int)rows,
                           (int)size, eps, *d, x_out);
    else
        hipLaunchKernelGGL((rms_norm_wave_kernel<8, 1>), grid, dim3(256), 0, ctx->stream, x_out, w, out, (int)rows,
                           (int)size, eps, *d, x_out);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// gx = rms_norm_backward(x, w, g) (+ add) with g = the deferred sum `d`. No weight gradient.
int ft_internal_rms_norm_backward_sum(ft_context* ctx, const float* x, const float* w, const ft_deferred_sum* d,
                                      const float* add, float* gx, size_t rows, size_t size, float eps) {
    FT_CHECK_ARG(ctx && x && w && d && d->partial && d->pending() && gx, "rms_norm_backward_sum: bad argument");
    FT_CHECK_ARG(ft_internal_norm_can_sum(rows, size) && aligned16(d->partial) && aligned16(d->add) && d->stride % 4 == 0 &&
                     aligned16(x) && aligned16(w) && aligned16(gx) && aligned16(add),
                 "rms_norm_backward_sum: shape or alignment outside the fused kernel's");
    const bool tail = d->tail_shift > 0;
    if (tail) FT_CHECK_ARG(tail_sum_fits(d, rows, size), "rms_norm_backward_sum: tail tiles of another product");
    if (rows == 0) return FT_OK;
    ft_prof_scope prof(ctx, "rms_norm_backward_kernel", 0.0,
                       (8.0 + 4.0 * d->splits + (d->add ? 4.0 : 0.0) + (add ? 4.0 : 0.0)) * (double)rows * size);
    const dim3 grid(ft_div_up(rows, 4));
    if (tail && size <= 1024)
        hipLaunchKernelGGL((rms_norm_backward_wave_kernel<4, 2>), grid, dim3(256), 0, ctx->stream, x, w,
                           (const float*)nullptr, add, gx, (int)rows, (int)size, eps, *d);
    else if (tail)
        hipLaunchKernelGGL((rms_norm_backward_wave_kernel<8, 2>), grid, dim3(256), 0, ctx->stream, x, w,
                           (const float*)nullptr, add, gx, (int)rows, (int)size, eps, *d);
    else if (size <= 1024)
        hipLaunchKernelGGL((rms_norm_backward_wave_kernel<4, 1>), grid, dim3(256), 0, ctx->stream, x, w,
                           (const float*)nullptr, add, gx, (int)rows, (int)size, eps, *d);
    else
        hipLaunchKernelGGL((rms_norm_backward_wave_kernel<8, 1>), grid, dim3(256), 0, ctx->stream, x, w,
                           (const float*)nullptr, add, gx, (int)rows, (int)size, eps, *d);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// y[rows, cols] += bias[cols] on every row.
int ft_internal_row_bias_add(ft_context* ctx, float* y, const float* bias, size_t rows, size_t cols) {
    FT_CHECK_ARG(ctx && y && bias, "row_bias_add: NULL argument");
    FT_CHECK_ARG(cols > 0 && cols < (1u << 30), "row_bias_add: %zu columns", cols);
    if (rows == 0) return FT_OK;
    ft_prof_scope prof(ctx, "row_bias_add_kernel", 0.0, 8.0 * (double)rows * cols);
    const size_t blocks = std::min<size_t>(ft_div_up(rows * cols, 256), 4096);
    hipLaunchKernelGGL(row_bias_add_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, y, bias, rows,
                       (int)cols);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// out[cols] = (or +=, when `accumulate`) the sum of g[rows, cols] over its rows.
int ft_internal_col_sum(ft_context* ctx, const float* g, float* out, size_t rows, size_t cols, int accumulate) {
    FT_CHECK_ARG(ctx && g && out, "col_sum: NULL argument");
    FT_CHECK_ARG(cols > 0 && cols < (1u << 30), "col_sum: %zu columns", cols);
    ft_prof_scope prof(ctx, "col_sum_kernel", 0.0, 4.0 * (double)rows * cols);
    hipLaunchKernelGGL(col_sum_kernel, dim3((unsigned)ft_div_up(cols, 64)), dim3(256), 0, ctx->stream, g, out, rows,
                       (int)cols, accumulate);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// (cos, sin) of pos * theta^(-2i/head_dim) for seq positions; table holds seq * head_dim/2 float2.
int ft_internal_rope_table(ft_context* ctx, float* table, size_t seq, size_t head_dim, size_t pos, float theta) {
    const size_t n = seq * head_dim / 2;
    if (n == 0) return FT_OK;
    hipLaunchKernelGGL(rope_table_kernel, dim3(ft_div_up(n, 256)), dim3(256), 0, ctx->stream,
                       reinterpret_cast<float2*>(table), (unsigned)seq, (unsigned)head_dim, (unsigned)pos, theta);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// Rotates a [batch, seq, heads_a*head_dim] and a [batch, seq, heads_b*head_dim] tensor in one
// launch (src may equal dst). head_dim must be a multiple of 8 and the tensors 16-byte aligned.
int ft_internal_rope_pair(ft_context* ctx, const float* a_src, float* a_dst, size_t heads_a, const float* b_src,
                          float* b_dst, size_t heads_b, const float* table, size_t batch, size_t seq,
                          size_t head_dim, int inverse) {
    FT_CHECK_ARG(head_dim % 8 == 0 && aligned16(a_src) && aligned16(a_dst) && aligned16(b_src) && aligned16(b_dst),
                 "rope pair: head_dim %zu must be a multiple of 8 and the tensors aligned", head_dim);
    RopeJob j0{a_src, a_dst, (unsigned)heads_a, batch * seq * heads_a * head_dim / 8};
    RopeJob j1{b_src, b_dst, (unsigned)heads_b, batch * seq * heads_b * head_dim / 8};
    const size_t qmax = j0.quads > j1.quads ? j0.quads : j1.quads;
    if (qmax == 0) return FT_OK;
    ft_prof_scope prof(ctx, "rope_apply_kernel", 0.0, 8.0 * (double)(j0.quads + j1.quads) * 8);
    hipLaunchKernelGGL(rope_apply_kernel, dim3(ft_div_up(qmax, 256), 2), dim3(256), 0, ctx->stream, j0, j1,
                       reinterpret_cast<const float2*>(table), (unsigned)seq, (unsigned)head_dim,
                       inverse ? -1.0f : 1.0f);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_internal_multi_grad_norm(ft_context* ctx, const ft_segment* segs_dev, size_t nseg, float* partials_dev,
                                float max_norm, float* control_dev) {
    if (nseg == 0) return FT_OK;
    ft_prof_scope prof(ctx, "multi_sum_squares+finish", 0.0, 4.0 * (double)nseg * FT_SUM_SQUARES_CHUNK);
    hipLaunchKernelGGL(multi_sum_squares_kernel, dim3((unsigned)nseg), dim3(256), 0, ctx->stream, segs_dev,
                       partials_dev);
    FT_LAUNCH_CHECK();
    hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(256), 0, ctx->stream, partials_dev, nseg, max_norm,
                       control_dev);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_internal_multi_adamw(ft_context* ctx, const ft_segment* segs_dev, size_t nseg, const ft_adam_params* p,
                            float grad_scale, const float* control_dev) {
    if (nseg == 0) return FT_OK;
    ft_prof_scope prof(ctx, "multi_adamw_kernel", 0.0, 28.0 * (double)nseg * FT_SUM_SQUARES_CHUNK);
    hipLaunchKernelGGL(multi_adamw_kernel, dim3((unsigned)nseg), dim3(256), 0, ctx->stream, segs_dev, *p,
                       grad_scale, control_dev);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// ---------------------------------------------------------------------------
// ft_rms_norm_backward_noalloc: the same two kernels as the norm-weight-gradient path of
// ft_rms_norm_backward, with the partial rows (one per workgroup) in a fixed device array
// instead of a pooled allocation, for callers that cannot allocate (HIP graph capture, tight
// serving loops). Every device the library runs on holds its own copy of the array (2 MiB) at
// its own address until the process ends; the array's name is only a host-side handle, the
// address kernels take comes from hipGetSymbolAddress, looked up once per device.
// ---------------------------------------------------------------------------
namespace {
constexpr int kNoAllocMaxParts = 256;    // partial rows = workgroups of the first kernel
constexpr int kNoAllocMaxSize = 2048;    // floats per row the wave kernels hold in registers
constexpr int kNoAllocMaxDevices = 64;
}  // namespace

static __device__ __align__(256) float scratch[kNoAllocMaxParts * kNoAllocMaxSize];

static std::atomic<float*> g_noalloc_scratch[kNoAllocMaxDevices] = {};  // written once per device, under the mutex
static std::mutex g_noalloc_mutex;

// Device address of `scratch` on `device`, which must be the current device.
int ft_internal_noalloc_init(int device) {
    FT_CHECK_ARG(device >= 0 && device < kNoAllocMaxDevices, "no-alloc scratch: device %d is outside 0..%d", device,
                 kNoAllocMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (g_noalloc_scratch[device].load(std::memory_order_acquire)) return FT_OK;
    float* ptr = nullptr;
    FT_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    FT_CHECK_ARG(ptr != nullptr, "no-alloc scratch: hipGetSymbolAddress returned NULL on device %d", device);
    g_noalloc_scratch[device].store(ptr, std::memory_order_release);
    return FT_OK;
}

extern "C" {

int ft_zero(ft_context* ctx, void* dev, size_t bytes) {
    FT_CHECK_ARG(ctx && (bytes == 0 || dev), "ft_zero: NULL argument");
    FT_CHECK_ARG(bytes % 4 == 0, "ft_zero: %zu bytes is not a whole number of words", bytes);
    EwArgs p{nullptr, nullptr, nullptr, (float*)dev, nullptr, bytes / 4, 0.0f};
    return ew_launch<Ew::Zero>(ctx, p);
}

int ft_add(ft_context* ctx, const float* a, const float* b, float* out, size_t n) {
    FT_CHECK_ARG(ctx && (n == 0 || (a && b && out)), "ft_add: NULL argument");
    EwArgs p{a, b, nullptr, out, nullptr, n, 0.0f};
    return ew_launch<Ew::Add>(ctx, p);
}

int ft_add_backward(ft_context* ctx, const float* g, float* ga, float* gb, size_t n) {
    FT_CHECK_ARG(ctx && (n == 0 || (g && ga && gb)), "ft_add_backward: NULL argument");
    EwArgs p{g, nullptr, nullptr, ga, gb, n, 0.0f};
    return ew_launch<Ew::AddBackward>(ctx, p);
}

int ft_silu_gate_fused(ft_context* ctx, const float* first, const float* second, float* out, size_t n) {
    FT_CHECK_ARG(ctx && (n == 0 || (first && second && out)), "ft_silu_gate_fused: NULL argument");
    EwArgs p{first, second, nullptr, out, nullptr, n, 0.0f};
    return ew_launch<Ew::SiluGate>(ctx, p);
}

int ft_silu_gate_backward(ft_context* ctx, const float* first, const float* second, const float* g,
                          float* g_first, float* g_second, size_t n) {
    FT_CHECK_ARG(ctx && (n == 0 || (first && second && g && g_first && g_second)),
                 "ft_silu_gate_backward: NULL argument");
    EwArgs p{first, second, g, g_first, g_second, n, 0.0f};
    return ew_launch<Ew::SiluGateBackward>(ctx, p);
}

int ft_gradient_scale(ft_context* ctx, float* x, size_t n, float scale) {
    FT_CHECK_ARG(ctx && (n == 0 || x), "ft_gradient_scale: NULL argument");
    EwArgs p{nullptr, nullptr, nullptr, x, nullptr, n, scale};
    return ew_launch<Ew::Scale>(ctx, p);
}

int ft_clip_grad_by_norm(ft_context* ctx, float* x, size_t n, float scale) {
    return ft_gradient_scale(ctx, x, n, scale);
}

int ft_gradient_accumulate(ft_context* ctx, float* acc, const float* g, size_t n) {
    FT_CHECK_ARG(ctx && (n == 0 || (acc && g)), "ft_gradient_accumulate: NULL argument");
    EwArgs p{g, nullptr, nullptr, acc, nullptr, n, 0.0f};
    return ew_launch<Ew::Accumulate>(ctx, p);
}

int ft_embedding(ft_context* ctx, const float* table, size_t vocab, size_t hidden, const uint32_t* ids,
                 size_t n, float* out) {
    FT_CHECK_ARG(ctx && table && ids && out, "ft_embedding: NULL argument");
    if (n == 0 || hidden == 0) return FT_OK;
    ft_prof_scope prof(ctx, "embedding_kernel", 0.0, 8.0 * (double)n * hidden);
    hipLaunchKernelGGL(embedding_kernel, dim3(ft_div_up(n, 4)), dim3(256), 0, ctx->stream, table, vocab, hidden,
                       ids, n, out);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_rope_table(ft_context* ctx, float* table, size_t seq, size_t head_dim, size_t pos, float theta) {
    FT_CHECK_ARG(ctx && table, "ft_rope_table: NULL argument");
    FT_CHECK_ARG(head_dim >= 2 && head_dim % 2 == 0, "ft_rope_table: head_dim %zu must be even", head_dim);
    return ft_internal_rope_table(ctx, table, seq, head_dim, pos, theta);
}

int ft_rope_apply(ft_context* ctx, const float* x, float* out, size_t batch, size_t seq, size_t hidden,
                  size_t head_dim, const float* table, int inverse) {
    FT_CHECK_ARG(ctx && x && out && table, "ft_rope_apply: NULL argument");
    FT_CHECK_ARG(head_dim > 0 && hidden % head_dim == 0, "ft_rope_apply: hidden %zu is not a multiple of head_dim %zu",
                 hidden, head_dim);
    return ft_internal_rope_pair(ctx, x, out, hidden / head_dim, x, out, 0, table, batch, seq, head_dim, inverse);
}

int ft_rms_norm_eps(ft_context* ctx, const float* x, const float* w, float* out, size_t rows, size_t size,
                    float eps) {
    FT_CHECK_ARG(ctx && x && w && out, "ft_rms_norm_eps: NULL argument");
    FT_CHECK_ARG(size > 0, "ft_rms_norm_eps: size is 0");
    if (rows == 0) return FT_OK;
    const int vec = (size % 4 == 0) && aligned16(x) && aligned16(w) && aligned16(out);
    ft_prof_scope prof(ctx, "rms_norm_kernel", 0.0, 8.0 * (double)rows * size);
    if (vec && size <= 2048 && rows < (1u << 30)) {
        const dim3 grid(ft_div_up(rows, 4));
        if (size <= 1024)
            hipLaunchKernelGGL((rms_norm_wave_kernel<4>), grid, dim3(256), 0, ctx->stream, x, w, out, (int)rows,
                               (int)size, eps, ft_deferred_sum{}, (float*)nullptr);
        else
            hipLaunchKernelGGL((rms_norm_wave_kernel<8>), grid, dim3(256), 0, ctx->stream, x, w, out, (int)rows,
                               (int)size, eps, ft_deferred_sum{}, (float*)nullptr);
        FT_LAUNCH_CHECK();
        return FT_OK;
    }
    hipLaunchKernelGGL(rms_norm_kernel, dim3((unsigned)rows), dim3(256), 0, ctx->stream, x, w, out, rows, size,
                       eps, vec);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_rms_norm_backward(ft_context* ctx, const float* x, const float* w, const float* g, float* gx, float* gw,
                         size_t rows, size_t size, float eps) {
    FT_CHECK_ARG(ctx && x && w && g && gx, "ft_rms_norm_backward: NULL argument");
    FT_CHECK_ARG(size > 0, "ft_rms_norm_backward: size is 0");
    if (!gw && rows > 0 && size % 4 == 0 && size <= 2048 && aligned16(x) && aligned16(w) && aligned16(g) &&
        aligned16(gx))
        return ft_internal_rms_norm_backward_add(ctx, x, w, g, nullptr, gx, rows, size, eps);
    if (rows == 0) {
        if (gw) return ft_zero(ctx, gw, size * 4);
        return FT_OK;
    }
    if (gw && size % 4 == 0 && size <= 2048 && rows < (1u << 30) && aligned16(x) && aligned16(w) && aligned16(g) &&
        aligned16(gx)) {
        size_t wgs = (rows + 3) / 4;
        const size_t cap = (size_t)ctx->num_cus;
        if (wgs > cap) wgs = cap;
        float* partial = nullptr;
        FT_TRY(ft_alloc(ctx, wgs * size * sizeof(float), (void**)&partial));
        ft_prof_scope prof(ctx, "rms_norm_backward_gw_kernel", 0.0, 12.0 * (double)rows * size);
        const size_t lds = 3 * size * sizeof(float);
        if (size <= 1024)
            hipLaunchKernelGGL((rms_norm_backward_gw_wave_kernel<4>), dim3((unsigned)wgs), dim3(256), lds, ctx->stream,
                               x, w, g, gx, partial, (int)rows, (int)size, eps);
        else
            hipLaunchKernelGGL((rms_norm_backward_gw_wave_kernel<8>), dim3((unsigned)wgs), dim3(256), lds, ctx->stream,
                               x, w, g, gx, partial, (int)rows, (int)size, eps);
        FT_LAUNCH_CHECK();
        hipLaunchKernelGGL(column_sum_sliced_kernel, dim3(ft_div_up(size, 16)), dim3(256), 0, ctx->stream, partial, gw,
                           (int)wgs, (int)size);
        FT_LAUNCH_CHECK();
        return ft_free(ctx, partial);
    }
    constexpr int RPW = 8;
    const size_t wgs = (rows + RPW - 1) / RPW;
    float* partial = nullptr;
    if (gw) FT_TRY(ft_alloc(ctx, wgs * size * sizeof(float), (void**)&partial));
    ft_prof_scope prof(ctx, "rms_norm_backward_kernel", 0.0, 12.0 * (double)rows * size);
    hipLaunchKernelGGL((rms_norm_backward_kernel<RPW>), dim3((unsigned)wgs), dim3(256), 0, ctx->stream, x, w, g,
                       gx, partial, rows, size, eps);
    FT_LAUNCH_CHECK();
    if (gw) {
        hipLaunchKernelGGL(column_sum_kernel, dim3(ft_div_up(size, 256)), dim3(256), 0, ctx->stream, partial, gw,
                           wgs, size);
        FT_LAUNCH_CHECK();
        FT_TRY(ft_free(ctx, partial));
    }
    return FT_OK;
}

int ft_rms_norm_backward_noalloc(ft_context* ctx, const float* x, const float* w, const float* g, float* gx,
                                 float* gw, size_t rows, size_t size, float eps) {
    FT_CHECK_ARG(ctx && x && w && g && gx && gw, "ft_rms_norm_backward_noalloc: NULL argument");
    FT_CHECK_ARG(size > 0 && size % 4 == 0 && size <= (size_t)kNoAllocMaxSize,
                 "ft_rms_norm_backward_noalloc: size %zu must be a multiple of 4 and at most %d", size,
                 kNoAllocMaxSize);
    FT_CHECK_ARG(rows > 0 && rows < (1u << 30), "ft_rms_norm_backward_noalloc: rows %zu is outside 1..2^30-1", rows);
    FT_CHECK_ARG(aligned16(x) && aligned16(w) && aligned16(g) && aligned16(gx),
                 "ft_rms_norm_backward_noalloc: x, w, g and gx must be 16-byte aligned");
    FT_CHECK_ARG(ctx->device >= 0 && ctx->device < kNoAllocMaxDevices, "ft_rms_norm_backward_noalloc: device %d",
                 ctx->device);
    float* partial = g_noalloc_scratch[ctx->device].load(std::memory_order_acquire);
    // Every context looks the address up when it is created (ft_internal_noalloc_init); looking it up
    // here could load a code object and would change the caller's current device.
    FT_CHECK_ARG(partial, "ft_rms_norm_backward_noalloc: scratch address not initialised for device %d", ctx->device);
    // Same launch shape as ft_rms_norm_backward: one partial row per workgroup, every row of the
    // array that the second kernel reads is written in full by the first (nothing to clear).
    size_t wgs = (rows + 3) / 4;
    size_t cap = (size_t)ctx->num_cus;
    if (cap > (size_t)kNoAllocMaxParts) cap = kNoAllocMaxParts;
    if (wgs > cap) wgs = cap;
    const size_t lds = 3 * size * sizeof(float);
    if (size <= 1024)
        hipLaunchKernelGGL((rms_norm_backward_gw_wave_kernel<4>), dim3((unsigned)wgs), dim3(256), lds, ctx->stream, x, w,
                           g, gx, partial, (int)rows, (int)size, eps);
    else
        hipLaunchKernelGGL((rms_norm_backward_gw_wave_kernel<8>), dim3((unsigned)wgs), dim3(256), lds, ctx->stream, x, w,
                           g, gx, partial, (int)rows, (int)size, eps);
    FT_LAUNCH_CHECK();
    hipLaunchKernelGGL(column_sum_sliced_kernel, dim3(ft_div_up(size, 16)), dim3(256), 0, ctx->stream, partial, gw,
                       (int)wgs, (int)size);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

static int rope_launch(ft_context* ctx, const float* src, float* dst, size_t batch, size_t seq, size_t hidden,
                       size_t head_dim, size_t pos, float theta, int inverse, const char* who) {
    FT_CHECK_ARG(ctx && src && dst, "%s: NULL argument", who);
    FT_CHECK_ARG(head_dim >= 2 && head_dim % 2 == 0, "%s: head_dim %zu must be even", who, head_dim);
    FT_CHECK_ARG(hidden % head_dim == 0, "%s: hidden %zu is not a multiple of head_dim %zu", who, hidden, head_dim);
    const size_t pairs = batch * seq * hidden / 2;
    if (pairs == 0) return FT_OK;
    ft_prof_scope prof(ctx, "rope_kernel", 0.0, 8.0 * (double)pairs * 2);
    hipLaunchKernelGGL(rope_kernel, dim3(ft_div_up(pairs, 256)), dim3(256), 0, ctx->stream, src, dst, pairs,
                       (unsigned)head_dim, (unsigned)seq, (unsigned)pos, (unsigned)(hidden / head_dim), theta,
                       inverse ? -1.0f : 1.0f);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_rope_theta(ft_context* ctx, float* t, size_t batch, size_t seq, size_t hidden, size_t head_dim, size_t pos,
                  float theta) {
    return rope_launch(ctx, t, t, batch, seq, hidden, head_dim, pos, theta, 0, "ft_rope_theta");
}

int ft_rope_theta_inverse(ft_context* ctx, float* t, size_t batch, size_t seq, size_t hidden, size_t head_dim,
                          size_t pos, float theta) {
    return rope_launch(ctx, t, t, batch, seq, hidden, head_dim, pos, theta, 1, "ft_rope_theta_inverse");
}

int ft_rope_theta_to(ft_context* ctx, const float* src, float* dst, size_t batch, size_t seq, size_t hidden,
                     size_t head_dim, size_t pos, float theta, int inverse) {
    return rope_launch(ctx, src, dst, batch, seq, hidden, head_dim, pos, theta, inverse, "ft_rope_theta_to");
}

int ft_sum_squares_partial(ft_context* ctx, const float* x, size_t n, float* out, size_t offset, size_t* chunks) {
    FT_CHECK_ARG(ctx && out && (n == 0 || x), "ft_sum_squares_partial: NULL argument");
    const size_t blocks = (n + FT_SUM_SQUARES_CHUNK - 1) / FT_SUM_SQUARES_CHUNK;
    if (chunks) *chunks = blocks;
    if (blocks == 0) return FT_OK;
    hipLaunchKernelGGL(sum_squares_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, x, n, out, offset);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_masked_cross_entropy_weighted(ft_context* ctx, const float* logits, const uint32_t* targets,
                                     const float* weights, float* grad, float* row_loss, size_t rows, size_t vocab,
                                     float grad_scale) {
    FT_CHECK_ARG(ctx && logits && targets && weights && grad && row_loss,
                 "ft_masked_cross_entropy_weighted: NULL argument");
    FT_CHECK_ARG(vocab > 0, "ft_masked_cross_entropy_weighted: vocab is 0");
    if (rows == 0) return FT_OK;
    const bool vec = (vocab % 4 == 0) && aligned16(logits) && aligned16(grad);
    const dim3 grid((unsigned)rows);
    ft_prof_scope prof(ctx, "masked_ce_kernel", 0.0, 8.0 * (double)rows * vocab);
    if (!vec) {
        hipLaunchKernelGGL(masked_ce_scalar_kernel, grid, dim3(256), 0, ctx->stream, logits, targets, weights, grad,
                           row_loss, rows, vocab, grad_scale);
    } else if (vocab <= (size_t)kCeThreads * 4 * 4) {
        hipLaunchKernelGGL((masked_ce_kernel<4>), grid, dim3(kCeThreads), 0, ctx->stream, logits, targets, weights,
                           grad, row_loss, rows, vocab, grad_scale);
    } else if (vocab <= (size_t)kCeThreads * 4 * 12) {
        hipLaunchKernelGGL((masked_ce_kernel<12>), grid, dim3(kCeThreads), 0, ctx->stream, logits, targets, weights,
                           grad, row_loss, rows, vocab, grad_scale);
    } else {
        hipLaunchKernelGGL((masked_ce_kernel<0>), grid, dim3(kCeThreads), 0, ctx->stream, logits, targets, weights,
                           grad, row_loss, rows, vocab, grad_scale);
    }
    FT_LAUNCH_CHECK();
    return FT_OK;
}

int ft_adamw_update(ft_context* ctx, float* w, const float* g, float* m, float* v, size_t n,
                    const ft_adam_params* p) {
    FT_CHECK_ARG(ctx && p && (n == 0 || (w && g && m && v)), "ft_adamw_update: NULL argument");
    if (n == 0) return FT_OK;
    ft_prof_scope prof(ctx, "adamw_kernel", 0.0, 28.0 * (double)n);
    const size_t cap = (size_t)ctx->num_cus * 16;
    size_t done = 0;
    if (n >= 4 && aligned16(w) && aligned16(g) && aligned16(m) && aligned16(v)) {
        const size_t n4 = n / 4;
        size_t blocks = (n4 + 255) / 256;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(adamw_vec4_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                           reinterpret_cast<float4*>(w), reinterpret_cast<const float4*>(g),
                           reinterpret_cast<float4*>(m), reinterpret_cast<float4*>(v), n4, *p, 1.0f);
        FT_LAUNCH_CHECK();
        done = n4 * 4;
    }
    if (done < n) {
        size_t blocks = (n - done + 255) / 256;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(adamw_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, w + done, g + done,
                           m + done, v + done, n - done, *p, 1.0f);
        FT_LAUNCH_CHECK();
    }
    return FT_OK;
}

int ft_adamw_update_multi(ft_context* ctx, float* const* w, const float* const* g, float* const* m, float* const* v,
                          const size_t* sizes, size_t count, const ft_adam_params* p, float grad_scale) {
    FT_CHECK_ARG(ctx && p && (count == 0 || (w && g && m && v && sizes)), "ft_adamw_update_multi: NULL argument");
    std::vector<ft_segment> segs;
    for (size_t t = 0; t < count; t++) {
        FT_CHECK_ARG(sizes[t] == 0 || (w[t] && g[t] && m[t] && v[t]), "ft_adamw_update_multi: tensor %zu is NULL", t);
        for (size_t off = 0; off < sizes[t]; off += FT_SUM_SQUARES_CHUNK) {
            const size_t n = sizes[t] - off < FT_SUM_SQUARES_CHUNK ? sizes[t] - off : FT_SUM_SQUARES_CHUNK;
            segs.push_back(ft_segment{w[t] + off, const_cast<float*>(g[t]) + off, m[t] + off, v[t] + off, (uint32_t)n});
        }
    }
    if (segs.empty()) return FT_OK;
    ft_segment* dev = nullptr;
    FT_TRY(ft_alloc(ctx, segs.size() * sizeof(ft_segment), (void**)&dev));
    int rc = ft_upload(ctx, dev, segs.data(), segs.size() * sizeof(ft_segment));
    if (rc == FT_OK) rc = ft_internal_multi_adamw(ctx, dev, segs.size(), p, grad_scale, nullptr);
    const int rc2 = ft_free(ctx, dev);
    return rc != FT_OK ? rc : rc2;
}

}  // extern "C"
