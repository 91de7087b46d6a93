// f32 matrix products on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32).
//
// gemm_kernel: out[M,N] = op(a) @ op(b) (+ a2[M,K2] @ op(b2)) for the three
// layouts of the reference's tile kernel (a@b, a@b^T, a^T@b), with b stored as
// f32 or as packed f16 (converted to f32 while the tile is staged into LDS).
// The optional second product is the rank-r LoRA term: it runs as extra
// iterations of the same K loop, so the fused linear costs r/K more MFMAs and
// no extra pass over the output.
//
// Tiling: 256 threads = 4 waves, each wave owns a WM x WN block of 32x32 MFMA
// accumulators. Tiles of BK = 32 are double-buffered in LDS in a "k-quad
// major" layout [BK/4][rows][4]: one ds_read_b128 gives a lane the four k
// values it feeds to four consecutive MFMAs (lanes 0-31 take the even quads,
// lanes 32-63 the odd ones; the sum over k does not care about the order).
//
// skinny_kernel: products with at most 32 output columns (the LoRA x@A, dT, dA
// and dB products), operands read straight from global memory into MFMA
// operand registers, the reduction dimension split across the 4 waves.
#include "ft_common.h"
#include "ft_thin.h"

#include <cmath>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

constexpr int BK = 32;
constexpr int KQ = BK / 4;
constexpr int LDS_PAD = 8;  // floats: makes the k-quad row stride = 8 (mod 32) banks

struct GemmArgs {
    const float* a;
    const void* b;
    float* out;
    const float* a2;
    const float* b2;
    const float* add;  // optional [M,N] term added in the epilogue (may be `out` itself)
    int M, N, K, K2;
    long lda, ldb, ldc, lda2, ldb2;
    int tiles_n;
};

// ---- guarded 4-element loads along the contiguous dimension --------------

__device__ __forceinline__ float4 load4(const float* p, int nvalid) {
    if (nvalid >= 4 && (((uintptr_t)p) & 15) == 0) return *reinterpret_cast<const float4*>(p);
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nvalid > 0) r.x = p[0];
    if (nvalid > 1) r.y = p[1];
    if (nvalid > 2) r.z = p[2];
    if (nvalid > 3) r.w = p[3];
    return r;
}

__device__ __forceinline__ float4 load4(const _Float16* p, int nvalid) {
    if (nvalid >= 4 && (((uintptr_t)p) & 7) == 0) {
        const half4_t h = *reinterpret_cast<const half4_t*>(p);
        return make_float4((float)h.x, (float)h.y, (float)h.z, (float)h.w);
    }
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nvalid > 0) r.x = (float)p[0];
    if (nvalid > 1) r.y = (float)p[1];
    if (nvalid > 2) r.z = (float)p[2];
    if (nvalid > 3) r.w = (float)p[3];
    return r;
}

__device__ __forceinline__ int clamp04(int v) { return v < 0 ? 0 : (v > 4 ? 4 : v); }

// A ROWS x BK tile on its way from global memory to LDS, held in registers.
// KCONTIG: element (row, k) at base[row*ld + k]; otherwise at base[k*ld + row].
template <int ROWS, bool KCONTIG>
struct TileRegs {
    static constexpr int STRIDE = ROWS * 4 + LDS_PAD;  // floats per k-quad row in LDS
    static constexpr int SLOTS_K = ROWS * KQ / 256;    // one float4 (4 k of one row) each
    static constexpr int GROUPS = (ROWS / 4) * KQ;      // 4 rows x 4 k each
    static constexpr int SLOTS_M = (GROUPS + 255) / 256;
    static constexpr int NREG = KCONTIG ? SLOTS_K : SLOTS_M * 4;
    float4 r[NREG];

    template <typename T>
    __device__ __forceinline__ void load(const T* base, long ld, int row0, int row_limit, int k0, int k_limit) {
        const int tid = threadIdx.x;
        if constexpr (KCONTIG) {
#pragma unroll
            for (int i = 0; i < SLOTS_K; i++) {
                const int s = tid + i * 256;
                const int row = s / KQ, kq = s % KQ;
                const int gr = row0 + row, gk = k0 + kq * 4;
                const int nvalid = gr < row_limit ? clamp04(k_limit - gk) : 0;
                r[i] = load4(base + (long)gr * ld + gk, nvalid);
            }
        } else {
#pragma unroll
            for (int i = 0; i < SLOTS_M; i++) {
                const int s = tid + i * 256;
                float4 v[4];
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (s < GROUPS) {
                    const int rg = s % (ROWS / 4), kq = s / (ROWS / 4);
                    const int gr = row0 + rg * 4;
                    const int nvalid = clamp04(row_limit - gr);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int gk = k0 + kq * 4 + j;
                        if (gk < k_limit) v[j] = load4(base + (long)gk * ld + gr, nvalid);
                    }
                }
                // 4x4 transpose: register q holds the 4 k values of row q.
                r[i * 4 + 0] = make_float4(v[0].x, v[1].x, v[2].x, v[3].x);
                r[i * 4 + 1] = make_float4(v[0].y, v[1].y, v[2].y, v[3].y);
                r[i * 4 + 2] = make_float4(v[0].z, v[1].z, v[2].z, v[3].z);
                r[i * 4 + 3] = make_float4(v[0].w, v[1].w, v[2].w, v[3].w);
            }
        }
    }

    __device__ __forceinline__ void store(float* lds) const {
        const int tid = threadIdx.x;
        if constexpr (KCONTIG) {
#pragma unroll
            for (int i = 0; i < SLOTS_K; i++) {
                const int s = tid + i * 256;
                const int row = s / KQ, kq = s % KQ;
                *reinterpret_cast<float4*>(lds + kq * STRIDE + row * 4) = r[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < SLOTS_M; i++) {
                const int s = tid + i * 256;
                if (s < GROUPS) {
                    const int rg = s % (ROWS / 4), kq = s / (ROWS / 4);
                    float* dst = lds + kq * STRIDE + rg * 16;
#pragma unroll
                    for (int q = 0; q < 4; q++) *reinterpret_cast<float4*>(dst + q * 4) = r[i * 4 + q];
                }
            }
        }
    }
};

// LAYOUT 0: a[M,K]   b[K,N]   (a k-contiguous, b n-contiguous)
// LAYOUT 1: a[M,K]   b[N,K]   (both k-contiguous)
// LAYOUT 2: a[K,M]   b[K,N]   (both m/n-contiguous)
template <int BM, int BN, int WM, int WN, int LAYOUT, bool HALF_B>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
    constexpr bool A_KC = LAYOUT != 2;
    constexpr bool B_KC = LAYOUT == 1;
    constexpr int FM = WM / 32, FN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    static_assert((BM / WM) * (BN / WN) == 4, "4 waves per workgroup");
    using ATile = TileRegs<BM, A_KC>;
    using BTile = TileRegs<BN, B_KC>;
    using BType = typename std::conditional<HALF_B, _Float16, float>::type;

    __shared__ __attribute__((aligned(16))) float As[2][KQ * (BM * 4 + LDS_PAD)];
    __shared__ __attribute__((aligned(16))) float Bs[2][KQ * (BN * 4 + LDS_PAD)];

    const int tile = blockIdx.x;
    const int m0 = (tile / p.tiles_n) * BM;
    const int n0 = (tile % p.tiles_n) * BN;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l32 = lane % 32, half = lane / 32;

    floatx16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int nt1 = (p.K + BK - 1) / BK;
    const int nt2 = (LAYOUT != 2 && p.a2) ? (p.K2 + BK - 1) / BK : 0;
    const int nt = nt1 + nt2;
    const BType* bmat = reinterpret_cast<const BType*>(p.b);

    ATile ta;
    BTile tb;

    // Tiles past nt1 belong to the second product (always f32, a2 k-contiguous,
    // b2 oriented like b); they reuse the same registers and LDS slots.
    auto fetch = [&](int t) {
        if (t < nt1) {
            ta.load(p.a, p.lda, m0, p.M, t * BK, p.K);
            tb.load(bmat, p.ldb, n0, p.N, t * BK, p.K);
        } else if constexpr (LAYOUT != 2) {
            ta.load(p.a2, p.lda2, m0, p.M, (t - nt1) * BK, p.K2);
            tb.load(p.b2, p.ldb2, n0, p.N, (t - nt1) * BK, p.K2);
        }
    };
    auto stash = [&](int buf) {
        ta.store(As[buf]);
        tb.store(Bs[buf]);
    };

    if (nt > 0) {
        fetch(0);
        stash(0);
    }
    __syncthreads();
    for (int t = 0; t < nt; t++) {
        const int buf = t & 1;
        if (t + 1 < nt) fetch(t + 1);
        const float* as = As[buf];
        const float* bs = Bs[buf];
#pragma unroll
        for (int s = 0; s < KQ / 2; s++) {
            const int kq = 2 * s + half;
            float4 af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; i++)
                af[i] = *reinterpret_cast<const float4*>(as + kq * (BM * 4 + LDS_PAD) + (wm0 + i * 32 + l32) * 4);
#pragma unroll
            for (int j = 0; j < FN; j++)
                bf[j] = *reinterpret_cast<const float4*>(bs + kq * (BN * 4 + LDS_PAD) + (wn0 + j * 32 + l32) * 4);
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].x, bf[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].y, bf[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].z, bf[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].w, bf[j].w, acc[i][j], 0, 0, 0);
                }
        }
        if (t + 1 < nt) stash(buf ^ 1);
        __syncthreads();
    }

    // Accumulator register r of a lane is row (r/4)*8 + (lane/32)*4 + r%4,
    // column lane%32 of its 32x32 block.
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++) {
            const int col = n0 + wn0 + j * 32 + l32;
            if (col >= p.N) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm0 + i * 32 + (r / 4) * 8 + half * 4 + (r % 4);
                if (row < p.M) {
                    const long o = (long)row * p.ldc + col;
                    p.out[o] = p.add ? acc[i][j][r] + p.add[o] : acc[i][j][r];
                }
            }
        }
}

// ---------------------------------------------------------------------------
// Fast path: the same product for operands that are 16-byte aligned with
// leading dimensions and K, K2 multiples of 4 (and, for operands whose rows run
// along the contiguous dimension, a row count that is a multiple of 4). Edge
// tiles are handled without branches: out-of-range rows read a clamped (valid)
// address and produce values that are never stored, out-of-range k is zeroed
// by a select. The loop body is straight-line code.
//
// LDS layouts: a k-contiguous operand is staged "k-quad major" as above
// ([BK/4][rows][4], one ds_read_b128 per 4 MFMAs); an operand whose rows are
// contiguous in memory is staged k-major ([BK][rows]) exactly as loaded, so no
// register transpose is needed and both the b128 stores and the b32 operand
// reads are free of bank conflicts.
// ---------------------------------------------------------------------------

// 16 bytes of zeros that out-of-range k loads are redirected to, so that no
// select has to wait for the load.
__device__ __attribute__((aligned(16))) float g_zero16[4] = {0.f, 0.f, 0.f, 0.f};

typedef float float2_t __attribute__((ext_vector_type(2)));

template <int ROWS, bool KCONTIG, int BKT>
struct FastTile {
    static constexpr int KQT = BKT / 4;
    static constexpr int PAD = 4;
    static constexpr int KQ_STRIDE = ROWS * 4 + PAD;   // k-quad major: floats per quad row (== 4 mod 32)
    static constexpr int K_STRIDE = ROWS + PAD;        // k-major: floats per k row
    static constexpr int LDS_FLOATS = KCONTIG ? KQT * KQ_STRIDE : BKT * K_STRIDE;
    static constexpr int SLOTS = KCONTIG ? ROWS * KQT / 256 : BKT * (ROWS / 4) / 256;
    static_assert(SLOTS >= 1, "tile too small for 256 threads");
    // Raw loaded bits: 4 floats, or 4 halfs in .x/.y. Converted when stored to
    // LDS, so nothing between the load and the MFMA block depends on it.
    float4 r[SLOTS];
    // Byte offset of each slot from the tile's (uniform) base pointer: constant
    // over the K loop, so a load costs no per-lane address arithmetic.
    unsigned off[SLOTS];

    __device__ __forceinline__ static void slot_coords(int i, int& row, int& k) {
        const int s = threadIdx.x + i * 256;
        if constexpr (KCONTIG) {
            row = s / KQT;
            k = (s % KQT) * 4;
        } else {
            row = (s % (ROWS / 4)) * 4;
            k = s / (ROWS / 4);
        }
    }

    // Offsets for an operand with leading dimension ld (elements of esize bytes);
    // rows past row_limit are clamped to a valid row (their results are never stored).
    __device__ __forceinline__ void set_offsets(long ld, int row0, int row_limit, int esize) {
#pragma unroll
        for (int i = 0; i < SLOTS; i++) {
            int row, k;
            slot_coords(i, row, k);
            int gr = row0 + row;
            if constexpr (KCONTIG) {
                gr = gr < row_limit ? gr : row_limit - 1;
                off[i] = (unsigned)(((long)gr * ld + k) * esize);
            } else {
                gr = gr + 4 <= row_limit ? gr : row_limit - 4;
                off[i] = (unsigned)(((long)k * ld + gr) * esize);
            }
        }
    }

    // tile_base = operand base advanced to k0 (uniform). GUARD: k0 + k may run
    // past k_limit; such slots read a line of zeros instead.
    template <typename T, bool GUARD>
    __device__ __forceinline__ void load(const char* tile_base, int k0, int k_limit) {
#pragma unroll
        for (int i = 0; i < SLOTS; i++) {
            const char* src = tile_base + off[i];
            if constexpr (GUARD) {
                int row, k;
                slot_coords(i, row, k);
                if (k0 + k >= k_limit) src = reinterpret_cast<const char*>(g_zero16);
            }
            if constexpr (sizeof(T) == 2) {
                const float2_t raw = *reinterpret_cast<const float2_t*>(src);
                r[i].x = raw.x;
                r[i].y = raw.y;
            } else {
                r[i] = *reinterpret_cast<const float4*>(src);
            }
        }
    }

    template <typename T>
    __device__ __forceinline__ void store(float* lds) const {
#pragma unroll
        for (int i = 0; i < SLOTS; i++) {
            int row, k;
            slot_coords(i, row, k);
            float4 v;
            if constexpr (sizeof(T) == 2) {
                float2_t raw;
                raw.x = r[i].x;
                raw.y = r[i].y;
                const half4_t h = __builtin_bit_cast(half4_t, raw);
                v = make_float4((float)h.x, (float)h.y, (float)h.z, (float)h.w);
            } else {
                v = r[i];
            }
            if constexpr (KCONTIG)
                *reinterpret_cast<float4*>(lds + (k / 4) * KQ_STRIDE + row * 4) = v;
            else
                *reinterpret_cast<float4*>(lds + k * K_STRIDE + row) = v;
        }
    }

    // The 4 k values lane (row, half) feeds to MFMAs 4*step .. 4*step+3.
    __device__ __forceinline__ static float4 frag(const float* lds, int step, int half, int row) {
        if constexpr (KCONTIG) {
            return *reinterpret_cast<const float4*>(lds + (2 * step + half) * KQ_STRIDE + row * 4);
        } else {
            const float* p = lds + (8 * step + 4 * half) * K_STRIDE + row;
            return make_float4(p[0], p[K_STRIDE], p[2 * K_STRIDE], p[3 * K_STRIDE]);
        }
    }
};

template <int BM, int BN, int WM, int WN, int LAYOUT, bool HALF_B, int BKT>
__global__ __launch_bounds__(256) void gemm_fast_kernel(GemmArgs p) {
    constexpr bool A_KC = LAYOUT != 2;
    constexpr bool B_KC = LAYOUT == 1;
    constexpr int FM = WM / 32, FN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    constexpr int STEPS = BKT / 8;
    static_assert((BM / WM) * (BN / WN) == 4, "4 waves per workgroup");
    using ATile = FastTile<BM, A_KC, BKT>;
    using BTile = FastTile<BN, B_KC, BKT>;
    using BType = typename std::conditional<HALF_B, _Float16, float>::type;

    __shared__ __attribute__((aligned(16))) float As[2][ATile::LDS_FLOATS];
    __shared__ __attribute__((aligned(16))) float Bs[2][BTile::LDS_FLOATS];

    const int tile = blockIdx.x;
    const int m0 = (tile / p.tiles_n) * BM;
    const int n0 = (tile % p.tiles_n) * BN;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l32 = lane % 32, half = lane / 32;

    floatx16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int nt1 = (p.K + BKT - 1) / BKT;
    const int nt1_full = p.K / BKT;  // tiles that need no k guard
    const int nt2 = (LAYOUT != 2 && p.a2) ? (p.K2 + BKT - 1) / BKT : 0;
    const int nt = nt1 + nt2;
    const long a_kstep = (A_KC ? 1 : p.lda) * 4;                                // bytes per k
    const long b_kstep = (B_KC ? 1 : p.ldb) * (long)sizeof(BType);
    const long b2_kstep = (B_KC ? 1 : p.ldb2) * 4;

    ATile ta;
    BTile tb;
    ta.set_offsets(p.lda, m0, p.M, 4);
    tb.set_offsets(p.ldb, n0, p.N, (int)sizeof(BType));

    // Tiles past nt1 belong to the second (LoRA) product: f32 operands, same
    // orientation, their own leading dimensions (offsets are re-derived once).
    auto fetch = [&](int t) {
        if (t < nt1_full) {
            ta.template load<float, false>(reinterpret_cast<const char*>(p.a) + (long)t * BKT * a_kstep, 0, 0);
            tb.template load<BType, false>(reinterpret_cast<const char*>(p.b) + (long)t * BKT * b_kstep, 0, 0);
        } else if (t < nt1) {
            ta.template load<float, true>(reinterpret_cast<const char*>(p.a) + (long)t * BKT * a_kstep, t * BKT, p.K);
            tb.template load<BType, true>(reinterpret_cast<const char*>(p.b) + (long)t * BKT * b_kstep, t * BKT, p.K);
        } else if constexpr (LAYOUT != 2) {
            const int k0 = (t - nt1) * BKT;
            if (t == nt1) {
                ta.set_offsets(p.lda2, m0, p.M, 4);
                tb.set_offsets(p.ldb2, n0, p.N, 4);
            }
            ta.template load<float, true>(reinterpret_cast<const char*>(p.a2) + (long)k0 * 4, k0, p.K2);
            tb.template load<float, true>(reinterpret_cast<const char*>(p.b2) + (long)k0 * b2_kstep, k0, p.K2);
        }
    };
    auto stash = [&](int t, int buf) {
        ta.template store<float>(As[buf]);
        if (t < nt1)
            tb.template store<BType>(Bs[buf]);
        else
            tb.template store<float>(Bs[buf]);
    };
    auto mfma_step = [&](const float4 (&af)[FM], const float4 (&bf)[FN]) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].x, bf[j].x, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].y, bf[j].y, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].z, bf[j].z, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].w, bf[j].w, acc[i][j], 0, 0, 0);
            }
    };

    if (nt > 0) {
        fetch(0);
        stash(0, 0);
    }
    __syncthreads();
    for (int t = 0; t < nt; t++) {
        const int buf = t & 1;
        const float* as = As[buf];
        const float* bs = Bs[buf];
        float4 af[2][FM], bf[2][FN];
        // Order inside one K tile (the scheduling barriers pin it): operand
        // reads of step 0 and 1, MFMAs of step 0, THEN the global loads of the
        // next tile (their address setup runs under step 0's matrix work
        // instead of in front of it), remaining steps, and the next tile's LDS
        // stores (f16 -> f32 conversion included) before the last step.
#pragma unroll
        for (int i = 0; i < FM; i++) af[0][i] = ATile::frag(as, 0, half, wm0 + i * 32 + l32);
#pragma unroll
        for (int j = 0; j < FN; j++) bf[0][j] = BTile::frag(bs, 0, half, wn0 + j * 32 + l32);
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const int cur = s & 1, nxt = cur ^ 1;
            if (s + 1 < STEPS) {
#pragma unroll
                for (int i = 0; i < FM; i++) af[nxt][i] = ATile::frag(as, s + 1, half, wm0 + i * 32 + l32);
#pragma unroll
                for (int j = 0; j < FN; j++) bf[nxt][j] = BTile::frag(bs, s + 1, half, wn0 + j * 32 + l32);
            }
            __builtin_amdgcn_sched_barrier(0);
            mfma_step(af[cur], bf[cur]);
            __builtin_amdgcn_sched_barrier(0);
            if (s == 0 && t + 1 < nt) {
                fetch(t + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s == STEPS - 2 && t + 1 < nt) {
                stash(t + 1, buf ^ 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++) {
            const int col = n0 + wn0 + j * 32 + l32;
            if (col >= p.N) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm0 + i * 32 + (r / 4) * 8 + half * 4 + (r % 4);
                if (row < p.M) {
                    const long o = (long)row * p.ldc + col;
                    p.out[o] = p.add ? acc[i][j][r] + p.add[o] : acc[i][j][r];
                }
            }
        }
}

// ---------------------------------------------------------------------------
// Asynchronous path for the shapes the training step is made of: f32 a[M,K],
// packed f16 b, K a multiple of 32. Both operand tiles go from global memory
// straight into LDS with global_load_lds_dwordx4 (no VGPR staging, no LDS
// stores, no per-tile address arithmetic), NST tiles deep, so a workgroup
// always has NST-1 tiles of loads in flight behind the one it multiplies.
// b stays f16 in LDS and is converted as it is read into MFMA operands.
//
// A lane's 16 bytes land at (LDS base of the instruction) + 16 * lane, so the
// LDS image of a tile is fixed by which global address each lane is given:
//   a tile   [BM rows][32 k] f32, 128 B per row, 8 rows per instruction; the
//            16-byte column c of row r holds k-quad c ^ ((r >> 1) & 7): measured, this
//            is the swizzle with which the ds_read_b128 of a wave (32 rows x 2 k-quads)
//            runs at the rate of a linear read (c ^ (r & 7) takes twice as long).
//   b tile   layout 1 (b[N,K]): [BN rows][32 k] f16, 64 B per row, 16 rows per
//            instruction, 16-byte column c holds k-octet c ^ ((r >> 2) & 3) (likewise measured).
//            layout 0 (b[K,N]): [32 k][BN n] f16 exactly as in memory; a lane
//            reads its column's 4 k values as four 16-bit loads.
// The K loop is unrolled over the stages; the waits are explicit (s_waitcnt
// vmcnt(n) + s_barrier, not __syncthreads, whose fence would drain every
// outstanding load).
// The rank-r second product is loaded into registers before the loop and
// multiplied from a small LDS tile after it (K2 <= 16).
// ---------------------------------------------------------------------------

// global_load_lds_dwordx4 with a uniform 64-bit base, a per-lane 32-bit byte
// offset and a uniform LDS destination (M0). Written as inline assembly so the
// compiler does not track it: with the builtin it drains every outstanding
// LDS-DMA load (vmcnt(0)) in front of the first LDS read after the loop
// back-edge, which defeats the multi-stage pipeline. The waits are explicit.
__device__ __forceinline__ void glds16(const char* base, unsigned voff, const float* lds_dst) {
    const unsigned l = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)lds_dst);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(l) : "memory", "m0");
}

// One launch covers up to kAsyncMaxProb products that share M (and usually the a
// operand): q/k/v or gate/up of one input, each with its own b, output, rank-r
// term and residual. A product may itself be a sum over up to kAsyncMaxSeg K
// segments with their own a and b (dx = dq Wq^T + dk Wk^T + dv Wv^T): the tile
// pipeline runs through the segments without draining.
constexpr int kAsyncMaxSeg = 3, kAsyncMaxProb = 3;

struct AsyncSeg {
    const float* a;   // [M, 32 * nt] f32
    const void* b;    // packed f16: layout 0 [K, N], layout 1 [N, K]
    const float* a2;  // rank-r term of this segment ([M, K2] and [K2, N] / [N, K2]), or NULL
    const float* b2;
    int lda, ldb, lda2, ldb2;
    int nt;           // K tiles of this segment
    int K2;
};

struct AsyncProb {
    AsyncSeg seg[kAsyncMaxSeg];
    float* out;
    const float* add;  // optional [M, N] term added in the epilogue (may be `out` itself)
    // Fused epilogues (one segment, no rank-r term):
    //   kEpiGateUp     b_alt is a second b of the same shape; out = a@b, out2 = a@b_alt,
    //                  out3 = silu(out2) * out            (up, gate, activation)
    //   kEpiSiluBwd    with d = a@b (never stored), e1 = gate, e2 = up:
    //                  out = d * e2 * silu'(e1), out2 = d * silu(e1)   (d_gate, d_up)
    const void* b_alt;
    float* out2;
    float* out3;
    const float* e1;
    const float* e2;
    int N, ldc, tile_begin, nseg;  // tile_begin: first n tile of this product in the batch's row of n tiles
    long partial_off;  // split-K: this product's slice of AsyncBatch::partial, [splits][M][N]
    // RoPE on the output (64x64 tiles, head_dim 64, so a tile is one head of 64 rows): element
    // (row, h*64 + i) pairs with (row, h*64 + i + 32) and rotates by the (cos, sin) of token position
    // row % rope_seq, table [rope_seq][32] float2. NULL = no rotation.
    const float2* rope;
    int rope_seq;
};

constexpr int kEpiPlain = 0, kEpiGateUp = 1, kEpiSiluBwd = 2;

// Split-K (few tiles, e.g. one sequence per pass: M = 256): blockIdx.y takes a
// contiguous share of the K tiles and writes its partial tile to `partial`;
// splitk_reduce_kernel adds the shares in order (and the residual) into `out`.
struct AsyncBatch {
    AsyncProb p[kAsyncMaxProb];
    int count, M;
    int splits;        // 1 = none
    float* partial;
    int tiles_m, tiles_n;  // row blocks; n tiles of all products together
    int xcds;              // chunks of the tile order (one per XCD), 1 = workgroup id order
    int panel;             // n tiles per panel of the tile order
    // Tail split: a tile count a little above a multiple of the CU count (800 on 256) leaves 32 CUs with a
    // fourth workgroup, and the launch lasts as long as they do (56 us for 768 tiles, 71 us for 800). The last
    // tiles of the tile order (positions >= tail_first) are instead each shared out along K over
    // 1 << tail_shift workgroups, whose partial tiles ([tile][share][BM x BN] in `partial`)
    // splitk_tail_reduce_kernel adds. tail_first == tiles_m * tiles_n: none. Never with splits > 1.
    int tail_first, tail_shift;
};

// Position in the tile order -> (row block, n tile over all products): panels of `panel` n tiles,
// inside a panel row block after row block.
__host__ __device__ __forceinline__ void tile_in_order(const AsyncBatch& g, int idx, int* tm, int* tn) {
    const int per_panel = g.tiles_m * g.panel;
    const int last = (g.tiles_n - 1) / g.panel;
    int pnl = idx / per_panel;
    pnl = pnl < last ? pnl : last;
    const int rem = idx - pnl * per_panel;
    const int width = pnl == last ? g.tiles_n - last * g.panel : g.panel;
    *tm = rem / width;
    *tn = pnl * g.panel + rem % width;
}

template <int NSEG, typename T>
__device__ __forceinline__ T seg_pick(const T (&v)[NSEG], int s) {
    if constexpr (NSEG == 1) return v[0];
    else if constexpr (NSEG == 2) return s == 0 ? v[0] : v[1];
    else return s == 0 ? v[0] : (s == 1 ? v[1] : v[2]);
}

// out = (add +) sum over the K shares, in share order. One thread per 4 outputs;
// blockIdx.y = product of the batch.
struct SplitReduceArgs {
    const float* partial[kAsyncMaxProb];
    const float* add[kAsyncMaxProb];
    float* out[kAsyncMaxProb];
    long n4[kAsyncMaxProb];  // M * N / 4
    int splits;
};

__global__ __launch_bounds__(256) void splitk_reduce_kernel(SplitReduceArgs a) {
    const int pi = blockIdx.y;
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.n4[pi]) return;
    const float4* src = reinterpret_cast<const float4*>(a.partial[pi]) + i;
    const long n4 = a.n4[pi];
    const int splits = a.splits;
    float4 v = a.add[pi] ? reinterpret_cast<const float4*>(a.add[pi])[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    // four shares' loads in flight at a time (a share past the end re-reads the last one and is not added)
    for (int s0 = 0; s0 < splits; s0 += 4) {
        float4 t[4];
#pragma unroll
        for (int u = 0; u < 4; u++) t[u] = src[(long)(s0 + u < splits ? s0 + u : splits - 1) * n4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (s0 + u < splits) {
                v.x += t[u].x;
                v.y += t[u].y;
                v.z += t[u].z;
                v.w += t[u].w;
            }
        }
    }
    reinterpret_cast<float4*>(a.out[pi])[i] = v;
}

// The shares of one tail tile (64 x 64), added in share order (after the residual): one workgroup of 1024
// threads per tile, a thread per four consecutive columns with the loads of all shares in flight at once.
__global__ __launch_bounds__(1024) void splitk_tail_reduce_kernel(AsyncBatch g) {
    int tm, tn;
    tile_in_order(g, g.tail_first + (int)blockIdx.x, &tm, &tn);
    int pi = 0;
    if (g.count > 1 && tn >= g.p[1].tile_begin) pi = 1;
    if (g.count > 2 && tn >= g.p[2].tile_begin) pi = 2;
    const AsyncProb& p = g.p[pi];
    const int m0 = tm * 64, n0 = (tn - p.tile_begin) * 64;
    const int shares = 1 << g.tail_shift;
    const int row = threadIdx.x / 16, col = (threadIdx.x % 16) * 4;
    if (m0 + row >= g.M || n0 + col >= p.N) return;  // N is a multiple of 4 on this path
    const float* src = g.partial + ((long)blockIdx.x << g.tail_shift) * 4096 + row * 64 + col;
    float4 t[8];
#pragma unroll
    for (int sh = 0; sh < 8; sh++) t[sh] = *reinterpret_cast<const float4*>(src + (sh < shares ? sh : shares - 1) * 4096);
    const long o = (long)(m0 + row) * p.ldc + n0 + col;
    float4 v = p.add ? *reinterpret_cast<const float4*>(p.add + o) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int sh = 0; sh < 8; sh++) {
        if (sh < shares) {
            v.x += t[sh].x;
            v.y += t[sh].y;
            v.z += t[sh].z;
            v.w += t[sh].w;
        }
    }
    *reinterpret_cast<float4*>(p.out + o) = v;
}

// Output elements leave with the non-temporal hint: nobody in this launch reads them again, and
// lines that do not linger dirty in L2 shorten the write-back at the end of the kernel
// (0.5-1 us per launch, measured).
template <typename P>
__device__ __forceinline__ void store_streaming(P* dst, float v) { __builtin_nontemporal_store(v, dst); }

typedef ft_global_f GlobalF;
typedef float CosSin __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(1))) CosSin GlobalF2;
template <typename T>
__device__ __forceinline__ T pinned(T v) {
    return ft_pinned(v);
}

// KW = 2: eight waves; a stage holds two consecutive K tiles and waves 4-7 multiply the second
// one of every stage for the same 64x64 output tile (the two sums meet in LDS after the loop):
// twice the waves per SIMD for products whose tiles leave a CU with at most two workgroups.
template <int BM, int BN, int WM, int WN, int LAYOUT, int NSEG, int EPI = kEpiPlain, int KW = 1>
__global__ __launch_bounds__(256 * KW) void gemm_async_kernel(AsyncBatch g) {
    static_assert(LAYOUT == 0 || LAYOUT == 1, "a is k-contiguous on this path");
    static_assert(NSEG == 1 || NSEG == kAsyncMaxSeg, "one segment, or the general case");
    static_assert(EPI == kEpiPlain || NSEG == 1, "fused epilogues take one segment");
    constexpr int NST = 3;
    constexpr int NB = EPI == kEpiGateUp ? 2 : 1;  // b matrices multiplied against the same a tile
    constexpr int FM = WM / 32, FN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    static_assert((BM / WM) * (BN / WN) == 4, "4 waves per workgroup");
    constexpr int A_FLOATS = BM * 32;             // f32 tile
    constexpr int B_FLOATS = BN * 16;             // f16 tile, in float units
    constexpr int SUB = A_FLOATS + NB * B_FLOATS;  // one K tile of 32
    constexpr int STAGE = KW * SUB;
    static_assert(KW == 1 || (KW == 2 && BM == 64 && BN == 64), "K-sharing waves: 64x64 tiles");
    constexpr int A_CH = BM / 8 / 4;              // 1 KiB chunks per wave
    constexpr int B_CH = BN / 16 / 4;
    constexpr int LPT = A_CH + NB * B_CH;         // load instructions per wave per tile
    constexpr int WAIT = (NST - 2) * LPT;         // loads that may still be in flight when tile t is needed
    using ExA = FastTile<BM, true, 16>;
    using ExB = FastTile<BN, LAYOUT == 1, 16>;

    __shared__ __attribute__((aligned(16))) float St0[STAGE];
    __shared__ __attribute__((aligned(16))) float St1[STAGE];
    __shared__ __attribute__((aligned(16))) float St2[STAGE];
    // The rank-r products' operand tiles take the first stage's place once the K loop is over:
    // a stage set of their own would cost the 128x128 tile its second workgroup per CU.
    static_assert(ExA::LDS_FLOATS % 4 == 0 && ExA::LDS_FLOATS + ExB::LDS_FLOATS <= STAGE, "rank-r tiles fit a stage");
    float* const ExAs = St0;
    float* const ExBs = St0 + ExA::LDS_FLOATS;

    // Workgroup -> tile. The products of a batch form one row of n tiles per row block
    // (tile_begin = a product's first n tile). Tile order: panels of `panel` n tiles; inside a
    // panel row block after row block. Consecutive workgroup ids go to different XCDs, each with
    // its own L2: XCD x takes the x-th contiguous chunk of that order, so the workgroups resident
    // on one XCD cover a compact block of rows and columns and share their operand tiles in L2.
    // The scalars of the argument block this workgroup needs are fetched in two batches (the header,
    // then the product's entry) and pinned in registers. Left to itself the compiler fetches each of them
    // again in front of every use (a scalar load and a full wait per element of the epilogue loops),
    // which held every workgroup of a launch for microseconds before its first tile request.
    // (All the reads first, then all the pins: a pin waits for its value, and a wait in front of a
    // later read would make two round trips of one.)
    const int r_xcds = g.xcds, r_tail_first = g.tail_first, r_tail_shift = g.tail_shift, r_tiles_m = g.tiles_m,
              r_tiles_n = g.tiles_n, r_panel = g.panel, r_count = g.count, r_splits = g.splits,
              r_begin1 = g.p[1].tile_begin, r_begin2 = g.p[2].tile_begin, r_M = g.M;
    float* const r_partial = g.partial;
    // (The pointers are device memory: saying so keeps their loads and stores `global_*` instructions
    // once the pinning has hidden where they came from.)
    struct SegRegs {
        const char* a;
        const char* b;
        const float* a2;
        int lda, ldb, nt;
    };
    struct ProbRegs {
        const AsyncSeg* seg;
        GlobalF* out;
        const GlobalF* add;
        const void* b_alt;
        GlobalF* out2;
        GlobalF* out3;
        const GlobalF* e1;
        const GlobalF* e2;
        int N, ldc, tile_begin, nseg;
        long partial_off;
        const GlobalF2* rope;
        int rope_seq;
        SegRegs sr[NSEG];
    };
    struct RawProb {
        float* out;
        const float* add;
        const void* b_alt;
        float* out2;
        float* out3;
        const float* e1;
        const float* e2;
        int N, ldc, tile_begin, nseg;
        long partial_off;
        const float2* rope;
        int rope_seq;
        const void* sa[NSEG];
        const void* sb[NSEG];
        const float* sa2[NSEG];
        int slda[NSEG], sldb[NSEG], snt[NSEG];
    };
    auto read_prob = [&](const AsyncProb& pk) {
        RawProb q{pk.out, pk.add, pk.b_alt, pk.out2, pk.out3, pk.e1, pk.e2, pk.N, pk.ldc, pk.tile_begin, pk.nseg,
                  pk.partial_off, pk.rope, pk.rope_seq, {}, {}, {}, {}, {}, {}};
#pragma unroll
        for (int s = 0; s < NSEG; s++) {  // every slot is read (unused ones are zero), so the offsets are constants
            const AsyncSeg& sg = pk.seg[s];
            q.sa[s] = sg.a;
            q.sb[s] = sg.b;
            q.sa2[s] = sg.a2;
            q.slda[s] = sg.lda;
            q.sldb[s] = sg.ldb;
            q.snt[s] = sg.nt;
        }
        return q;
    };
    auto pin_prob = [&](const AsyncProb& pk, const RawProb& r) {
        ProbRegs q{pk.seg,
                   (GlobalF*)pinned(r.out),
                   (const GlobalF*)pinned(r.add),
                   EPI == kEpiGateUp ? pinned(r.b_alt) : nullptr,
                   EPI != kEpiPlain ? (GlobalF*)pinned(r.out2) : nullptr,
                   EPI == kEpiGateUp ? (GlobalF*)pinned(r.out3) : nullptr,
                   EPI == kEpiSiluBwd ? (const GlobalF*)pinned(r.e1) : nullptr,
                   EPI == kEpiSiluBwd ? (const GlobalF*)pinned(r.e2) : nullptr,
                   pinned(r.N),
                   pinned(r.ldc),
                   pinned(r.tile_begin),
                   pinned(r.nseg),
                   pinned(r.partial_off),
                   (const GlobalF2*)pinned(r.rope),
                   pinned(r.rope_seq),
                   {}};
#pragma unroll
        for (int s = 0; s < NSEG; s++)
            q.sr[s] = SegRegs{reinterpret_cast<const char*>(pinned(r.sa[s])), reinterpret_cast<const char*>(pinned(r.sb[s])),
                              pinned(r.sa2[s]), pinned(r.slda[s]), pinned(r.sldb[s]), pinned(r.snt[s])};
        return q;
    };
    // The first product's entry sits at a constant offset: it is fetched with the header, and only a
    // workgroup of a later product of the batch pays a second round trip to the argument block.
    const RawProb raw0 = read_prob(g.p[0]);
    const int g_xcds = pinned(r_xcds), g_tail_first = pinned(r_tail_first), g_tail_shift = pinned(r_tail_shift);
    const int g_tiles_m = pinned(r_tiles_m), g_tiles_n = pinned(r_tiles_n), g_panel = pinned(r_panel);
    const int g_count = pinned(r_count), g_splits = pinned(r_splits);
    const int begin1 = pinned(r_begin1), begin2 = pinned(r_begin2);
    const int M = pinned(r_M);
    GlobalF* const g_partial = (GlobalF*)pinned(r_partial);
    ProbRegs p = pin_prob(g.p[0], raw0);
    int bid = (int)blockIdx.x;
    // A workgroup past the whole tiles takes one K share of a tail tile (uniform per workgroup).
    const bool tail = bid >= g_tail_first;
    int tail_share = 0;
    if (tail) {
        const int u = bid - g_tail_first;
        tail_share = u & ((1 << g_tail_shift) - 1);
        bid = g_tail_first + (u >> g_tail_shift);
    } else if (g_xcds == 8) {  // (8 or 1: shifts instead of divisions on the way to the first tile request)
        const int total = g_tail_first;  // the whole tiles: all of them when there is no tail
        const int x = bid & 7, q = total >> 3, r = total & 7;
        bid = x * q + (x < r ? x : r) + (bid >> 3);
    }
    int tm, tn;
    {
        const int per_panel = g_tiles_m * g_panel;
        const int last = (g_tiles_n - 1) / g_panel;
        int pnl = bid / per_panel;
        pnl = pnl < last ? pnl : last;
        const int rem = bid - pnl * per_panel;
        const int width = pnl == last ? g_tiles_n - last * g_panel : g_panel;
        tm = rem / width;
        tn = pnl * g_panel + rem % width;
    }
    int pi = 0;
    if (g_count > 1 && tn >= begin1) pi = 1;
    if (g_count > 2 && tn >= begin2) pi = 2;
    if (pi != 0) p = pin_prob(g.p[pi], read_prob(g.p[pi]));
    const int m0 = tm * BM;
    const int n0 = (tn - p.tile_begin) * BN;
    const int lane = threadIdx.x % 64, wave = (threadIdx.x / 64) % 4;
    const int grp = KW == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x / 256));  // wave-uniform
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l32 = lane % 32, half = lane / 32;

    floatx16 acc[FM][FN * NB];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN * NB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Uniform description of the segments (a missing one repeats the last: never reached).
    const char* abase[NSEG];
    const char* bbase[NSEG];
    int lda_b[NSEG], ldb_b[NSEG], tend[NSEG];
    bool has_ext[NSEG];
#pragma unroll
    for (int s = 0; s < NSEG; s++) {
        const SegRegs& sg = p.sr[s < p.nseg ? s : 0];
        abase[s] = sg.a;
        bbase[s] = sg.b;
        lda_b[s] = sg.lda * 4;
        ldb_b[s] = sg.ldb * 2;
        tend[s] = (s > 0 ? tend[s - 1] : 0) + (s < p.nseg ? sg.nt : 0);
        has_ext[s] = NB == 1 && grp == 0 && s < p.nseg && sg.a2 != nullptr;
    }
    const char* balt = reinterpret_cast<const char*>(p.b_alt);
    // This workgroup's share of the K tiles: [t0, nt).
    // (KW = 2: counted in pairs of tiles; the host only chooses it when every segment has an even number.)
    const int nt_all = tend[NSEG - 1] / KW;
    const int split = tail ? tail_share : (int)blockIdx.y;
    const int nsplit = tail ? 1 << g_tail_shift : g_splits;
    // (32-bit: at most 2^15 K tiles and 8 shares; most launches have one share)
    const int t0 = nsplit == 1 ? 0 : (int)((unsigned)(nt_all * split) / (unsigned)nsplit);
    const int nt = nsplit == 1 ? nt_all : (int)((unsigned)(nt_all * (split + 1)) / (unsigned)nsplit);
    if (split > 0) {
#pragma unroll
        for (int s = 0; s < NSEG; s++) has_ext[s] = false;  // the rank-r term is added once, by share 0
    }

    // Per-lane source coordinates: byte offset = row * (leading dimension in
    // bytes) + col. The products are formed once per segment (offA / offB), so
    // the K loop itself carries no per-lane address arithmetic.
    unsigned rowA[A_CH], colA[A_CH], rowB[B_CH], colB[B_CH], offA[A_CH], offB[B_CH];
#pragma unroll
    for (int j = 0; j < A_CH; j++) {
        const int c = wave + 4 * j, r = lane / 8, cs = lane % 8;
        int row = m0 + 8 * c + r;
        row = row < M ? row : M - 1;
        rowA[j] = (unsigned)row;
        colA[j] = (unsigned)((cs ^ ((4 * c + (r >> 1)) & 7)) * 16);
        offA[j] = rowA[j] * (unsigned)lda_b[0] + colA[j];
    }
#pragma unroll
    for (int j = 0; j < B_CH; j++) {
        const int c = wave + 4 * j;
        if constexpr (LAYOUT == 1) {
            const int r = lane / 4, cs = lane % 4;
            int n = n0 + 16 * c + r;
            n = n < p.N ? n : p.N - 1;
            rowB[j] = (unsigned)n;
            colB[j] = (unsigned)((cs ^ ((r >> 2) & 3)) * 16);
        } else {
            constexpr int LPR = BN / 8, RPC = 64 / LPR;
            const int kr = lane / LPR, cs = lane % LPR;
            int col = n0 + cs * 8;
            col = col + 8 <= p.N ? col : p.N - 8;
            rowB[j] = (unsigned)(c * RPC + kr);
            colB[j] = (unsigned)(col * 2);
        }
        offB[j] = rowB[j] * (unsigned)ldb_b[0] + colB[j];
    }
    int seg_cur = 0;           // segment the offsets are formed for
    int seg_first = 0;         // its first tile
    const char* aseg = abase[0];
    const char* bseg = bbase[0];
    long b_step = LAYOUT == 1 ? 64L : 32L * ldb_b[0];  // bytes per K tile

    auto issue = [&](int t, float* st) {
        t = t < nt ? t : nt - 1;  // past the end: re-read the last tile into a stage nobody reads
        t = KW * t + grp;         // this wave group's tile of the pair
        st += grp * SUB;
        if constexpr (NSEG > 1) {
            int s = 0;
            if (t >= tend[0]) s = 1;
            if (t >= tend[1]) s = 2;
            if (s != seg_cur) {  // uniform, taken once per segment
                seg_cur = s;
                seg_first = s == 1 ? tend[0] : tend[1];
                const int la = seg_pick<NSEG>(lda_b, s), lb = seg_pick<NSEG>(ldb_b, s);
                aseg = seg_pick<NSEG>(abase, s);
                bseg = seg_pick<NSEG>(bbase, s);
                b_step = LAYOUT == 1 ? 64L : 32L * lb;
#pragma unroll
                for (int j = 0; j < A_CH; j++) offA[j] = rowA[j] * (unsigned)la + colA[j];
#pragma unroll
                for (int j = 0; j < B_CH; j++) offB[j] = rowB[j] * (unsigned)lb + colB[j];
            }
        }
        const int tl = t - seg_first;
        const char* at = aseg + (long)tl * 128;
        const char* bt = bseg + (long)tl * b_step;
#pragma unroll
        for (int j = 0; j < A_CH; j++) glds16(at, offA[j], st + (wave + 4 * j) * 256);
#pragma unroll
        for (int j = 0; j < B_CH; j++) glds16(bt, offB[j], st + A_FLOATS + (wave + 4 * j) * 256);
        if constexpr (NB == 2) {
            const char* bt2 = balt + (long)tl * b_step;
#pragma unroll
            for (int j = 0; j < B_CH; j++) glds16(bt2, offB[j], st + A_FLOATS + B_FLOATS + (wave + 4 * j) * 256);
        }
    };
    auto a_frag = [&](const float* st, int s, int row) -> float4 {
        const int kq = 2 * s + half;
        return *reinterpret_cast<const float4*>(st + row * 32 + ((kq ^ ((row >> 1) & 7)) * 4));
    };
    auto b_frag = [&](const float* st, int s, int n, int jb) -> float4 {
        const char* bs = reinterpret_cast<const char*>(st + A_FLOATS + jb * B_FLOATS);
        if constexpr (LAYOUT == 1) {
            const int kq = 2 * s + half;
            const int col = (kq >> 1) ^ ((n >> 2) & 3);
            const half4_t h = *reinterpret_cast<const half4_t*>(bs + n * 64 + col * 16 + (kq & 1) * 8);
            return make_float4((float)h.x, (float)h.y, (float)h.z, (float)h.w);
        } else {
            const _Float16* q = reinterpret_cast<const _Float16*>(bs) + (8 * s + 4 * half) * BN + n;
            return make_float4((float)q[0], (float)q[BN], (float)q[2 * BN], (float)q[3 * BN]);
        }
    };
    auto mfma_step = [&](const float4 (&af)[FM], const float4 (&bf)[FN * NB]) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN * NB; j++) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].x, bf[j].x, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].y, bf[j].y, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].z, bf[j].z, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].w, bf[j].w, acc[i][j], 0, 0, 0);
            }
    };
    // The K loop, rotated by three quarters of a tile: the wait for tile t + 1, the barrier, the
    // refill of the stage tile t has just left and the first fragment reads of tile t + 1 all sit
    // in front of the LAST group of MFMAs of tile t, so a wave comes out of the barrier with 4 MFMAs
    // still to issue while its first reads of the new tile are in flight (with the barrier at the
    // top of a tile every wave of the workgroup met that LDS latency at the same moment).
    float4 af[2][FM], bf[2][FN * NB];
    auto read_frags = [&](const float* cur, int s, int buf) {
#pragma unroll
        for (int i = 0; i < FM; i++) af[buf][i] = a_frag(cur, s, wm0 + i * 32 + l32);
#pragma unroll
        for (int j = 0; j < FN * NB; j++) bf[buf][j] = b_frag(cur, s, wn0 + (j % FN) * 32 + l32, j / FN);
    };
    // Tile t: `stage` holds it, `next` holds tile t + 1; fragments of its first k-quads are in af[0] / bf[0].
    auto iter = [&](int t, float* stage, const float* next) {
        const float* cur = stage + grp * SUB;
#pragma unroll
        for (int s = 0; s < 3; s++) {
            read_frags(cur, s + 1, (s + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_step(af[s & 1], bf[s & 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // This wave's reads of the stage are complete (lgkmcnt 0) and tile t + 1 has landed (at
        // most tile t + 2's loads in flight); after the barrier that holds for every wave, so
        // the stage can take tile t + 3.
        __builtin_amdgcn_s_waitcnt(0x0070 | (WAIT & 15) | ((WAIT >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        issue(t + NST, stage);
        read_frags(next + grp * SUB, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_step(af[1], bf[1]);
        __builtin_amdgcn_sched_barrier(0);
    };

    // Prologue: tiles t0 .. t0+2 requested, the first one landed, its first fragments read.
    issue(t0, St0);
    issue(t0 + 1, St1);
    // Epilogue operands (the residual of `out = a@b + add`, gate and up of the SiLU-gate backward,
    // the rotation's cos and sin) are requested here, behind the first two tiles and in front of the
    // K loop: after the last MFMA their latency would be paid when the workgroups of a CU all finish
    // together. The loop's vmcnt waits cover them (they are older than every later tile request).
    // Out-of-range elements read element 0 instead of branching around the load.
    constexpr bool PRE = BM == 64 && BN == 64 && NSEG == 1 && (EPI == kEpiPlain || EPI == kEpiSiluBwd);
    float2 pre[PRE ? 16 : 1];  // plain: .x = residual, or (cos, sin); SiLU backward: (gate, up)
    bool pre_add = false;
    if constexpr (PRE) {
        const GlobalF* s1 = EPI == kEpiSiluBwd ? p.e1 : p.add;
        pre_add = grp == 0 && (EPI == kEpiSiluBwd || (p.add != nullptr && g_splits == 1 && !tail && p.rope == nullptr));
        bool rotated = false;
        if constexpr (EPI == kEpiPlain) rotated = p.rope != nullptr;
        if (rotated) {  // the rotation's (cos, sin) of this lane's 16 rows (never together with a residual)
            const int pos0 = (m0 + wm0 + half * 4) % p.rope_seq;  // one division; the rows follow by steps < 64
#pragma unroll
            for (int r = 0; r < 16; r++) {
                int pos = pos0 + (r / 4) * 8 + (r % 4);
                if (pos >= p.rope_seq) pos -= p.rope_seq;
                if (pos >= p.rope_seq) pos %= p.rope_seq;  // sequences shorter than a tile
                const CosSin cs = p.rope[(long)pos * 32 + l32];
                pre[r] = make_float2(cs.x, cs.y);
            }
        } else if (pre_add) {
            const int col = n0 + wn0 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm0 + (r / 4) * 8 + half * 4 + (r % 4);
                const long o = row < M && col < p.N ? (long)row * p.ldc + col : 0;
                pre[r].x = s1[o];
                if constexpr (EPI == kEpiSiluBwd) pre[r].y = p.e2[o];
            }
        }
    }

    // The rank-r products' operands: ordinary loads, consumed last.
    ExA xa[NSEG];
    ExB xb[NSEG];
#pragma unroll
    for (int s = 0; s < NSEG; s++) {
        if (has_ext[s]) {
            const AsyncSeg& sg = p.seg[s];
            xa[s].set_offsets(sg.lda2, m0, M, 4);
            xb[s].set_offsets(sg.ldb2, n0, p.N, 4);
            xa[s].template load<float, true>(reinterpret_cast<const char*>(sg.a2), 0, sg.K2);
            xb[s].template load<float, true>(reinterpret_cast<const char*>(sg.b2), 0, sg.K2);
        }
    }

    __builtin_amdgcn_s_waitcnt(0x0F70 | (WAIT & 15) | ((WAIT >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    issue(t0 + 2, St2);
    read_frags(St0 + grp * SUB, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    for (int t = t0; t < nt; t += NST) {
        iter(t, St0, St1);
        if (t + 1 < nt) iter(t + 1, St1, St2);
        if (t + 2 < nt) iter(t + 2, St2, St0);
    }

    if constexpr (KW == 2) {
        // The second wave group hands its sums over through the second stage and retires.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();  // loads landed, every wave has left the last stage
        static_assert(KW == 1 || FN * NB * 16 * 256 <= STAGE, "the hand-over fits a stage");
        float* red = St1 + wave * 64 + lane;
        if (grp == 1) {
#pragma unroll
            for (int j = 0; j < FN * NB; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) red[(j * 16 + r) * 256] = acc[0][j][r];
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int j = 0; j < FN * NB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[0][j][r] += red[(j * 16 + r) * 256];
    }
#pragma unroll
    for (int s = 0; s < NSEG; s++) {
        if (has_ext[s]) {  // never with two b matrices
            // The stage is free when every wave's loads have landed and every wave has left the
            // last K tile (or the previous segment's rank-r tile).
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            xa[s].template store<float>(ExAs);
            xb[s].template store<float>(ExBs);
            __syncthreads();
#pragma unroll
            for (int st = 0; st < 2; st++) {
                float4 af[FM], bf[FN * NB];
#pragma unroll
                for (int i = 0; i < FM; i++) af[i] = ExA::frag(ExAs, st, half, wm0 + i * 32 + l32);
#pragma unroll
                for (int j = 0; j < FN * NB; j++) bf[j] = ExB::frag(ExBs, st, half, wn0 + (j % FN) * 32 + l32);
                mfma_step(af, bf);
            }
        }
    }
    // Nothing may still be landing in LDS when the workgroup retires.
    __builtin_amdgcn_s_waitcnt(0x0F70);

    if constexpr (EPI == kEpiPlain && BM == 64 && BN == 64) {
        if (p.rope) {  // uniform per workgroup; never together with split-K
            // The partner column (+-32) belongs to the neighbouring wave: exchange through the
            // stage memory (free now: every wave has waited for its own loads, the barrier makes
            // that true of all of them).
            __syncthreads();
            float* mine = (wave < 2 ? St0 : St1) + (wave & 1) * 1024;
            const float* other = (wave < 2 ? St0 : St1) + ((wave & 1) ^ 1) * 1024;
#pragma unroll
            for (int r = 0; r < 16; r++) mine[r * 64 + lane] = acc[0][0][r];
            __syncthreads();
            const int col = n0 + wn0 + l32;
            const bool upper = wn0 != 0;  // this wave holds i + 32
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm0 + (r / 4) * 8 + half * 4 + (r % 4);
                if (row < M && col < p.N) {
                    float2 cs;
                    if constexpr (PRE) {
                        cs = pre[r];
                    } else {
                        const CosSin t = p.rope[(long)(row % p.rope_seq) * 32 + l32];
                        cs = make_float2(t.x, t.y);
                    }
                    const float self = acc[0][0][r], peer = other[r * 64 + lane];
                    // lower: x1*c - x2*s ; upper: x1*s + x2*c  (x1 = lower half, x2 = upper half)
                    p.out[(long)row * p.ldc + col] = upper ? peer * cs.y + self * cs.x : self * cs.x - peer * cs.y;
                }
            }
            return;
        }
    }

    // What becomes of a finished element is the same for the whole workgroup: chosen once, outside the loops.
    auto emit_all = [&](auto&& emit) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++) {
                const int col = n0 + wn0 + j * 32 + l32;
                if (col >= p.N) continue;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm0 + i * 32 + (r / 4) * 8 + half * 4 + (r % 4);
                    if (row < M) emit(i, j, r, row, col);
                }
            }
    };
    if constexpr (EPI == kEpiGateUp) {
        emit_all([&](int i, int j, int r, int row, int col) {
            const long o = (long)row * p.ldc + col;
            const float up = acc[i][j][r], x = acc[i][FN + j][r];
            store_streaming(&p.out[o], up);
            store_streaming(&p.out2[o], x);
            store_streaming(&p.out3[o], x * (1.0f / (1.0f + __expf(-x))) * up);
        });
    } else if constexpr (EPI == kEpiSiluBwd) {
        emit_all([&](int i, int j, int r, int row, int col) {
            const long o = (long)row * p.ldc + col;
            const float d = acc[i][j][r], x = pre[r].x, y = pre[r].y;
            const float sg = 1.0f / (1.0f + __expf(-x));
            store_streaming(&p.out2[o], d * (x * sg));
            store_streaming(&p.out[o], d * y * (sg * (1.0f + x * (1.0f - sg))));
        });
    } else if (tail) {
        GlobalF* dst = g_partial + ((((long)(bid - g_tail_first)) << g_tail_shift) + split) * (BM * BN);
        emit_all([&](int i, int j, int r, int row, int col) { dst[(row - m0) * BN + (col - n0)] = acc[i][j][r]; });
    } else if (g_splits > 1) {
        GlobalF* dst = g_partial + p.partial_off + (long)split * M * p.N;
        emit_all([&](int i, int j, int r, int row, int col) { dst[(long)row * p.N + col] = acc[i][j][r]; });
    } else if (PRE && pre_add) {
        emit_all([&](int i, int j, int r, int row, int col) {
            store_streaming(&p.out[(long)row * p.ldc + col], acc[i][j][r] + pre[PRE ? r : 0].x);
        });
    } else if (p.add) {
        emit_all([&](int i, int j, int r, int row, int col) {
            const long o = (long)row * p.ldc + col;
            store_streaming(&p.out[o], acc[i][j][r] + p.add[o]);
        });
    } else {
        emit_all([&](int i, int j, int r, int row, int col) {
            store_streaming(&p.out[(long)row * p.ldc + col], acc[i][j][r]);
        });
    }
}

// ---------------------------------------------------------------------------
// f32 x f32 on the same pipeline (global -> LDS DMA, three stages, explicit
// waits): the plain matmul / matmul_bt / matmul_at of the engine, where b is an
// f32 tensor. An operand tile is either
//   KC  k-contiguous in memory (a[M,K]; b[N,K]): [64 rows][32 k], 128 B per row,
//       swizzled as in gemm_async_kernel, one ds_read_b128 per k-quad, or
//   KM  k-major (a[K,M] of matmul_at; b[K,N]): [32 k][64] exactly as in memory
//       (4 k rows per DMA instruction), four ds_read_b32 per k-quad.
// 64x64 tiles, 32x32 per wave; K a multiple of 32, M / N multiples of 4 where an
// operand is KM. Tile order as in gemm_async_kernel.
// ---------------------------------------------------------------------------
struct F32AsyncArgs {
    const float* a;
    const float* b;
    float* out;
    int M, N, nt;        // nt = K / 32
    int lda, ldb, ldc;
    int tiles_m, tiles_n, xcds, panel;
    int splits;          // shares of the K tiles (blockIdx.y); > 1: partial tiles go to `partial` [splits][M][N]
    float* partial;
};

template <bool A_KM, bool B_KM>
__global__ __launch_bounds__(256) void gemm_f32_async_kernel(F32AsyncArgs g) {
    constexpr int NST = 3, TILE = 64 * 32, STAGE = 2 * TILE;
    constexpr int LPT = 4;                         // 2 + 2 load instructions per wave per K tile
    __shared__ __attribute__((aligned(16))) float St0[STAGE];
    __shared__ __attribute__((aligned(16))) float St1[STAGE];
    __shared__ __attribute__((aligned(16))) float St2[STAGE];
    int bid = (int)blockIdx.x;
    if (g.xcds > 1) {
        const int total = (int)gridDim.x, x = bid % g.xcds, q = total / g.xcds, r = total % g.xcds;
        bid = x * q + (x < r ? x : r) + bid / g.xcds;
    }
    const int per_panel = g.tiles_m * g.panel;
    const int last = (g.tiles_n - 1) / g.panel;
    int pnl = bid / per_panel;
    pnl = pnl < last ? pnl : last;
    const int rem = bid - pnl * per_panel;
    const int width = pnl == last ? g.tiles_n - last * g.panel : g.panel;
    const int m0 = (rem / width) * 64, n0 = (pnl * g.panel + rem % width) * 64;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int wm0 = (wave / 2) * 32, wn0 = (wave % 2) * 32;
    const int l32 = lane % 32, half = lane / 32;

    // Per-lane byte offsets of the two DMA instructions a wave issues per operand and K tile.
    unsigned offA[2], offB[2];
    auto offsets = [&](bool km, int base0, int extent, int ld, unsigned (&off)[2]) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int c = wave + 4 * j;  // chunk of 1 KiB
            if (km) {
                const int kr = lane / 16, cs = lane % 16;
                int col = base0 + cs * 4;
                col = col + 4 <= extent ? col : extent - 4;
                off[j] = (unsigned)(4 * c + kr) * (unsigned)ld * 4u + (unsigned)col * 4u;
            } else {
                const int r = lane / 8, cs = lane % 8;
                int row = base0 + 8 * c + r;
                row = row < extent ? row : extent - 1;
                off[j] = (unsigned)row * (unsigned)ld * 4u + (unsigned)((cs ^ ((4 * c + (r >> 1)) & 7)) * 16);
            }
        }
    };
    offsets(A_KM, m0, g.M, g.lda, offA);
    offsets(B_KM, n0, g.N, g.ldb, offB);
    const long a_step = A_KM ? 32L * g.lda * 4 : 128L, b_step = B_KM ? 32L * g.ldb * 4 : 128L;
    const char* abase = reinterpret_cast<const char*>(g.a);
    const char* bbase = reinterpret_cast<const char*>(g.b);
    // This workgroup's share of the K tiles: [t0, nt).
    const int split = (int)blockIdx.y;
    const int t0 = (int)(((long)g.nt * split) / g.splits);
    const int nt = (int)(((long)g.nt * (split + 1)) / g.splits);
    auto issue = [&](int t, float* st) {
        t = t < nt ? t : nt - 1;  // past the end: re-read the last tile into a stage nobody reads
        const char* at = abase + (long)t * a_step;
        const char* bt = bbase + (long)t * b_step;
#pragma unroll
        for (int j = 0; j < 2; j++) glds16(at, offA[j], st + (wave + 4 * j) * 256);
#pragma unroll
        for (int j = 0; j < 2; j++) glds16(bt, offB[j], st + TILE + (wave + 4 * j) * 256);
    };
    auto frag = [&](const float* tile, bool km, int s, int idx) -> float4 {
        const int kq = 2 * s + half;
        if (km) {
            const float* q = tile + (4 * kq) * 64 + idx;
            return make_float4(q[0], q[64], q[128], q[192]);
        }
        return *reinterpret_cast<const float4*>(tile + idx * 32 + ((kq ^ ((idx >> 1) & 7)) * 4));
    };
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    // Rotated like the loop of gemm_async_kernel: wait, barrier, refill and the first fragment
    // reads of tile t + 1 come before the last MFMA group of tile t.
    float4 af[2], bf[2];
    auto iter = [&](int t, float* cur, const float* next) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const int c = s & 1, nx = c ^ 1;
            if (s + 1 < 4) {
                af[nx] = frag(cur, A_KM, s + 1, wm0 + l32);
                bf[nx] = frag(cur + TILE, B_KM, s + 1, wn0 + l32);
            } else {
                // own reads of the stage complete, tile t + 1 landed (tile t + 2 may be in flight)
                __builtin_amdgcn_s_waitcnt(0x0070 | LPT);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                issue(t + NST, cur);
                af[nx] = frag(next, A_KM, 0, wm0 + l32);
                bf[nx] = frag(next + TILE, B_KM, 0, wn0 + l32);
            }
            __builtin_amdgcn_sched_barrier(0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c].x, bf[c].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c].y, bf[c].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c].z, bf[c].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c].w, bf[c].w, acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    issue(t0, St0);
    issue(t0 + 1, St1);
    __builtin_amdgcn_s_waitcnt(0x0F70 | LPT);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    issue(t0 + 2, St2);
    af[0] = frag(St0, A_KM, 0, wm0 + l32);
    bf[0] = frag(St0 + TILE, B_KM, 0, wn0 + l32);
    __builtin_amdgcn_sched_barrier(0);
    for (int t = t0; t < nt; t += NST) {
        iter(t, St0, St1);
        if (t + 1 < nt) iter(t + 1, St1, St2);
        if (t + 2 < nt) iter(t + 2, St2, St0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // nothing may still be landing in LDS when the workgroup retires
    const int col = n0 + wn0 + l32;
    if (col >= g.N) return;
    float* dst = g.splits > 1 ? g.partial + (long)split * g.M * g.N : g.out;
    const int ld = g.splits > 1 ? g.N : g.ldc;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = m0 + wm0 + (r / 4) * 8 + half * 4 + (r % 4);
        if (row < g.M) dst[(long)row * ld + col] = acc[r];
    }
}

// ---------------------------------------------------------------------------
// out[R, C] (C <= 32) = scale * X[R, Kr] @ Y[Kr, C].
//   XT:  X is stored [Kr, R] (element (row,k) at x[k*ldx + row])
//   YT:  Y is stored [C, Kr] (element (k,col) at y[col*ldy + k])
//   OT:  out is stored [C, R]
// One workgroup per 32 rows; wave w reduces k in [w*span, (w+1)*span).
// ---------------------------------------------------------------------------
template <bool XT, bool YT, bool OT>
__global__ __launch_bounds__(256) void skinny_kernel(const float* __restrict__ x, const float* __restrict__ y,
                                                     float* __restrict__ out, int R, int Kr, int C, long ldx,
                                                     long ldy, long ldo, float scale) {
    __shared__ float red[4][32 * 33];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int l32 = lane % 32, half = lane / 32;
    const int r0 = blockIdx.x * 32;
    const int row = r0 + l32;
    const bool row_ok = row < R;
    const bool col_ok = l32 < C;
    // k range of this wave, in steps of 8
    const int steps = (Kr + 7) / 8;
    const int per = (steps + 3) / 4;
    int s_begin = wave * per;
    const int s_end = (s_begin + per < steps) ? s_begin + per : steps;
    if (s_begin > s_end) s_begin = s_end;

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;

    auto load_x = [&](int k) -> float4 {  // X[row][k..k+3]
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (!row_ok) return v;
        if constexpr (!XT) {
            v = load4(x + (long)row * ldx + k, clamp04(Kr - k));
        } else {
            if (k + 0 < Kr) v.x = x[(long)(k + 0) * ldx + row];
            if (k + 1 < Kr) v.y = x[(long)(k + 1) * ldx + row];
            if (k + 2 < Kr) v.z = x[(long)(k + 2) * ldx + row];
            if (k + 3 < Kr) v.w = x[(long)(k + 3) * ldx + row];
        }
        return v;
    };
    auto load_y = [&](int k) -> float4 {  // Y[k..k+3][col]
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (!col_ok) return v;
        if constexpr (YT) {
            v = load4(y + (long)l32 * ldy + k, clamp04(Kr - k));
        } else {
            if (k + 0 < Kr) v.x = y[(long)(k + 0) * ldy + l32];
            if (k + 1 < Kr) v.y = y[(long)(k + 1) * ldy + l32];
            if (k + 2 < Kr) v.z = y[(long)(k + 2) * ldy + l32];
            if (k + 3 < Kr) v.w = y[(long)(k + 3) * ldy + l32];
        }
        return v;
    };

    constexpr int U = 4;
    int s = s_begin;
    for (; s + U <= s_end; s += U) {
        float4 xv[U], yv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = (s + u) * 8 + half * 4;
            xv[u] = load_x(k);
            yv[u] = load_y(k);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u].x, yv[u].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u].y, yv[u].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u].z, yv[u].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u].w, yv[u].w, acc, 0, 0, 0);
        }
    }
    for (; s < s_end; s++) {
        const int k = s * 8 + half * 4;
        const float4 xv = load_x(k), yv = load_y(k);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.x, yv.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.y, yv.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.z, yv.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.w, yv.w, acc, 0, 0, 0);
    }

#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int i = (r / 4) * 8 + half * 4 + (r % 4);
        red[wave][i * 33 + l32] = acc[r];
    }
    __syncthreads();
    auto emit = [&](int i, int j, float v) {
        if (r0 + i < R && j < C) {
            if constexpr (OT)
                out[(long)j * ldo + r0 + i] = v * scale;
            else
                out[(long)(r0 + i) * ldo + j] = v * scale;
        }
    };
    // 1024 outputs, 256 threads: the 4 waves are added in fixed order.
    for (int e = threadIdx.x; e < 32 * 32; e += 256) {
        const int i = e / 32, j = e % 32;
        emit(i, j, ((red[0][i * 33 + j] + red[1][i * 33 + j]) + red[2][i * 33 + j]) + red[3][i * 33 + j]);
    }
}

// ---------------------------------------------------------------------------
// Matrix-pipe probe: v_mfma_f32_32x32x2_f32 on register operands only, no memory
// traffic inside the loop. CHAINS independent accumulators per wave (1 = every
// MFMA depends on the one before, as in a 32x32 wave tile). Measures what the
// matrix pipes sustain, the ceiling the GEMM kernels are compared with.
// ---------------------------------------------------------------------------
template <int CHAINS>
__global__ __launch_bounds__(256) void mfma_probe_kernel(float* __restrict__ out, int rounds, int random_operands) {
    floatx16 acc[CHAINS];
#pragma unroll
    for (int c = 0; c < CHAINS; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = 0.0f;
    // Operands: 16 pairs of pseudo-random values in (-1, 1) per lane, as a GEMM on N(0,1)-like
    // data would feed (the power a matrix pipe draws depends on how many operand bits toggle).
    float a[16], b[16];
    unsigned h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int u = 0; u < 16; u++) {
        h = h * 1664525u + 1013904223u;
        a[u] = random_operands ? (float)(int)(h >> 8) * (1.0f / 8388608.0f) - 1.0f : 1.0f;
        h = h * 1664525u + 1013904223u;
        b[u] = random_operands ? (float)(int)(h >> 8) * (1.0f / 8388608.0f) - 1.0f : 1.0f;
    }
    for (int i = 0; i < rounds; i++) {
#pragma unroll
        for (int u = 0; u < 16 / CHAINS; u++)
#pragma unroll
            for (int c = 0; c < CHAINS; c++)
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u * CHAINS + c], b[u * CHAINS + c], acc[c], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < 16; u++) asm volatile("" : "+v"(a[u]), "+v"(b[u]));  // opaque: nothing to hoist
    }
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < CHAINS; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += acc[c][r];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

constexpr size_t kSplitScratchFloats = (size_t)16 << 20;  // 64 MiB of split-K partial tiles

bool aligned16p(const void* q) { return (((uintptr_t)q) & 15) == 0; }

// XCDs of the device (MI355X: 8 of 32 CUs, each with its own L2).
static int ft_gemm_xcds(ft_context* ctx) { return ctx->num_cus % 8 == 0 && ctx->num_cus >= 64 ? 8 : 1; }

template <int BM, int BN, int WM, int WN>
int launch_async(ft_context* ctx, AsyncBatch g, int layout, int epi = kEpiPlain) {
    const int tiles_m = (g.M + BM - 1) / BM;
    int tiles_n = 0, max_seg = 1;
    double flops = 0.0, bytes = 0.0, a_bytes = 0.0, b_bytes = 0.0;
    for (int i = 0; i < g.count; i++) {
        AsyncProb& p = g.p[i];
        p.tile_begin = tiles_n;
        tiles_n += (p.N + BN - 1) / BN;
        if (p.nseg > max_seg) max_seg = p.nseg;
        double a_this = 0.0;  // the products of a batch share their a operand
        for (int s = 0; s < p.nseg; s++) {
            a_this += 4.0 * g.M * 32.0 * p.seg[s].nt;
            b_bytes += 2.0 * p.N * 32.0 * p.seg[s].nt * (epi == kEpiGateUp ? 2 : 1);
        }
        if (a_this > a_bytes) a_bytes = a_this;
        for (int s = 0; s < p.nseg; s++) {
            const double k = 32.0 * p.seg[s].nt, k2 = p.seg[s].a2 ? (double)p.seg[s].K2 : 0.0;
            flops += 2.0 * g.M * (double)p.N * (k + k2);
            bytes += 4.0 * g.M * (k + k2) + 2.0 * p.N * k + 4.0 * p.N * k2;
        }
        bytes += (p.add ? 8.0 : 4.0) * g.M * (double)p.N;
    }
    const int tiles = tiles_m * tiles_n;
    g.tiles_m = tiles_m;
    g.tiles_n = tiles_n;
    // Panel width: the tiles resident on one XCD at a time (32 CUs x workgroups per CU) should
    // need about as many bytes of a (rows x a_bytes per row block) as of b (columns x b_bytes
    // per n tile).
    g.xcds = ft_gemm_xcds(ctx);
    {
        const double resident = 32.0 * (BM == 64 ? (epi == kEpiGateUp ? 3 : 4) : 2);
        const double a_blk = a_bytes / tiles_m, b_blk = b_bytes / (tiles_n > 0 ? tiles_n : 1);
        int want = b_blk > 0 ? (int)(sqrt(resident * a_blk / b_blk) + 0.5) : tiles_n;
        if (want < 1) want = 1;
        int panels = (int)((double)tiles_n / want + 0.5);
        if (panels < 1) panels = 1;
        g.panel = (tiles_n + panels - 1) / panels;
        if (g.panel < 1) g.panel = 1;
    }
    g.splits = 1;
    g.partial = nullptr;
    // Split-K when the tiles alone cannot occupy the chip and the K loop is long enough to share
    // out (at least 4 K tiles per share): aims at about two workgroups per CU.
    int min_kt = 1 << 30;
    bool mn4 = true;
    size_t out_floats = 0;
    for (int i = 0; i < g.count; i++) {
        int kt = 0;
        for (int s = 0; s < g.p[i].nseg; s++) kt += g.p[i].seg[s].nt;
        if (kt < min_kt) min_kt = kt;
        mn4 = mn4 && ((size_t)g.M * g.p[i].N) % 4 == 0 && g.p[i].ldc == g.p[i].N;
        out_floats += (size_t)g.M * g.p[i].N;
    }
    bool any_rope = false;
    for (int i = 0; i < g.count; i++) any_rope = any_rope || g.p[i].rope != nullptr;
    // Also with fewer than 1.5 tiles per CU when K is very long (the head's input gradient, K = vocabulary):
    // the extra pass over the output is then a fraction of a percent.
    const bool few_tiles = (size_t)tiles * 4 <= (size_t)ctx->num_cus * 5;
    const bool long_k = (size_t)tiles * 2 < 3 * (size_t)ctx->num_cus && min_kt >= 512;
    // Eight waves on a tile (two K tiles per stage, see the kernel) need whole pairs of tiles in every segment.
    bool pairs_ok = BM == 64 && epi == kEpiPlain && !any_rope && min_kt >= 8;
    for (int i = 0; i < g.count && pairs_ok; i++)
        for (int s = 0; s < g.p[i].nseg; s++) pairs_ok = pairs_ok && g.p[i].seg[s].nt % 2 == 0;
    bool pairs = false;
    g.tail_first = tiles;
    g.tail_shift = 0;
    if (BM == 64 && epi == kEpiPlain && tiles > ctx->num_cus && !long_k) {
        // A remainder over the CUs of at most a quarter of them (288 tiles: the 576-column products of the 135M
        // shape; 800: q/k/v at 360M): its tiles (the last of the order) must be plain ones (no RoPE epilogue,
        // whole float4 groups).
        const int cus = ctx->num_cus, tail = tiles % cus;
        // at most 8 shares of at least 3 K tiles each (4 and 8 shares measured alike: 66-68 us against 73)
        // (with eight waves per tile the K tiles are shared out in pairs)
        const bool pairs_here = pairs_ok && (size_t)tiles <= 2 * (size_t)cus && min_kt >= 32;
        const int kt_units = pairs_here ? min_kt / 2 : min_kt;
        int shift = 0;
        while (shift < 3 && (tail << (shift + 1)) <= cus && (kt_units >> (shift + 1)) >= 3) shift++;
        bool ok = tail > 0 && shift >= 2 && (size_t)(tail << shift) * BM * BN <= kSplitScratchFloats;
        auto tail_is_plain = [&]() {
            bool plain = true;
            for (int u = 0; u < tail && plain; u++) {
                int tm, tn;
                tile_in_order(g, tiles - tail + u, &tm, &tn);
                int pi = 0;
                if (g.count > 1 && tn >= g.p[1].tile_begin) pi = 1;
                if (g.count > 2 && tn >= g.p[2].tile_begin) pi = 2;
                const AsyncProb& p = g.p[pi];
                plain = p.rope == nullptr && p.N % 4 == 0 && p.ldc % 4 == 0 && aligned16p(p.out) && aligned16p(p.add);
            }
            return plain;
        };
        if (ok && !tail_is_plain()) {
            // q and k are rotated, v is not: with panels as wide as the last product the order ends in its tiles
            // alone (narrower panels re-read more of a; the launch is matrix-bound).
            const AsyncProb& last = g.p[g.count - 1];
            const int lw = (last.N + BN - 1) / BN;
            const int keep = g.panel;
            ok = g.count > 1 && last.rope == nullptr && lw > 0 && last.tile_begin % lw == 0 && tail <= tiles_m * lw;
            if (ok) {
                g.panel = lw;
                ok = tail_is_plain();
                if (!ok) g.panel = keep;
            }
        }
        if (ok) {
            if (!ctx->gemm_scratch) {
                FT_HIP(hipSetDevice(ctx->device));
                FT_HIP(hipMalloc((void**)&ctx->gemm_scratch, kSplitScratchFloats * sizeof(float)));
            }
            g.tail_first = tiles - tail;
            g.tail_shift = shift;
            g.partial = ctx->gemm_scratch;
        }
    }
    if (g.tail_shift == 0 && epi == kEpiPlain && mn4 && !any_rope && tiles > 0 && (few_tiles || long_k)) {
        int want = (int)((2 * (size_t)ctx->num_cus + tiles - 1) / tiles);
        // A few tiles more than CUs (288 on 256: the 576-column products): with w shares a CU holds
        // ceil(288 w / 256) of them, 2, 3, 4 for w = 1, 2, 3, i.e. 2, 1.5, 1.33 tiles' worth; measured,
        // three shares beat two (and four) in the 135M-shaped step. (Only where the tail split above does not
        // apply: it leaves a CU with one whole tile and an eighth, 15.3 -> 14.9 ms per 135M step.)
        if (BM == 64 && tiles > ctx->num_cus) want = 3;
        // 128x128 tiles hold two workgroups on a CU: the shares must fit one round of them
        if (BM == 128) want = (int)(2 * (size_t)ctx->num_cus / tiles);
        if (want > 8) want = 8;
        if (want > min_kt / 4) want = min_kt / 4;
        // Many shares (one sequence per pass): the second wave group takes half of them, which
        // halves the partial tiles. (Up to five shares are faster as they are: measured.)
        if (want >= 6 && pairs_ok) {
            pairs = true;
            want = (want + 1) / 2;
        }
        if (want >= 2 && out_floats * want <= kSplitScratchFloats) {
            if (!ctx->gemm_scratch) {
                FT_HIP(hipSetDevice(ctx->device));
                FT_HIP(hipMalloc((void**)&ctx->gemm_scratch, kSplitScratchFloats * sizeof(float)));
            }
            g.splits = want;
            g.partial = ctx->gemm_scratch;
            long off = 0;
            for (int i = 0; i < g.count; i++) {
                g.p[i].partial_off = off;
                off += (long)want * g.M * g.p[i].N;
            }
        }
    }
    const dim3 grid((unsigned)(g.tail_first + ((tiles - g.tail_first) << g.tail_shift)), (unsigned)g.splits);
    // A deferred sum is honoured for one plain product with a dense output: its shares are the plain
    // [splits][M][N] arrays, or the partial tiles of a tail split.
    ft_deferred_sum* const defer = ctx->defer;
    ctx->defer = nullptr;
    if (defer) *defer = ft_deferred_sum{};
    auto reduce_shares = [&]() -> int {
        if (g.tail_shift > 0) {
            if (defer && BM == 64 && g.count == 1 && epi == kEpiPlain && g.p[0].ldc == g.p[0].N) {
                defer->partial = g.partial;
                defer->add = g.p[0].add;
                defer->out = g.p[0].out;
                defer->tail_first = g.tail_first;
                defer->tail_shift = g.tail_shift;
                defer->tiles_m = g.tiles_m;
                defer->tiles_n = g.tiles_n;
                defer->panel = g.panel;
                return FT_OK;
            }
            hipLaunchKernelGGL(splitk_tail_reduce_kernel, dim3((unsigned)(tiles - g.tail_first)), dim3(1024), 0,
                               ctx->stream, g);
            FT_LAUNCH_CHECK();
            return FT_OK;
        }
        if (g.splits == 1) return FT_OK;
        if (defer && g.count == 1 && epi == kEpiPlain && g.p[0].ldc == g.p[0].N) {
            defer->partial = g.partial + g.p[0].partial_off;
            defer->add = g.p[0].add;
            defer->stride = (long)g.M * g.p[0].N;
            defer->splits = g.splits;
            return FT_OK;
        }
        SplitReduceArgs ra{};
        long n4max = 0;
        for (int i = 0; i < g.count; i++) {
            ra.partial[i] = g.partial + g.p[i].partial_off;
            ra.add[i] = g.p[i].add;
            ra.out[i] = g.p[i].out;
            ra.n4[i] = (long)g.M * g.p[i].N / 4;
            if (ra.n4[i] > n4max) n4max = ra.n4[i];
        }
        ra.splits = g.splits;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3(ft_div_up((size_t)n4max, 256), (unsigned)g.count), dim3(256), 0,
                           ctx->stream, ra);
        FT_LAUNCH_CHECK();
        return FT_OK;
    };
    char name[96];
    if (epi != kEpiPlain) {
        // both fused forms: one product, one segment, 64x64 tiles (the only instantiation)
        if constexpr (BM == 64) {
            const bool gu = epi == kEpiGateUp;
            snprintf(name, sizeof(name), "gemm_async_kernel<64, 64, 32, 32, %d, 1, %s>", layout,
                     gu ? "gate_up" : "silu_bwd");
            const double mn = (double)g.M * g.p[0].N;
            ft_prof_scope prof(ctx, name, gu ? 2.0 * flops : flops,
                               gu ? bytes + 64.0 * g.p[0].N * g.p[0].seg[0].nt + 8.0 * mn : bytes + 12.0 * mn);
            // Fewer tiles than CUs (one sequence per pass): eight waves share the K loop of a tile.
            const bool few = (size_t)tiles <= (size_t)ctx->num_cus && g.p[0].seg[0].nt % 2 == 0 && g.p[0].seg[0].nt >= 8;
            if (gu && few)
                hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 0, 1, kEpiGateUp, 2>), grid, dim3(512), 0,
                                   ctx->stream, g);
            else if (gu)
                hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 0, 1, kEpiGateUp>), grid, dim3(256), 0,
                                   ctx->stream, g);
            else if (few)
                hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 1, 1, kEpiSiluBwd, 2>), grid, dim3(512), 0,
                                   ctx->stream, g);
            else
                hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 1, 1, kEpiSiluBwd>), grid, dim3(256), 0,
                                   ctx->stream, g);
            FT_LAUNCH_CHECK();
            return FT_OK;
        } else {
            return ft_set_error(FT_ERR_INVALID, "fused epilogues use 64x64 tiles");
        }
    }
    // Eight waves on a tile when the tiles alone leave at most two workgroups on a CU and the K
    // loop can be shared in pairs of tiles.
    pairs = pairs || (pairs_ok && g.splits == 1 && (size_t)tiles <= 2 * (size_t)ctx->num_cus && min_kt >= 32);
    if constexpr (BM == 64) {
        if (pairs) {
            snprintf(name, sizeof(name), "gemm_async_kernel<%d, %d, %d, %d, %d, %d, 0, 2>", BM, BN, WM, WN, layout,
                     max_seg > 1 ? kAsyncMaxSeg : 1);
            ft_prof_scope prof(ctx, name, flops, bytes);
            if (max_seg == 1) {
                if (layout == 0)
                    hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 0, 1, kEpiPlain, 2>), grid, dim3(512), 0,
                                       ctx->stream, g);
                else
                    hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 1, 1, kEpiPlain, 2>), grid, dim3(512), 0,
                                       ctx->stream, g);
            } else {
                if (layout == 0)
                    hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 0, kAsyncMaxSeg, kEpiPlain, 2>), grid,
                                       dim3(512), 0, ctx->stream, g);
                else
                    hipLaunchKernelGGL((gemm_async_kernel<64, 64, 32, 32, 1, kAsyncMaxSeg, kEpiPlain, 2>), grid,
                                       dim3(512), 0, ctx->stream, g);
            }
            FT_LAUNCH_CHECK();
            return reduce_shares();
        }
    }
    snprintf(name, sizeof(name), "gemm_async_kernel<%d, %d, %d, %d, %d, %d>", BM, BN, WM, WN, layout,
             max_seg > 1 ? kAsyncMaxSeg : 1);
    ft_prof_scope prof(ctx, name, flops, bytes);
    if (max_seg == 1) {
        if (layout == 0)
            hipLaunchKernelGGL((gemm_async_kernel<BM, BN, WM, WN, 0, 1>), grid, dim3(256), 0, ctx->stream, g);
        else
            hipLaunchKernelGGL((gemm_async_kernel<BM, BN, WM, WN, 1, 1>), grid, dim3(256), 0, ctx->stream, g);
    } else {
        if (layout == 0)
            hipLaunchKernelGGL((gemm_async_kernel<BM, BN, WM, WN, 0, kAsyncMaxSeg>), grid, dim3(256), 0,
                               ctx->stream, g);
        else
            hipLaunchKernelGGL((gemm_async_kernel<BM, BN, WM, WN, 1, kAsyncMaxSeg>), grid, dim3(256), 0,
                               ctx->stream, g);
    }
    FT_LAUNCH_CHECK();
    return reduce_shares();
}

// Tile choice, from measurements of the whole step on MI355X at M = 2048: 128x128
// tiles (64x64 per wave) reach the highest MFMA rate but only pay off when there
// are many of them per CU (the vocabulary head); everything else runs best as
// 64x64 tiles, four workgroups resident per CU (three with two b tiles per stage; 128x64
// and 64x128 tiles were measured too: no gain inside the step).
int launch_async_auto(ft_context* ctx, const AsyncBatch& g, int layout) {
    size_t tiles128 = 0;
    for (int i = 0; i < g.count; i++) tiles128 += (size_t)((g.M + 127) / 128) * (size_t)((g.p[i].N + 127) / 128);
    if (tiles128 >= 8 * (size_t)ctx->num_cus) return launch_async<128, 128, 64, 64>(ctx, g, layout);
    // A very long K over few tiles (the head's input gradient: K = vocabulary): the large tile with its K
    // tiles shared out runs at the rate of the many-tile case, and the extra pass over the partial tiles is
    // a fraction of a percent of the product.
    int min_kt = 1 << 30;
    bool plain = true;
    for (int i = 0; i < g.count; i++) {
        int kt = 0;
        for (int s = 0; s < g.p[i].nseg; s++) kt += g.p[i].seg[s].nt;
        min_kt = kt < min_kt ? kt : min_kt;
        plain = plain && g.p[i].rope == nullptr && ((size_t)g.M * g.p[i].N) % 4 == 0 && g.p[i].ldc == g.p[i].N;
    }
    if (plain && min_kt >= 512 && tiles128 * 2 <= 2 * (size_t)ctx->num_cus && tiles128 * 8 >= 2 * (size_t)ctx->num_cus)
        return launch_async<128, 128, 64, 64>(ctx, g, layout);
    return launch_async<64, 64, 32, 32>(ctx, g, layout);
}

// Can out[M,N] (+)= a[M,K] @ b (f16, `layout`) + a2[M,K2] @ b2 run on the asynchronous path?
bool async_eligible(int layout, const float* a, const void* b, const float* out, const float* add, size_t M, size_t K,
                    size_t N, const float* a2, const float* b2, size_t K2) {
    if (layout != 0 && layout != 1) return false;
    if (M == 0 || N == 0 || K < 32 || K % 32 != 0) return false;
    if (!aligned16p(a) || !aligned16p(b) || !aligned16p(out) || !out || !a || !b) return false;
    // The residual is read in 16-byte groups (epilogue and split-K reduce kernel alike).
    if (add && !aligned16p(add)) return false;
    if (layout == 0 && (N % 8 != 0 || N < 8)) return false;
    if (K2 > 0 && (K2 > 16 || K2 % 4 != 0 || !aligned16p(a2) || !aligned16p(b2))) return false;
    // Per-lane operand offsets are 32-bit byte offsets from a uniform base.
    const double lim = 4294967296.0;
    const double ldb = layout == 1 ? (double)K : (double)N;
    return 4.0 * (double)M * (double)K + 4.0 * 64 * (double)K < lim &&
           2.0 * ldb * (double)(layout == 1 ? N : K) + 2.0 * 64 * ldb < lim;
}

AsyncSeg make_seg(int layout, const float* a, const void* b, size_t K, size_t N, const float* a2, const float* b2,
                  size_t K2) {
    AsyncSeg sg{};
    sg.a = a;
    sg.b = b;
    sg.a2 = K2 > 0 ? a2 : nullptr;
    sg.b2 = K2 > 0 ? b2 : nullptr;
    sg.lda = (int)K;
    sg.ldb = layout == 1 ? (int)K : (int)N;
    sg.lda2 = (int)K2;
    sg.ldb2 = layout == 1 ? (int)K2 : (int)N;
    sg.nt = (int)(K / 32);
    sg.K2 = (int)K2;
    return sg;
}

template <int BM, int BN, int WM, int WN, int BKF = 32>
int launch_cfg(ft_context* ctx, GemmArgs p, int layout, bool half_b, bool fast) {
    const int tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const dim3 grid((unsigned)(tiles_m * p.tiles_n));
    char name[96];
    if (fast)
        snprintf(name, sizeof(name), "gemm_fast_kernel<%d, %d, %d, %d, %d, %s, %d>", BM, BN, WM, WN, layout,
                 half_b ? "true" : "false", BKF);
    else
        snprintf(name, sizeof(name), "gemm_kernel<%d, %d, %d, %d, %d, %s>", BM, BN, WM, WN, layout,
                 half_b ? "true" : "false");
    const double kk = (double)p.K + (p.a2 ? (double)p.K2 : 0.0);
    ft_prof_scope prof(ctx, name, 2.0 * p.M * (double)p.N * kk,
                       4.0 * p.M * kk + (half_b ? 2.0 : 4.0) * p.N * (double)p.K + 4.0 * p.N * (p.a2 ? p.K2 : 0) +
                           4.0 * p.M * (double)p.N);
#define FT_GEMM_LAUNCH(L, H)                                                                             \
    do {                                                                                                 \
        if (fast)                                                                                        \
            hipLaunchKernelGGL((gemm_fast_kernel<BM, BN, WM, WN, L, H, BKF>), grid, dim3(256), 0, ctx->stream, p); \
        else                                                                                             \
            hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, L, H>), grid, dim3(256), 0, ctx->stream, p);      \
    } while (0)
    if (layout == 0) {
        if (half_b) FT_GEMM_LAUNCH(0, true); else FT_GEMM_LAUNCH(0, false);
    } else if (layout == 1) {
        if (half_b) FT_GEMM_LAUNCH(1, true); else FT_GEMM_LAUNCH(1, false);
    } else {
        FT_GEMM_LAUNCH(2, false);
    }
#undef FT_GEMM_LAUNCH
    FT_LAUNCH_CHECK();
    return FT_OK;
}

// Operands of the f32 DMA kernel: 16-byte aligned, K in whole tiles, at least two of them per
// workgroup, k-major operands in whole float4 groups, 32-bit per-lane offsets.
bool f32_async_eligible(int layout, const float* a, const void* b, const float* out, size_t M, size_t K, size_t N) {
    if (M == 0 || N == 0 || K < 64 || K % 32 != 0) return false;
    if (!aligned16p(a) || !aligned16p(b) || !out) return false;
    const bool a_km = layout == 2, b_km = layout != 1;
    if (a_km && (M % 4 != 0 || M < 4)) return false;
    if (b_km && (N % 4 != 0 || N < 4)) return false;
    if (M * N < 128 * 128) return false;  // tiny products: the register-staged kernels
    const double lim = 4294967296.0;
    const double a_span = a_km ? 4.0 * 36 * (double)M : 4.0 * ((double)M + 64) * (double)K;
    const double b_span = b_km ? 4.0 * 36 * (double)N : 4.0 * ((double)N + 64) * (double)K;
    return a_span < lim && b_span < lim;
}

int launch_f32_async(ft_context* ctx, int layout, const float* a, const float* b, float* out, size_t M, size_t K,
                     size_t N) {
    F32AsyncArgs g{};
    g.a = a;
    g.b = b;
    g.out = out;
    g.M = (int)M;
    g.N = (int)N;
    g.nt = (int)(K / 32);
    g.lda = layout == 2 ? (int)M : (int)K;
    g.ldb = layout == 1 ? (int)K : (int)N;
    g.ldc = (int)N;
    g.tiles_m = (int)((M + 63) / 64);
    g.tiles_n = (int)((N + 63) / 64);
    g.xcds = ft_gemm_xcds(ctx);
    // panels of about sqrt(96) n tiles: equal bytes of a and b per XCD-resident block of tiles
    int panels = (int)((double)g.tiles_n / 10.0 + 0.5);
    if (panels < 1) panels = 1;
    g.panel = (g.tiles_n + panels - 1) / panels;
    // Split K when the tiles occupy at most half of the CUs and K is long enough to share out
    // (at least 4 K tiles per share); the shares are added in order. (At 216 tiles of K = 2048
    // a three-way split measured no gain: 44.4 us against 42.6.)
    const size_t tiles = (size_t)g.tiles_m * g.tiles_n;
    g.splits = 1;
    if (tiles * 2 <= (size_t)ctx->num_cus && (M * N) % 4 == 0) {
        int want = (int)((2 * (size_t)ctx->num_cus + tiles - 1) / tiles);
        if (want > 8) want = 8;
        if (want > g.nt / 4) want = g.nt / 4;
        if (want >= 2 && M * N * (size_t)want <= kSplitScratchFloats) {
            if (!ctx->gemm_scratch) {
                FT_HIP(hipSetDevice(ctx->device));
                FT_HIP(hipMalloc((void**)&ctx->gemm_scratch, kSplitScratchFloats * sizeof(float)));
            }
            g.splits = want;
            g.partial = ctx->gemm_scratch;
        }
    }
    const dim3 grid((unsigned)tiles, (unsigned)g.splits);
    char name[64];
    snprintf(name, sizeof(name), "gemm_f32_async_kernel<%d>", layout);
    ft_prof_scope prof(ctx, name, 2.0 * M * (double)N * K, 4.0 * ((double)M * K + (double)N * K + (double)M * N));
    if (layout == 0)
        hipLaunchKernelGGL((gemm_f32_async_kernel<false, true>), grid, dim3(256), 0, ctx->stream, g);
    else if (layout == 1)
        hipLaunchKernelGGL((gemm_f32_async_kernel<false, false>), grid, dim3(256), 0, ctx->stream, g);
    else
        hipLaunchKernelGGL((gemm_f32_async_kernel<true, true>), grid, dim3(256), 0, ctx->stream, g);
    FT_LAUNCH_CHECK();
    if (g.splits > 1) {
        SplitReduceArgs ra{};
        ra.partial[0] = g.partial;
        ra.add[0] = nullptr;
        ra.out[0] = out;
        ra.n4[0] = (long)(M * N / 4);
        ra.splits = g.splits;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3(ft_div_up(M * N / 4, 256), 1), dim3(256), 0, ctx->stream, ra);
        FT_LAUNCH_CHECK();
    }
    return FT_OK;
}

int gemm_dispatch(ft_context* ctx, const char* who, int layout, bool half_b, const float* a, const void* b,
                  float* out, size_t M, size_t K, size_t N, const float* a2, const float* b2, size_t K2,
                  const float* add = nullptr) {
    FT_CHECK_ARG(ctx, "%s: ctx is NULL", who);
    FT_CHECK_ARG(M < (1u << 30) && N < (1u << 30) && K < (1u << 30) && K2 < (1u << 30), "%s: dimension too large", who);
    if (M == 0 || N == 0) return FT_OK;
    FT_CHECK_ARG(out && (K == 0 || (a && b)), "%s: NULL operand", who);
    FT_CHECK_ARG((a2 == nullptr) == (b2 == nullptr), "%s: a2 and b2 must come together", who);
    FT_CHECK_ARG(!(layout == 2 && (half_b || a2)), "%s: unsupported operand combination", who);
    GemmArgs p{};
    p.a = a;
    p.b = b;
    p.out = out;
    p.add = add;
    p.a2 = K2 > 0 ? a2 : nullptr;
    p.b2 = K2 > 0 ? b2 : nullptr;
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.K2 = (int)K2;
    p.lda = layout == 2 ? (long)M : (long)K;
    p.ldb = layout == 1 ? (long)K : (long)N;
    p.ldc = (long)N;
    p.lda2 = (long)K2;
    p.ldb2 = layout == 1 ? (long)K2 : (long)N;
    if (half_b && K > 0 && async_eligible(layout, a, b, out, add, M, K, N, p.a2, p.b2, p.a2 ? K2 : 0)) {
        AsyncBatch g{};
        g.count = 1;
        g.M = (int)M;
        g.p[0].seg[0] = make_seg(layout, a, b, K, N, p.a2, p.b2, p.a2 ? K2 : 0);
        g.p[0].nseg = 1;
        g.p[0].out = out;
        g.p[0].add = add;
        g.p[0].N = (int)N;
        g.p[0].ldc = (int)N;
        return launch_async_auto(ctx, g, layout);
    }
    if (!half_b && !p.a2 && !add && f32_async_eligible(layout, a, b, out, M, K, N))
        return launch_f32_async(ctx, layout, a, static_cast<const float*>(b), out, M, K, N);
    // Tile choice for the register-staged kernels, from measurements on MI355X at
    // M = 2048: 128x128 tiles when there are many per CU, else 64x64; a deep K
    // loop on few tiles prefers BK = 64 (half the barriers per MFMA).
    const size_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
    const size_t tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
    int best = tiles128 >= 8 * (size_t)ctx->num_cus ? 0 : 2;
    if (best == 2 && K >= 4096 && tiles64 <= 2 * (size_t)ctx->num_cus) best = 3;
    // The branch-free kernel needs aligned operands and whole float4 groups.
    auto al16 = [](const void* q) { return (((uintptr_t)q) & 15) == 0; };
    bool fast = al16(a) && al16(b) && al16(out) && K % 4 == 0 && K >= 4 && (p.lda % 4 == 0) && (p.ldb % 4 == 0);
    if (layout != 1) fast = fast && N % 4 == 0 && N >= 4;   // b rows run along n
    if (layout == 2) fast = fast && M % 4 == 0 && M >= 4;   // a rows run along m
    if (half_b) fast = fast && (p.ldb % 8 == 0 || layout == 1);
    if (p.a2) fast = fast && al16(a2) && al16(b2) && K2 % 4 == 0 && K2 >= 4;
    // Per-lane operand offsets are 32-bit byte offsets from a uniform base.
    const double lim = 4294967296.0;
    fast = fast && 4.0 * (double)M * (double)(layout == 2 ? 1 : K) + 4.0 * 64 * (double)p.lda < lim &&
           4.0 * (double)N * (double)(layout == 1 ? K : 1) + 4.0 * 64 * (double)p.ldb < lim;
    if (best == 0) return launch_cfg<128, 128, 64, 64>(ctx, p, layout, half_b, fast);
    if (best == 3) return launch_cfg<64, 64, 32, 32, 64>(ctx, p, layout, half_b, fast);
    return launch_cfg<64, 64, 32, 32>(ctx, p, layout, half_b, fast);
}

template <bool XT, bool YT, bool OT>
int skinny_launch(ft_context* ctx, const float* x, const float* y, float* out, size_t R, size_t Kr, size_t C,
                  long ldx, long ldy, long ldo, float scale) {
    if (R == 0 || C == 0) return FT_OK;
    char name[64];
    snprintf(name, sizeof(name), "skinny_kernel<%s, %s, %s>", XT ? "true" : "false", YT ? "true" : "false",
             OT ? "true" : "false");
    ft_prof_scope prof(ctx, name, 2.0 * R * (double)Kr * C, 4.0 * ((double)R * Kr + (double)Kr * C + (double)R * C));
    hipLaunchKernelGGL((skinny_kernel<XT, YT, OT>), dim3(ft_div_up(R, 32)), dim3(256), 0, ctx->stream, x, y, out,
                       (int)R, (int)Kr, (int)C, ldx, ldy, ldo, scale);
    FT_LAUNCH_CHECK();
    return FT_OK;
}

}  // namespace

extern "C" {

int ft_mfma_probe(ft_context* ctx, size_t rounds, size_t waves_per_simd, size_t chains, int random_operands,
                  double* seconds, double* flops) {
    FT_CHECK_ARG(ctx && seconds && flops, "ft_mfma_probe: NULL argument");
    FT_CHECK_ARG(rounds >= 1 && rounds <= (1u << 24), "ft_mfma_probe: rounds %zu is outside 1..2^24", rounds);
    FT_CHECK_ARG(waves_per_simd >= 1 && waves_per_simd <= 4, "ft_mfma_probe: waves_per_simd %zu is outside 1..4",
                 waves_per_simd);
    FT_CHECK_ARG(chains == 1 || chains == 2 || chains == 4, "ft_mfma_probe: chains must be 1, 2 or 4");
    const size_t wgs = (size_t)ctx->num_cus * waves_per_simd;  // 256 threads = one wave per SIMD of a CU
    float* out = nullptr;
    FT_TRY(ft_alloc(ctx, wgs * 256 * sizeof(float), (void**)&out));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    float ms = 0.0f;
    hipError_t err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err == hipSuccess) err = hipEventRecord(e0, ctx->stream);
    if (err == hipSuccess) {
        const dim3 grid((unsigned)wgs);
        if (chains == 1)
            hipLaunchKernelGGL(mfma_probe_kernel<1>, grid, dim3(256), 0, ctx->stream, out, (int)rounds,
                               random_operands);
        else if (chains == 2)
            hipLaunchKernelGGL(mfma_probe_kernel<2>, grid, dim3(256), 0, ctx->stream, out, (int)rounds,
                               random_operands);
        else
            hipLaunchKernelGGL(mfma_probe_kernel<4>, grid, dim3(256), 0, ctx->stream, out, (int)rounds,
                               random_operands);
        err = hipGetLastError();
    }
    if (err == hipSuccess) err = hipEventRecord(e1, ctx->stream);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    FT_TRY(ft_free(ctx, out));
    FT_HIP(err);
    *seconds = (double)ms * 1e-3;
    *flops = (double)wgs * 4.0 * (double)rounds * 16.0 * 4096.0;  // waves x MFMAs x 2*32*32*2
    return FT_OK;
}

int ft_matmul(ft_context* ctx, const float* a, const float* b, float* out, size_t M, size_t K, size_t N) {
    return gemm_dispatch(ctx, "ft_matmul", 0, false, a, b, out, M, K, N, nullptr, nullptr, 0);
}
int ft_matmul_bt(ft_context* ctx, const float* a, const float* b, float* out, size_t M, size_t K, size_t N) {
    return gemm_dispatch(ctx, "ft_matmul_bt", 1, false, a, b, out, M, K, N, nullptr, nullptr, 0);
}
int ft_matmul_at(ft_context* ctx, const float* a, const float* b, float* out, size_t M, size_t K, size_t N) {
    return gemm_dispatch(ctx, "ft_matmul_at", 2, false, a, b, out, M, K, N, nullptr, nullptr, 0);
}
int ft_matmul_f16b(ft_context* ctx, const float* a, const uint16_t* b, float* out, size_t M, size_t K, size_t N) {
    return gemm_dispatch(ctx, "ft_matmul_f16b", 0, true, a, b, out, M, K, N, nullptr, nullptr, 0);
}
int ft_matmul_bt_f16b(ft_context* ctx, const float* a, const uint16_t* b, float* out, size_t M, size_t K, size_t N) {
    return gemm_dispatch(ctx, "ft_matmul_bt_f16b", 1, true, a, b, out, M, K, N, nullptr, nullptr, 0);
}

int ft_lora_down(ft_context* ctx, const float* x, const float* a, float* t, size_t M, size_t K, size_t r,
                 float scale) {
    FT_CHECK_ARG(ctx && x && a && t, "ft_lora_down: NULL argument");
    FT_CHECK_ARG(r >= 1 && r <= 32, "ft_lora_down: rank %zu is outside 1..32", r);
    ft_thin_problem tp{x, a, t, (int)M, (int)K, 0, (int)r, (long)K, (long)r, (long)r, scale, 0, 0, 0, 0};
    if (ft_thin_rowwise_ok(tp)) return ft_thin_rowwise(ctx, &tp, 1);
    return skinny_launch<false, false, false>(ctx, x, a, t, M, K, r, (long)K, (long)r, (long)r, scale);
}

int ft_lora_linear(ft_context* ctx, const float* x, const void* w, int w_dtype, const float* t, const float* b,
                   const float* residual, float* y, size_t M, size_t K, size_t N, size_t r) {
    FT_CHECK_ARG(w_dtype == FT_DTYPE_F32 || w_dtype == FT_DTYPE_F16, "ft_lora_linear: dtype %d", w_dtype);
    return gemm_dispatch(ctx, "ft_lora_linear", 0, w_dtype == FT_DTYPE_F16, x, w, y, M, K, N, t, b, r, residual);
}

int ft_lora_grad_down(ft_context* ctx, const float* dy, const float* b, float* dt, size_t M, size_t N, size_t r,
                      float scale) {
    FT_CHECK_ARG(ctx && dy && b && dt, "ft_lora_grad_down: NULL argument");
    FT_CHECK_ARG(r >= 1 && r <= 32, "ft_lora_grad_down: rank %zu is outside 1..32", r);
    // dt[m][j] = sum_n dy[m][n] * b[j][n]
    ft_thin_problem tp{dy, b, dt, (int)M, (int)N, 0, (int)r, (long)N, (long)N, (long)r, scale, 1, 0, 0, 0};
    if (ft_thin_rowwise_ok(tp)) return ft_thin_rowwise(ctx, &tp, 1);
    return skinny_launch<false, true, false>(ctx, dy, b, dt, M, N, r, (long)N, (long)N, (long)r, scale);
}

int ft_lora_linear_dx(ft_context* ctx, const float* dy, const void* w, int w_dtype, const float* dt,
                      const float* a, const float* residual, float* dx, size_t M, size_t K, size_t N, size_t r) {
    FT_CHECK_ARG(w_dtype == FT_DTYPE_F32 || w_dtype == FT_DTYPE_F16, "ft_lora_linear_dx: dtype %d", w_dtype);
    // dx[M,K] = dy[M,N] @ w[K,N]^T + dt[M,r] @ a[K,r]^T: layout 1 with output width K, reduction N.
    return gemm_dispatch(ctx, "ft_lora_linear_dx", 1, w_dtype == FT_DTYPE_F16, dy, w, dx, M, N, K, dt, a, r, residual);
}

int ft_lora_linear_group(ft_context* ctx, const float* x, const ft_lora_linear_desc* linears, size_t count,
                         size_t M, size_t K) {
    FT_CHECK_ARG(ctx && linears && count >= 1 && count <= (size_t)kAsyncMaxProb,
                 "ft_lora_linear_group: 1..%d linears per call", kAsyncMaxProb);
    bool batch = M < (1u << 30) && K < (1u << 30) && M > 0;
    bool any_rope = false;
    for (size_t i = 0; i < count; i++) {
        const ft_lora_linear_desc& d = linears[i];
        FT_CHECK_ARG(d.w_dtype == FT_DTYPE_F32 || d.w_dtype == FT_DTYPE_F16, "ft_lora_linear_group: dtype %d",
                     d.w_dtype);
        if (d.rope_table) {
            FT_CHECK_ARG(d.residual == nullptr && d.N % 64 == 0 && d.rope_seq > 0 && M % d.rope_seq == 0,
                         "ft_lora_linear_group: a rotated output needs head_dim 64, whole rows of rope_seq tokens "
                         "and no residual");
            any_rope = true;
        }
        FT_CHECK_ARG(d.r == 0 || (d.t && d.b), "ft_lora_linear_group: linear %zu has a rank but no factors", i);
        batch = batch && d.w_dtype == FT_DTYPE_F16 && d.N < (1u << 30) &&
                async_eligible(0, x, d.w, d.y, d.residual, M, K, d.N, d.t, d.b, d.r);
    }
    if (batch && count > 1) {
        AsyncBatch g{};
        g.count = (int)count;
        g.M = (int)M;
        for (size_t i = 0; i < count; i++) {
            const ft_lora_linear_desc& d = linears[i];
            g.p[i].seg[0] = make_seg(0, x, d.w, K, d.N, d.t, d.b, d.r);
            g.p[i].nseg = 1;
            g.p[i].out = d.y;
            g.p[i].add = d.residual;
            g.p[i].N = (int)d.N;
            g.p[i].ldc = (int)d.N;
            g.p[i].rope = reinterpret_cast<const float2*>(d.rope_table);
            g.p[i].rope_seq = (int)d.rope_seq;
        }
        if (!any_rope) return launch_async_auto(ctx, g, 0);
        return launch_async<64, 64, 32, 32>(ctx, g, 0);  // the rotation lives in the 64x64 epilogue
    }
    for (size_t i = 0; i < count; i++) {
        const ft_lora_linear_desc& d = linears[i];
        FT_TRY(ft_lora_linear(ctx, x, d.w, d.w_dtype, d.r ? d.t : nullptr, d.r ? d.b : nullptr, d.residual, d.y, M, K,
                              d.N, d.r));
        if (d.rope_table)
            FT_TRY(ft_rope_apply(ctx, d.y, d.y, M / d.rope_seq, d.rope_seq, d.N, 64, d.rope_table, 0));
    }
    return FT_OK;
}

int ft_lora_linear_dx_group(ft_context* ctx, const ft_lora_dx_desc* linears, size_t count, const float* residual,
                            float* dx, size_t M, size_t K) {
    FT_CHECK_ARG(ctx && linears && dx && count >= 1 && count <= (size_t)kAsyncMaxSeg,
                 "ft_lora_linear_dx_group: 1..%d linears per call", kAsyncMaxSeg);
    bool batch = M < (1u << 30) && K < (1u << 30) && M > 0 && K > 0;
    size_t tiles = 0;
    for (size_t i = 0; i < count; i++) {
        const ft_lora_dx_desc& d = linears[i];
        FT_CHECK_ARG(d.w_dtype == FT_DTYPE_F32 || d.w_dtype == FT_DTYPE_F16, "ft_lora_linear_dx_group: dtype %d",
                     d.w_dtype);
        FT_CHECK_ARG(d.r == 0 || (d.dt && d.a), "ft_lora_linear_dx_group: linear %zu has a rank but no factors", i);
        batch = batch && d.w_dtype == FT_DTYPE_F16 && d.N < (1u << 30) &&
                async_eligible(1, d.dy, d.w, dx, residual, M, d.N, K, d.dt, d.a, d.r);
        tiles += d.N / 32;
    }
    if (batch && count > 1 && tiles < (1u << 30)) {
        AsyncBatch g{};
        g.count = 1;
        g.M = (int)M;
        for (size_t i = 0; i < count; i++) {
            const ft_lora_dx_desc& d = linears[i];
            g.p[0].seg[i] = make_seg(1, d.dy, d.w, d.N, K, d.dt, d.a, d.r);
        }
        g.p[0].nseg = (int)count;
        g.p[0].out = dx;
        g.p[0].add = residual;
        g.p[0].N = (int)K;
        g.p[0].ldc = (int)K;
        return launch_async_auto(ctx, g, 1);
    }
    for (size_t i = 0; i < count; i++) {
        const ft_lora_dx_desc& d = linears[i];
        FT_TRY(ft_lora_linear_dx(ctx, d.dy, d.w, d.w_dtype, d.r ? d.dt : nullptr, d.r ? d.a : nullptr,
                                 i == 0 ? residual : dx, dx, M, K, d.N, d.r));
    }
    return FT_OK;
}

int ft_mlp_gate_up(ft_context* ctx, const float* x, const void* w_gate, const void* w_up, int w_dtype, float* gate,
                   float* up, float* act, size_t M, size_t K, size_t N) {
    FT_CHECK_ARG(ctx && x && w_gate && w_up && gate && up && act, "ft_mlp_gate_up: NULL argument");
    FT_CHECK_ARG(w_dtype == FT_DTYPE_F32 || w_dtype == FT_DTYPE_F16, "ft_mlp_gate_up: dtype %d", w_dtype);
    if (M == 0 || N == 0) return FT_OK;
    const bool fused = w_dtype == FT_DTYPE_F16 && M < (1u << 30) && K < (1u << 30) && N < (1u << 30) &&
                       async_eligible(0, x, w_up, up, nullptr, M, K, N, nullptr, nullptr, 0) &&
                       async_eligible(0, x, w_gate, gate, nullptr, M, K, N, nullptr, nullptr, 0) && aligned16p(act);
    if (fused) {
        AsyncBatch g{};
        g.count = 1;
        g.M = (int)M;
        g.p[0].seg[0] = make_seg(0, x, w_up, K, N, nullptr, nullptr, 0);
        g.p[0].nseg = 1;
        g.p[0].b_alt = w_gate;
        g.p[0].out = up;
        g.p[0].out2 = gate;
        g.p[0].out3 = act;
        g.p[0].N = (int)N;
        g.p[0].ldc = (int)N;
        return launch_async<64, 64, 32, 32>(ctx, g, 0, kEpiGateUp);
    }
    FT_TRY(ft_lora_linear(ctx, x, w_up, w_dtype, nullptr, nullptr, nullptr, up, M, K, N, 0));
    FT_TRY(ft_lora_linear(ctx, x, w_gate, w_dtype, nullptr, nullptr, nullptr, gate, M, K, N, 0));
    return ft_silu_gate_fused(ctx, gate, up, act, M * N);
}

int ft_mlp_down_backward(ft_context* ctx, const float* dy, const void* w_down, int w_dtype, const float* gate,
                         const float* up, float* d_gate, float* d_up, float* scratch, size_t M, size_t F, size_t H) {
    FT_CHECK_ARG(ctx && dy && w_down && gate && up && d_gate && d_up, "ft_mlp_down_backward: NULL argument");
    FT_CHECK_ARG(w_dtype == FT_DTYPE_F32 || w_dtype == FT_DTYPE_F16, "ft_mlp_down_backward: dtype %d", w_dtype);
    if (M == 0 || F == 0) return FT_OK;
    // d_act[M,F] = dy[M,H] @ w_down[F,H]^T: layout 1 with output width F, reduction H.
    const bool fused = w_dtype == FT_DTYPE_F16 && M < (1u << 30) && F < (1u << 30) && H < (1u << 30) &&
                       async_eligible(1, dy, w_down, d_gate, nullptr, M, H, F, nullptr, nullptr, 0);
    if (fused) {
        AsyncBatch g{};
        g.count = 1;
        g.M = (int)M;
        g.p[0].seg[0] = make_seg(1, dy, w_down, H, F, nullptr, nullptr, 0);
        g.p[0].nseg = 1;
        g.p[0].out = d_gate;
        g.p[0].out2 = d_up;
        g.p[0].e1 = gate;
        g.p[0].e2 = up;
        g.p[0].N = (int)F;
        g.p[0].ldc = (int)F;
        return launch_async<64, 64, 32, 32>(ctx, g, 1, kEpiSiluBwd);
    }
    FT_CHECK_ARG(scratch, "ft_mlp_down_backward: this operand combination needs the [M,F] scratch buffer");
    FT_TRY(ft_lora_linear_dx(ctx, dy, w_down, w_dtype, nullptr, nullptr, nullptr, scratch, M, F, H, 0));
    return ft_silu_gate_backward(ctx, gate, up, scratch, d_gate, d_up, M * F);
}

int ft_lora_grad_b(ft_context* ctx, const float* t, const float* dy, float* db, size_t M, size_t N, size_t r) {
    FT_CHECK_ARG(ctx && t && dy && db, "ft_lora_grad_b: NULL argument");
    FT_CHECK_ARG(r >= 1 && r <= 32, "ft_lora_grad_b: rank %zu is outside 1..32", r);
    // db^T[n][j] = sum_m dy[m][n] * t[m][j]: rows = n (dy read transposed), output stored transposed.
    ft_thin_problem tp{dy, t, db, (int)M, 0, (int)N, (int)r, (long)N, (long)r, (long)N, 1.0f, 0, 1, 0, 0};
    if (ft_thin_colwise_ok(tp)) return ft_thin_colwise(ctx, &tp, 1);
    return skinny_launch<true, false, true>(ctx, dy, t, db, N, M, r, (long)N, (long)r, (long)N, 1.0f);
}

int ft_lora_grad_a(ft_context* ctx, const float* x, const float* dt, float* da, size_t M, size_t K, size_t r) {
    FT_CHECK_ARG(ctx && x && dt && da, "ft_lora_grad_a: NULL argument");
    FT_CHECK_ARG(r >= 1 && r <= 32, "ft_lora_grad_a: rank %zu is outside 1..32", r);
    // da[k][j] = sum_m x[m][k] * dt[m][j]: rows = k (x read transposed).
    ft_thin_problem tp{x, dt, da, (int)M, 0, (int)K, (int)r, (long)K, (long)r, (long)r, 1.0f, 0, 0, 0, 0};
    if (ft_thin_colwise_ok(tp)) return ft_thin_colwise(ctx, &tp, 1);
    return skinny_launch<true, false, false>(ctx, x, dt, da, K, M, r, (long)K, (long)r, (long)r, 1.0f);
}

}  // extern "C"
