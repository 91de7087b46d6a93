// CPU restatement of the reference's kernels for one LoRA training step.
//
// TEST INFRASTRUCTURE ONLY. This file is the parity oracle: tests, the smoke
// check and the CPU-baseline leg of the benchmark call it. Nothing that ships
// (the HIP library, its host driver) may link, load or call it.
//
// Every function restates, in plain f32 loops, the arithmetic of one WGSL
// entry point or host routine of the reference; the citation above each
// function gives the reference file and lines it follows. Summation runs
// sequentially over the reduced index in f32 (the reference's shaders also
// accumulate in f32), except where the reference itself uses f64 on the host.
//
// Parity status: every function here is pinned by tests under tests/
// (golden gradient fixture of the reference, closed forms, torch library
// routines, finite differences). None is "parity unpinned".
//
// Build: g++ -O3 -fopenmp -shared -fPIC (see oracle/build.py). No fast-math:
// loops are written so the vectoriser needs no reassociation.

#include <cmath>
#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <vector>
#include <algorithm>

#if defined(_OPENMP)
#include <omp.h>
#endif

extern "C" {

int orc_num_threads(void) {
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n) {
#if defined(_OPENMP)
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

// ---------------------------------------------------------------------------
// f16 storage of frozen weights
// ---------------------------------------------------------------------------

// f32 -> IEEE binary16, round to nearest even, as `half::f16::from_f32`
// (ferrotensor-backend/src/tensor.rs:261-269; rounding rules pinned by the
// reference's tests at tensor.rs:564-608, 625-667). Overflow -> inf, NaN
// stays NaN (quiet), subnormals are produced, signed zero kept.
static inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t man = x & 0x007FFFFFu;
    const int32_t exp = (int32_t)((x >> 23) & 0xFFu);
    if (exp == 0xFF) {
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7E00u | (man >> 13));
    }
    const int32_t e = exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;  // rounds to zero
        const uint32_t m = man | 0x00800000u;
        const uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (half & 1u))) half += 1u;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half += 1u;  // may carry into exp (-> inf)
    return (uint16_t)(sign | half);
}

static inline float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 0x1F) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// `UnifiedTensor::from_f32_as_f16` packing: little-endian f16 values in
// element order, two per 32-bit word, first value in the low half
// (tensor.rs:258-269).
void orc_pack_f16(const float* in, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = f32_to_f16_bits(in[i]);
}

// The f32 values the f16 matmul kernels see: unpack of the storage above
// (ferrotensor-backend/src/engine/mod.rs:88-108).
void orc_unpack_f16(const uint16_t* in, float* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = f16_bits_to_f32(in[i]);
}

// `write_transposed` (tensor.rs:490-514): src is [rows, cols] row-major, out
// is [cols, rows] row-major.
void orc_transpose(const float* src, float* out, size_t rows, size_t cols) {
#pragma omp parallel for schedule(static)
    for (long c = 0; c < (long)cols; c++)
        for (size_t r = 0; r < rows; r++) out[(size_t)c * rows + r] = src[r * cols + (size_t)c];
}

// ---------------------------------------------------------------------------
// Matrix products (matmul.wgsl:51-166; engine/matmul.rs:94-156)
// layout 0: out[M,N] = a[M,K] @ b[K,N]
// layout 1: out[M,N] = a[M,K] @ b[N,K]^T
// layout 2: out[M,N] = a[K,M]^T @ b[K,N]
// f32 products and sums; each output element adds its K products in
// ascending k, as the naive triple loop does.
// ---------------------------------------------------------------------------

static void gemm_nn(const float* a, const float* b, float* out, size_t M, size_t K, size_t N) {
    constexpr size_t RB = 4, CB = 32;
    // Column panel outermost: the K x 32 panel of b stays in cache while the
    // rows of a stream past it.
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
    for (long j0 = 0; j0 < (long)N; j0 += CB) {
        for (long i0 = 0; i0 < (long)M; i0 += RB) {
            const size_t rb = std::min(RB, M - (size_t)i0);
            const size_t cb = std::min(CB, N - (size_t)j0);
            float acc[RB][CB];
            for (size_t r = 0; r < RB; r++)
                for (size_t c = 0; c < CB; c++) acc[r][c] = 0.0f;
            if (rb == RB && cb == CB) {
                for (size_t k = 0; k < K; k++) {
                    const float* brow = b + k * N + j0;
                    for (size_t r = 0; r < RB; r++) {
                        const float av = a[((size_t)i0 + r) * K + k];
#pragma omp simd
                        for (size_t c = 0; c < CB; c++) acc[r][c] += av * brow[c];
                    }
                }
            } else {
                for (size_t k = 0; k < K; k++) {
                    const float* brow = b + k * N + j0;
                    for (size_t r = 0; r < rb; r++) {
                        const float av = a[((size_t)i0 + r) * K + k];
                        for (size_t c = 0; c < cb; c++) acc[r][c] += av * brow[c];
                    }
                }
            }
            for (size_t r = 0; r < rb; r++)
                for (size_t c = 0; c < cb; c++) out[((size_t)i0 + r) * N + j0 + c] = acc[r][c];
        }
    }
}

void orc_matmul(const float* a, const float* b, float* out, size_t M, size_t K, size_t N, int layout) {
    if (M == 0 || N == 0) return;
    if (layout == 0) {
        gemm_nn(a, b, out, M, K, N);
    } else if (layout == 1) {
        std::vector<float> bt(K * N);
        orc_transpose(b, bt.data(), N, K);  // b is [N,K] -> [K,N]
        gemm_nn(a, bt.data(), out, M, K, N);
    } else {
        std::vector<float> at(K * M);
        orc_transpose(a, at.data(), K, M);  // a is [K,M] -> [M,K]
        gemm_nn(at.data(), b, out, M, K, N);
    }
}

// ---------------------------------------------------------------------------
// RMSNorm (kernels.wgsl:81-98, 110-151; closed form autograd/src/lib.rs:537-564)
// ---------------------------------------------------------------------------

void orc_rms_norm(const float* x, const float* w, float* out, size_t rows, size_t size, float eps) {
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)rows; r++) {
        const float* xr = x + (size_t)r * size;
        float ss = 0.0f;
        for (size_t i = 0; i < size; i++) ss += xr[i] * xr[i];
        const float inv = 1.0f / std::sqrt(ss / (float)size + eps);
        for (size_t i = 0; i < size; i++) out[(size_t)r * size + i] = xr[i] * inv * w[i];
    }
}

// gx = g*w*inv - x * (sum(g*w*x) * inv^3 / size); gw[i] = sum_rows g*x*inv.
void orc_rms_norm_backward(const float* x, const float* w, const float* g, float* gx, float* gw,
                           size_t rows, size_t size, float eps) {
    std::vector<float> invs(rows);
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)rows; r++) {
        const float* xr = x + (size_t)r * size;
        const float* gr = g + (size_t)r * size;
        float ss = 0.0f, gwx = 0.0f;
        for (size_t i = 0; i < size; i++) {
            ss += xr[i] * xr[i];
            gwx += gr[i] * w[i] * xr[i];
        }
        const float inv = 1.0f / std::sqrt(ss / (float)size + eps);
        const float coef = gwx * inv * inv * inv / (float)size;
        for (size_t i = 0; i < size; i++) gx[(size_t)r * size + i] = gr[i] * w[i] * inv - xr[i] * coef;
        invs[r] = inv;
    }
    if (gw) {
#pragma omp parallel for schedule(static)
        for (long i = 0; i < (long)size; i++) {
            float acc = 0.0f;
            for (size_t r = 0; r < rows; r++) acc += g[r * size + i] * x[r * size + i] * invs[r];
            gw[i] = acc;
        }
    }
}

// ---------------------------------------------------------------------------
// RoPE, rotate-half, in place (kernels.wgsl:48-73; host twin
// autograd/src/lib.rs:468-506). data is [batch, seq, hidden]; each head_dim
// slice pairs (i, i + head_dim/2); angle = +-(pos0 + t) * theta^(-2i/head_dim).
// ---------------------------------------------------------------------------

void orc_rope(float* data, size_t batch, size_t seq, size_t hidden, size_t head_dim, size_t pos0,
              float theta, int inverse) {
    const size_t half = head_dim / 2;
    const size_t heads = hidden / head_dim;
    const float sign = inverse ? -1.0f : 1.0f;
#pragma omp parallel for schedule(static) collapse(2)
    for (long b = 0; b < (long)batch; b++) {
        for (long t = 0; t < (long)seq; t++) {
            const float pos = (float)(pos0 + (size_t)t);
            float* tok = data + ((size_t)b * seq + (size_t)t) * hidden;
            for (size_t h = 0; h < heads; h++) {
                float* hv = tok + h * head_dim;
                for (size_t i = 0; i < half; i++) {
                    const float freq_exp = -2.0f * (float)i / (float)head_dim;
                    const float angle = sign * pos * std::pow(theta, freq_exp);
                    const float c = std::cos(angle), s = std::sin(angle);
                    const float v1 = hv[i], v2 = hv[i + half];
                    hv[i] = v1 * c - v2 * s;
                    hv[i + half] = v1 * s + v2 * c;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Attention (flash_attention_v2.wgsl:142-282; backward
// flash_attention_v2_backward.wgsl:1-23, 212-460).
// q/out/dO/dq [B,Sq,H,D]; k/v/dk/dv [B,Sk,Hkv,D]; kv head = h / (H/Hkv).
// Query i sits at position i + causal_offset; key j visible iff j <= that
// (when causal). scale = 1/sqrt(D). lse[(b*H+h)*Sq+i] = log sum exp of the
// scaled visible scores (3.0e38 for a row with no visible key).
// Computed directly (full softmax per row), not tiled: the tiling of the
// reference changes only the f32 summation order.
// ---------------------------------------------------------------------------

void orc_attention(const float* q, const float* k, const float* v, float* out, float* lse, size_t B,
                   size_t Sq, size_t Sk, size_t H, size_t Hkv, size_t D, int causal,
                   size_t causal_offset) {
    const float scale = 1.0f / std::sqrt((float)D);
    const size_t group = H / Hkv;
#pragma omp parallel for schedule(dynamic, 8) collapse(3)
    for (long b = 0; b < (long)B; b++) {
        for (long h = 0; h < (long)H; h++) {
            for (long i = 0; i < (long)Sq; i++) {
                const size_t kvh = (size_t)h / group;
                const float* qr = q + (((size_t)b * Sq + (size_t)i) * H + (size_t)h) * D;
                size_t kend = Sk;
                if (causal) kend = std::min(Sk, (size_t)i + causal_offset + 1);
                std::vector<float> s(kend);
                float m = -1.0e30f;
                for (size_t j = 0; j < kend; j++) {
                    const float* kr = k + (((size_t)b * Sk + j) * Hkv + kvh) * D;
                    float dot = 0.0f;
                    for (size_t d = 0; d < D; d++) dot += (qr[d] * scale) * kr[d];
                    s[j] = dot;
                    m = std::max(m, dot);
                }
                float l = 0.0f;
                for (size_t j = 0; j < kend; j++) {
                    s[j] = std::exp(s[j] - m);
                    l += s[j];
                }
                float* o = out + (((size_t)b * Sq + (size_t)i) * H + (size_t)h) * D;
                const float inv = l > 0.0f ? 1.0f / l : 0.0f;
                for (size_t d = 0; d < D; d++) o[d] = 0.0f;
                for (size_t j = 0; j < kend; j++) {
                    const float* vr = v + (((size_t)b * Sk + j) * Hkv + kvh) * D;
                    const float p = s[j];
                    for (size_t d = 0; d < D; d++) o[d] += p * vr[d];
                }
                for (size_t d = 0; d < D; d++) o[d] *= inv;
                if (lse) lse[((size_t)b * H + (size_t)h) * Sq + (size_t)i] = l > 0.0f ? m + std::log(l) : 3.0e38f;
            }
        }
    }
}

// Delta_i = dO_i . O_i; P_ij = exp(S_ij - L_i); dS_ij = P_ij (dO_i . V_j - Delta_i);
// dQ_i = scale * sum_j dS_ij K_j; dK_j = scale * sum_{heads of the group, i} dS_ij Q_i;
// dV_j = sum P_ij dO_i. Writes (does not accumulate into) dq, dk, dv.
void orc_attention_backward(const float* q, const float* k, const float* v, const float* out,
                            const float* d_out, float* dq, float* dk, float* dv, size_t B, size_t Sq,
                            size_t Sk, size_t H, size_t Hkv, size_t D, int causal,
                            size_t causal_offset) {
    const float scale = 1.0f / std::sqrt((float)D);
    const size_t group = H / Hkv;
    std::memset(dk, 0, sizeof(float) * B * Sk * Hkv * D);
    std::memset(dv, 0, sizeof(float) * B * Sk * Hkv * D);
    // Parallel over (batch, kv head): every dk/dv row belongs to one task.
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
    for (long b = 0; b < (long)B; b++) {
        for (long kvh = 0; kvh < (long)Hkv; kvh++) {
            std::vector<float> p(Sk), dp(Sk);
            for (size_t hg = 0; hg < group; hg++) {
                const size_t h = (size_t)kvh * group + hg;
                for (size_t i = 0; i < Sq; i++) {
                    const size_t row = (((size_t)b * Sq + i) * H + h) * D;
                    const float* qr = q + row;
                    const float* dor = d_out + row;
                    const float* orow = out + row;
                    size_t kend = Sk;
                    if (causal) kend = std::min(Sk, i + causal_offset + 1);
                    float delta = 0.0f;
                    for (size_t d = 0; d < D; d++) delta += dor[d] * orow[d];
                    float m = -1.0e30f;
                    for (size_t j = 0; j < kend; j++) {
                        const float* kr = k + (((size_t)b * Sk + j) * Hkv + (size_t)kvh) * D;
                        float dot = 0.0f;
                        for (size_t d = 0; d < D; d++) dot += (qr[d] * scale) * kr[d];
                        p[j] = dot;
                        m = std::max(m, dot);
                    }
                    float l = 0.0f;
                    for (size_t j = 0; j < kend; j++) l += std::exp(p[j] - m);
                    const float L = l > 0.0f ? m + std::log(l) : 3.0e38f;
                    float* dqr = dq + row;
                    for (size_t d = 0; d < D; d++) dqr[d] = 0.0f;
                    for (size_t j = 0; j < kend; j++) {
                        const size_t kvrow = (((size_t)b * Sk + j) * Hkv + (size_t)kvh) * D;
                        const float* kr = k + kvrow;
                        const float* vr = v + kvrow;
                        const float pij = std::exp(p[j] - L);
                        float dov = 0.0f;
                        for (size_t d = 0; d < D; d++) dov += dor[d] * vr[d];
                        const float ds = pij * (dov - delta);
                        float* dkr = dk + kvrow;
                        float* dvr = dv + kvrow;
                        for (size_t d = 0; d < D; d++) {
                            dqr[d] += ds * kr[d];
                            dkr[d] += ds * qr[d];
                            dvr[d] += pij * dor[d];
                        }
                    }
                    for (size_t d = 0; d < D; d++) dqr[d] *= scale;
                }
            }
            for (size_t j = 0; j < Sk; j++) {
                float* dkr = dk + (((size_t)b * Sk + j) * Hkv + (size_t)kvh) * D;
                for (size_t d = 0; d < D; d++) dkr[d] *= scale;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Elementwise (kernels.wgsl:189-203, 300-311, 744-780, 817-835)
// ---------------------------------------------------------------------------

void orc_add(const float* a, const float* b, float* out, size_t n) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; i++) out[i] = a[i] + b[i];
}

void orc_scale(float* x, size_t n, float s) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; i++) x[i] = x[i] * s;
}

// out = silu(a) * b with silu(a) = a * (1 / (1 + exp(-a))); the reference
// kernel names its first operand "up" but the model passes (gate, up)
// (ferrotensor-graph/src/lib.rs:504-510).
void orc_silu_gate(const float* a, const float* b, float* out, size_t n) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; i++) {
        const float x = a[i];
        const float silu = x * (1.0f / (1.0f + std::exp(-x)));
        out[i] = silu * b[i];
    }
}

// ga = g * b * s * (1 + a * (1 - s)); gb = g * a * s.
void orc_silu_gate_backward(const float* a, const float* b, const float* g, float* ga, float* gb,
                            size_t n) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; i++) {
        const float x = a[i];
        const float s = 1.0f / (1.0f + std::exp(-x));
        gb[i] = g[i] * (x * s);
        ga[i] = g[i] * b[i] * (s * (1.0f + x * (1.0f - s)));
    }
}

// ---------------------------------------------------------------------------
// Embedding gather on the host (autograd/src/lib.rs:1159-1179): id >= vocab
// gives a row of zeros.
// ---------------------------------------------------------------------------

void orc_embedding(const float* table, size_t vocab, size_t hidden, const uint32_t* ids, size_t n,
                   float* out) {
#pragma omp parallel for schedule(static)
    for (long t = 0; t < (long)n; t++) {
        float* o = out + (size_t)t * hidden;
        if ((size_t)ids[t] < vocab)
            std::memcpy(o, table + (size_t)ids[t] * hidden, hidden * sizeof(float));
        else
            std::memset(o, 0, hidden * sizeof(float));
    }
}

// ---------------------------------------------------------------------------
// Masked cross-entropy (kernels.wgsl:684-711; MASKED_CE_SKIP
// engine/training.rs:7). target 0xffffffff => zero grad row, zero loss.
// ---------------------------------------------------------------------------

void orc_masked_cross_entropy(const float* logits, const uint32_t* targets, const float* weights,
                              float* grad, float* row_loss, size_t rows, size_t vocab) {
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)rows; r++) {
        const float* x = logits + (size_t)r * vocab;
        float* g = grad + (size_t)r * vocab;
        const uint32_t t = targets[r];
        if (t == 0xffffffffu) {
            std::memset(g, 0, vocab * sizeof(float));
            row_loss[r] = 0.0f;
            continue;
        }
        float m = -3.4e38f;
        for (size_t i = 0; i < vocab; i++) m = std::max(m, x[i]);
        float se = 0.0f;
        for (size_t i = 0; i < vocab; i++) se += std::exp(x[i] - m);
        const float log_z = m + std::log(se);
        const float w = weights[r];
        for (size_t i = 0; i < vocab; i++) {
            float gv = std::exp(x[i] - log_z) * w;
            if (i == (size_t)t) gv -= w;
            g[i] = gv;
        }
        row_loss[r] = log_z - x[t];
    }
}

// ---------------------------------------------------------------------------
// Gradient norm partials (kernels.wgsl:720-735; SUM_SQUARES_CHUNK = 4096,
// engine/training.rs:263-283). Returns the number of chunks written at
// out[offset..].
// ---------------------------------------------------------------------------

size_t orc_sum_squares_partial(const float* x, size_t n, float* out, size_t offset) {
    const size_t chunk = 4096;
    const size_t blocks = (n + chunk - 1) / chunk;
    for (size_t b = 0; b < blocks; b++) {
        const size_t start = b * chunk, end = std::min(start + chunk, n);
        float acc = 0.0f;
        for (size_t i = start; i < end; i++) acc += x[i] * x[i];
        out[offset + b] = acc;
    }
    return blocks;
}

// ---------------------------------------------------------------------------
// AdamW (kernels.wgsl:357-387; AdamParams engine/training.rs:13-32).
// ---------------------------------------------------------------------------

void orc_adamw_update(float* w, const float* g, float* m, float* v, size_t n, float lr, float beta1,
                      float beta2, float eps, float weight_decay, float t) {
    const float bc1 = 1.0f - std::pow(beta1, t);
    const float bc2 = 1.0f - std::pow(beta2, t);
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; i++) {
        const float gi = g[i];
        const float mi = m[i] * beta1 + (1.0f - beta1) * gi;
        const float vi = v[i] * beta2 + (1.0f - beta2) * gi * gi;
        m[i] = mi;
        v[i] = vi;
        const float m_hat = mi / bc1;
        const float v_hat = vi / bc2;
        float wi = w[i];
        wi = wi - lr * (m_hat / (std::sqrt(v_hat) + eps) + weight_decay * wi);
        w[i] = wi;
    }
}

}  // extern "C"
