/*
 * ferrotensor_hip.h - C ABI of the MI355X (gfx950) kernel library behind
 * Ferrotensor's LoRA training step.
 *
 * The reference has no FFI: its kernel boundary is the concrete Rust API
 * `ferrotensor_backend::{ComputeEngine, UnifiedTensor, WgpuContext}`
 * (ferrotensor-backend/src/lib.rs:38-46). Each entry point below is what a Rust
 * shim implementing that API over HIP would bind; the comment above each one
 * cites the `ComputeEngine` / `UnifiedTensor` / `WgpuContext` method it
 * replaces.
 *
 * Conventions
 *  - Every function returns FT_OK (0) or an FT_ERR_* code; `ft_last_error()`
 *    returns the message of the calling thread's last failure. The reference
 *    panics on shape/dtype violations (assert!); this library never aborts.
 *  - Pointers named `*_dev`, and every tensor operand of an op, are device
 *    pointers in the context's device. Shapes are plain sizes. f32 tensors are
 *    row-major; "f16" operands are the packed little-endian binary16 storage of
 *    `UnifiedTensor::from_f32_as_f16` (tensor.rs:258-269): element i at byte 2*i.
 *  - Ops only enqueue work on the context's stream and return
 *    (context.rs:291-317); order of execution = order of calls;
 *    `ft_synchronize` waits (context.rs:380-391). A context has exactly one
 *    stream; the training step runs on it from its first kernel to its last.
 *  - Outputs are caller-allocated and written, never accumulated into, except
 *    the in-place ops (rope, gradient_scale, clip_grad_by_norm,
 *    gradient_accumulate, adamw_update), as in the reference.
 *  - One thread per context at a time (the reference's autograd is
 *    single-threaded, ferrotensor-autograd/src/lib.rs:11-14).
 */
#ifndef FERROTENSOR_HIP_H
#define FERROTENSOR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FT_OK 0
#define FT_ERR_INVALID 1  /* bad argument / shape (the reference's assert! panics) */
#define FT_ERR_HIP 2      /* a HIP runtime call failed */
#define FT_ERR_OOM 3      /* device allocation failed */

/* engine/training.rs:7 `MASKED_CE_SKIP`, training.rs `SUM_SQUARES_CHUNK`. */
#define FT_MASKED_CE_SKIP 0xffffffffu
#define FT_SUM_SQUARES_CHUNK 4096

/* DType of tensor.rs:18-40 (Q4 is out of scope). */
#define FT_DTYPE_F32 0
#define FT_DTYPE_F16 1

typedef struct ft_context ft_context;

/* Message of this thread's last failing call ("" if none). */
const char* ft_last_error(void);

/* ---- context: WgpuContext (context.rs:96-156, 373-391) ------------------- */

/* WgpuContext::try_new: binds HIP device `device`, creates one stream and the
 * buffer pool. */
int ft_context_create(int device, ft_context** out);
/* Same, but enqueues on a stream the caller owns (hipStream_t as void*). */
int ft_context_create_on_stream(int device, void* hip_stream, ft_context** out);
int ft_context_destroy(ft_context* ctx);
/* WgpuContext::synchronize (context.rs:380-391). */
int ft_synchronize(ft_context* ctx);
/* WgpuContext::flush (context.rs:373-378): a no-op here, launches are already submitted. */
int ft_flush(ft_context* ctx);
/* The hipStream_t the context enqueues on. */
void* ft_context_stream(ft_context* ctx);

/* ---- per-kernel timing (stands in for the reference's timestamp-query
 *      kernel timing, ferrotensor-backend/src/kernel_timing.rs:31-71) -------- */

/* Starts bracketing every kernel launch of this context with HIP events on its
 * stream and clears earlier totals. Costs two event records per launch: keep
 * it off in timed regions that report end-to-end throughput. */
int ft_profile_begin(ft_context* ctx);
/* Stops bracketing, waits for the stream, and reports how many distinct kernel
 * names have totals. */
int ft_profile_end(ft_context* ctx, size_t* kernels);
/* Totals of kernel `index`: launches, summed event time (ms), and the
 * algorithmic flops / bytes the launches were charged with (2MNK for GEMMs,
 * each array once for row kernels; KernelTimes labels, engine/matmul.rs:429-444). */
int ft_profile_kernel(ft_context* ctx, size_t index, const char** name, uint64_t* launches,
                      double* total_ms, double* flops, double* bytes);

/* Diagnostic with no counterpart in the reference: runs `rounds` x 16
 * v_mfma_f32_32x32x2_f32 per wave on register operands (no memory traffic) with
 * `waves_per_simd` (1..4) waves on every SIMD and `chains` (1, 2 or 4)
 * independent accumulators per wave, on operands that are all 1.0 or
 * (`random_operands` != 0) pseudo-random in (-1, 1), and reports the HIP-event time of the one
 * launch and the flops it executed: the rate the FP32 matrix pipes sustain, the
 * ceiling GEMM kernels are compared with. Waits for the stream. */
int ft_mfma_probe(ft_context* ctx, size_t rounds, size_t waves_per_simd, size_t chains, int random_operands,
                  double* seconds, double* flops);

/* ---- buffers: UnifiedTensor storage + BufferPool (tensor.rs, pool.rs) ---- */

/* UnifiedTensor::empty (tensor.rs:184-210): uninitialised device buffer from
 * the exact-size pool (pool.rs). */
int ft_alloc(ft_context* ctx, size_t bytes, void** out_dev);
/* Drop of the last Arc<TensorData> (tensor.rs:106-115): back to the pool. */
int ft_free(ft_context* ctx, void* dev);
/* Releases every pooled buffer to the driver. */
int ft_pool_trim(ft_context* ctx);
/* Bytes currently handed out / held idle by the pool. */
int ft_pool_stats(ft_context* ctx, size_t* live_bytes, size_t* idle_bytes);
/* UnifiedTensor::zeros (tensor.rs:213-217) on an existing buffer. */
int ft_zero(ft_context* ctx, void* dev, size_t bytes);
/* UnifiedTensor::write_data / new / from_bytes (tensor.rs:146-181, 220-255): host -> device. */
int ft_upload(ft_context* ctx, void* dst_dev, const void* src_host, size_t bytes);
/* UnifiedTensor::to_vec (tensor.rs:333-369): device -> host, waits for the copy. */
int ft_download(ft_context* ctx, void* dst_host, const void* src_dev, size_t bytes);
/* UnifiedTensor::from_f32_as_f16 (tensor.rs:258-269): rounds n f32 values to
 * f16 (nearest even) and uploads them packed; dst holds 2*n bytes rounded up
 * to a multiple of 4. */
int ft_upload_f32_as_f16(ft_context* ctx, void* dst_dev, const float* src_host, size_t n);
/* UnifiedTensor::from_f32_transposed (tensor.rs:385-406, 490-514): src is
 * [rows, cols] row-major; dst receives [cols, rows] as FT_DTYPE_F32 or _F16. */
int ft_upload_f32_transposed(ft_context* ctx, void* dst_dev, const float* src_host, size_t rows,
                             size_t cols, int dtype);
/* ComputeEngine::copy_tensor (engine/mod.rs:399-415): device -> device. */
int ft_copy_tensor(ft_context* ctx, const void* src_dev, size_t bytes, void* dst_dev,
                   size_t dst_byte_offset);

/* ---- matrix products (engine/matmul.rs:94-156) --------------------------- */

/* ComputeEngine::matmul: out[M,N] = a[M,K] @ b[K,N]. */
int ft_matmul(ft_context* ctx, const float* a, const float* b, float* out, size_t M, size_t K, size_t N);
/* ComputeEngine::matmul_bt: out[M,N] = a[M,K] @ b[N,K]^T. */
int ft_matmul_bt(ft_context* ctx, const float* a, const float* b, float* out, size_t M, size_t K, size_t N);
/* ComputeEngine::matmul_at: out[M,N] = a[K,M]^T @ b[K,N]. */
int ft_matmul_at(ft_context* ctx, const float* a, const float* b, float* out, size_t M, size_t K, size_t N);
/* ComputeEngine::matmul_f16b: matmul with b[K,N] stored as packed f16. */
int ft_matmul_f16b(ft_context* ctx, const float* a, const uint16_t* b, float* out, size_t M, size_t K, size_t N);
/* ComputeEngine::matmul_bt_f16b: matmul_bt with b[N,K] stored as packed f16. */
int ft_matmul_bt_f16b(ft_context* ctx, const float* a, const uint16_t* b, float* out, size_t M, size_t K, size_t N);

/* ---- LoRA linear, fused (replaces the 6 dispatches of Linear::project_2d,
 *      ferrotensor-graph/src/lib.rs:112-126, and of its backward,
 *      ferrotensor-autograd/src/lib.rs:262-290, 340-357) ---------------------- */

/* Up to 3 linears that read the same input in ONE launch (q/k/v, gate/up of
 * Lfm2Model::forward, ferrotensor-graph/src/lib.rs:255-330): linear i computes
 * y_i[M,N_i] = x[M,K] @ w_i[K,N_i] (+ t_i[M,r_i] @ b_i[r_i,N_i]) (+ residual_i),
 * exactly as ft_lora_linear does. The tiles of all of them share one grid, so a
 * narrow projection no longer leaves most of the chip idle. Linears that cannot
 * take the batched path (f32 weights, unaligned operands) run one by one. */
typedef struct ft_lora_linear_desc {
    const void* w;
    int32_t w_dtype;       /* FT_DTYPE_F32 or FT_DTYPE_F16 */
    const float* t;        /* NULL when r == 0 */
    const float* b;
    const float* residual; /* NULL = none; may alias y */
    float* y;
    size_t N;
    size_t r;
    /* RoPENode fused into the projection (Attention::forward, graph/src/lib.rs:367-414, applies
     * rope to q and k right after their projections): when not NULL, y is rotated with this
     * (cos, sin) table of ft_rope_table for rows of rope_seq tokens and heads of 64 values. */
    const float* rope_table;
    size_t rope_seq;
} ft_lora_linear_desc;
int ft_lora_linear_group(ft_context* ctx, const float* x, const ft_lora_linear_desc* linears, size_t count,
                         size_t M, size_t K);

/* The input gradient shared by up to 3 linears that read the same input
 * (MatMulNode::backward for each of them followed by the AddNode accumulation,
 * ferrotensor-autograd/src/lib.rs:262-357), in ONE launch:
 * dx[M,K] = (residual) + sum_i ( dy_i[M,N_i] @ w_i[K,N_i]^T + dt_i[M,r_i] @ a_i[K,r_i]^T ).
 * The sum runs inside the accumulators: one K loop over the concatenated N_i. */
typedef struct ft_lora_dx_desc {
    const float* dy;
    const void* w;
    int32_t w_dtype;
    const float* dt;       /* NULL when r == 0 */
    const float* a;
    size_t N;
    size_t r;
} ft_lora_dx_desc;
int ft_lora_linear_dx_group(ft_context* ctx, const ft_lora_dx_desc* linears, size_t count, const float* residual,
                            float* dx, size_t M, size_t K);

/* The gated-MLP front half in ONE launch (Lfm2Model's feed-forward,
 * ferrotensor-graph/src/lib.rs:312-330: two project_2d calls and silu_gate_fused):
 * gate[M,N] = x @ w_gate, up[M,N] = x @ w_up, act = silu(gate) * up. Each
 * workgroup multiplies one x tile against the matching tiles of both weights
 * and applies the activation in the epilogue; gate and up are still written
 * (the backward pass reads them). Frozen weights only (no rank-r term). */
int ft_mlp_gate_up(ft_context* ctx, const float* x, const void* w_gate, const void* w_up, int w_dtype,
                   float* gate, float* up, float* act, size_t M, size_t K, size_t N);
/* The gated-MLP back half in ONE launch: with d_act[M,F] = dy[M,H] @ w_down[F,H]^T
 * (MatMulNode::backward of the down projection) never stored, the epilogue applies
 * SiluGateNode::backward (engine/elementwise.rs:194-216):
 * d_gate = d_act * up * silu'(gate), d_up = d_act * silu(gate). `scratch` ([M,F]
 * floats, may be NULL) is only used when the operands rule out the fused kernel
 * (f32 weights, unaligned buffers). */
int ft_mlp_down_backward(ft_context* ctx, const float* dy, const void* w_down, int w_dtype,
                         const float* gate, const float* up, float* d_gate, float* d_up, float* scratch,
                         size_t M, size_t F, size_t H);

/* t[M,r] = scale * (x[M,K] @ a[K,r]): the `x @ A` product with the alpha/rank
 * scale applied where the reference applies it (graph/src/lib.rs:116-122).
 * r <= 32. */
int ft_lora_down(ft_context* ctx, const float* x, const float* a, float* t, size_t M, size_t K,
                 size_t r, float scale);
/* y[M,N] = x[M,K] @ w[K,N] + t[M,r] @ b[r,N] (+ residual[M,N]); w is f32
 * (w_dtype FT_DTYPE_F32) or packed f16. The rank-r product rides in the GEMM's
 * K loop; `residual` (NULL = none, may be y itself) is added in the epilogue,
 * which also absorbs the block's residual add (lfm.rs:116-139). */
int ft_lora_linear(ft_context* ctx, const float* x, const void* w, int w_dtype, const float* t,
                   const float* b, const float* residual, float* y, size_t M, size_t K, size_t N,
                   size_t r);
/* dt[M,r] = scale * (dy[M,N] @ b[r,N]^T): gradient of the scaled `x @ A`. */
int ft_lora_grad_down(ft_context* ctx, const float* dy, const float* b, float* dt, size_t M,
                      size_t N, size_t r, float scale);
/* dx[M,K] = dy[M,N] @ w[K,N]^T + dt[M,r] @ a[K,r]^T (+ residual[M,K]): both
 * MatMulNode input gradients and their AddNode sum in one GEMM; `residual`
 * (NULL = none, may be dx itself) carries a gradient that is being
 * accumulated (accumulate_grad, ferrotensor-autograd/src/lib.rs:206-218). */
int ft_lora_linear_dx(ft_context* ctx, const float* dy, const void* w, int w_dtype, const float* dt,
                      const float* a, const float* residual, float* dx, size_t M, size_t K, size_t N,
                      size_t r);
/* db[r,N] = t[M,r]^T @ dy[M,N]  (matmul_at of the scaled x@A and dy). */
int ft_lora_grad_b(ft_context* ctx, const float* t, const float* dy, float* db, size_t M, size_t N,
                   size_t r);
/* da[K,r] = x[M,K]^T @ dt[M,r]  (matmul_at of x and dt). */
int ft_lora_grad_a(ft_context* ctx, const float* x, const float* dt, float* da, size_t M, size_t K,
                   size_t r);

/* ---- normalisation (engine/norm.rs:20-99) -------------------------------- */

/* ComputeEngine::rms_norm_eps: out = x * rsqrt(mean(x^2) + eps) * w, rows x size. */
int ft_rms_norm_eps(ft_context* ctx, const float* x, const float* w, float* out, size_t rows,
                    size_t size, float eps);
/* ComputeEngine::rms_norm_backward: gx (rows x size) and gw (size); gw may be
 * NULL when the norm scale is frozen and nobody reads it. */
int ft_rms_norm_backward(ft_context* ctx, const float* x, const float* w, const float* g, float* gx,
                         float* gw, size_t rows, size_t size, float eps);
/* No counterpart in the reference. ft_rms_norm_backward with the norm-weight gradient keeps one
 * partial row per workgroup in a buffer it takes from the context's pool, which may call
 * hipMalloc. This variant is for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it): same kernels, same results, but the partial
 * rows live in a fixed device array of the library (2 MiB per GPU, held until the process ends)
 * and the call makes no allocation of any kind. Limits, reported as FT_ERR_INVALID: gw must not
 * be NULL, rows >= 1, size a multiple of 4 and <= 2048, x / w / g / gx 16-byte aligned. Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and safe. */
int ft_rms_norm_backward_noalloc(ft_context* ctx, const float* x, const float* w, const float* g,
                                 float* gx, float* gw, size_t rows, size_t size, float eps);

/* ---- RoPE (engine/attention.rs:21-83) ------------------------------------ */

/* ComputeEngine::rope_theta / rope_theta_inverse: in place on t[batch, seq,
 * hidden]; token i of each row sits at position pos + i. */
int ft_rope_theta(ft_context* ctx, float* t, size_t batch, size_t seq, size_t hidden, size_t head_dim,
                  size_t pos, float theta);
int ft_rope_theta_inverse(ft_context* ctx, float* t, size_t batch, size_t seq, size_t hidden,
                          size_t head_dim, size_t pos, float theta);
/* Out-of-place form (saves the copy RoPENode::backward and Tensor::rope_theta
 * make first, autograd/src/lib.rs:509-533, 1122-1139). */
int ft_rope_theta_to(ft_context* ctx, const float* src, float* dst, size_t batch, size_t seq,
                     size_t hidden, size_t head_dim, size_t pos, float theta, int inverse);

/* The (cos, sin) pairs of rope_theta for `seq` positions starting at `pos`:
 * table[seq][head_dim/2] float2 = (cos, sin)(position * theta^(-2i/head_dim)), computed exactly
 * as the rope kernel computes them; and the rotation of x [batch, seq, hidden] through such a
 * table (inverse != 0: the backward rotation). head_dim must be a multiple of 8 here. */
int ft_rope_table(ft_context* ctx, float* table, size_t seq, size_t head_dim, size_t pos, float theta);
int ft_rope_apply(ft_context* ctx, const float* x, float* out, size_t batch, size_t seq, size_t hidden,
                  size_t head_dim, const float* table, int inverse);

/* ---- attention (engine/attention.rs:165-177, 341-358, 581-594) ----------- */

/* AttentionOptions. window and dropout are not supported (0 only): the model
 * builder refuses windows (model_builder.rs:212-221) and every SmolLM2 config
 * has attention_dropout 0. */
typedef struct ft_attention_options {
    int32_t causal;
    uint32_t causal_offset;
    uint32_t window;
    float dropout_prob;
    uint64_t seed;
} ft_attention_options;

/* ComputeEngine::flash_attention_v2_with_stats. q/out [B,Sq,H,D], k/v
 * [B,Sk,Hkv,D], stats [B*H*Sq, 2] (slot 2*row+1 receives the row's
 * log-sum-exp, row = (b*H+h)*Sq+i); stats may be NULL. D <= 128. */
int ft_flash_attention_v2_with_stats(ft_context* ctx, const float* q, const float* k, const float* v,
                                     float* out, float* stats, size_t B, size_t Sq, size_t Sk,
                                     size_t H, size_t Hkv, size_t D, const ft_attention_options* opts);
/* ComputeEngine::flash_attention_v2_backward_with_stats: reads the saved
 * log-sum-exp, overwrites slot 2*row with Delta = dO.O, writes dq, dk, dv. */
int ft_flash_attention_v2_backward_with_stats(ft_context* ctx, const float* q, const float* k,
                                              const float* v, const float* out, const float* d_out,
                                              float* dq, float* dk, float* dv, float* stats, size_t B,
                                              size_t Sq, size_t Sk, size_t H, size_t Hkv, size_t D,
                                              const ft_attention_options* opts);

/* ---- elementwise (engine/elementwise.rs:8-17, 57-75, 183-216) ------------ */

/* ComputeEngine::add: out = a + b. */
int ft_add(ft_context* ctx, const float* a, const float* b, float* out, size_t n);
/* ComputeEngine::add_backward: ga = gb = g. */
int ft_add_backward(ft_context* ctx, const float* g, float* ga, float* gb, size_t n);
/* ComputeEngine::silu_gate_fused(first, second, out): out = silu(first) * second. */
int ft_silu_gate_fused(ft_context* ctx, const float* first, const float* second, float* out, size_t n);
/* ComputeEngine::silu_gate_backward(first, second, g, g_first, g_second). */
int ft_silu_gate_backward(ft_context* ctx, const float* first, const float* second, const float* g,
                          float* g_first, float* g_second, size_t n);

/* ---- training (engine/training.rs:54-76, 161-283) ------------------------ */

/* ComputeEngine::gradient_scale / clip_grad_by_norm: x *= scale, in place. */
int ft_gradient_scale(ft_context* ctx, float* x, size_t n, float scale);
int ft_clip_grad_by_norm(ft_context* ctx, float* x, size_t n, float scale);
/* ComputeEngine::gradient_accumulate: acc += g. */
int ft_gradient_accumulate(ft_context* ctx, float* acc, const float* g, size_t n);
/* ComputeEngine::sum_squares_partial: sum of x^2 per FT_SUM_SQUARES_CHUNK
 * elements into out[offset + b]; *chunks receives the number written. */
int ft_sum_squares_partial(ft_context* ctx, const float* x, size_t n, float* out, size_t offset,
                           size_t* chunks);
/* ComputeEngine::masked_cross_entropy_weighted: logits/grad [rows, vocab],
 * targets u32 [rows] (FT_MASKED_CE_SKIP = outside the loss), weights f32
 * [rows], row_loss [rows]. `grad_scale` multiplies the gradient (1.0 gives
 * the reference kernel; 1/grad_accum_steps folds the copy + gradient_scale of
 * MaskedCrossEntropyNode::backward, ferrotensor-trainer/src/lib.rs:553-572).
 * grad may alias logits. */
int ft_masked_cross_entropy_weighted(ft_context* ctx, const float* logits, const uint32_t* targets,
                                     const float* weights, float* grad, float* row_loss, size_t rows,
                                     size_t vocab, float grad_scale);

/* AdamParams (engine/training.rs:13-32). */
typedef struct ft_adam_params {
    float lr, beta1, beta2, eps, weight_decay, t;
} ft_adam_params;
/* ComputeEngine::adamw_update on one tensor. */
int ft_adamw_update(ft_context* ctx, float* w, const float* g, float* m, float* v, size_t n,
                    const ft_adam_params* p);
/* AdamW::apply_step over a list of tensors in one launch
 * (ferrotensor-autograd/src/lib.rs:1522-1552 issues one dispatch per tensor).
 * The four arrays hold `count` device pointers each (host memory), sizes the
 * element counts. `grad_scale` multiplies every gradient first (the clip scale
 * of Trainer::apply_gradients, trainer/src/lib.rs:336-343; 1.0 = none). */
int ft_adamw_update_multi(ft_context* ctx, float* const* w, const float* const* g, float* const* m,
                          float* const* v, const size_t* sizes, size_t count, const ft_adam_params* p,
                          float grad_scale);

/* ---- embedding gather (Tensor::embedding, autograd/src/lib.rs:1159-1179;
 *      done on the host in the reference) ------------------------------------ */

/* out[n, hidden] = table[ids[i]] or a zero row when ids[i] >= vocab. */
int ft_embedding(ft_context* ctx, const float* table, size_t vocab, size_t hidden, const uint32_t* ids,
                 size_t n, float* out);

/* ---- the step driver: Lfm2Model + Trainer over the ops above ------------- */

/* Lfm2Config fields the step uses (ferrotensor-loader/src/lib.rs:74-142). */
typedef struct ft_model_config {
    uint32_t vocab_size, hidden_size, intermediate_size, num_hidden_layers;
    uint32_t num_attention_heads, num_key_value_heads;
    float rms_norm_eps, rope_theta;
    int32_t tie_word_embeddings;
    int32_t f16_linears;   /* frozen linear weights stored as f16 (CLI default, main.rs:230-234) */
    /* Lfm2Model::with_block_checkpointing (lfm.rs:338-355): keep only each block's input
     * during training and recompute the block in backward (one extra forward per block). */
    int32_t checkpoint_blocks;
    /* 0 (default): training and evaluation run the final norm, the vocabulary head and the loss
     * on the supervised positions only. 1: on every position, as the reference does. A row's
     * results do not depend on which other rows share a launch, so both give the same bits,
     * unless the row count moves the head's input-gradient GEMM across the tile count at which
     * it splits K (a different summation order: rounding-level differences). */
    int32_t head_all_rows;
    /* Lfm2ModelBuilder::with_trainable_base (model_builder.rs:325-357): the linear weights are
     * stored f32 whatever f16_linears says, and they and the norm scales receive gradients and are
     * trained next to the adapters (`<prefix>.weight`, `...layernorm.weight`, `model.norm.weight`,
     * `lm_head.weight` in the parameter list; weight gradients in the stored [in, out] layout). The
     * embedding table stays frozen. 0 (default): LoRA factors only. */
    int32_t trainable_base;
} ft_model_config;

typedef struct ft_model ft_model;
typedef struct ft_trainer ft_trainer;

/* Lfm2ModelBuilder::build (model_builder.rs:623-709): an empty model; weights
 * arrive through ft_model_set_tensor. */
int ft_model_create(ft_context* ctx, const ft_model_config* cfg, ft_model** out);
int ft_model_destroy(ft_model* m);
/* Uploads one Hugging Face tensor by name (`model.embed_tokens.weight`,
 * `model.layers.N.self_attn.q_proj.weight` [out,in], `...input_layernorm.weight`,
 * `model.norm.weight`, `lm_head.weight`), applying the builder's rules
 * (model_builder.rs:400-424, 653-689): linears are transposed to [in,out] and
 * rounded to f16 when cfg.f16_linears; a tied head is the transposed embedding.
 * `<linear>.bias` [out] (model_builder.rs:454-469, Qwen2's query, key and value projections) is
 * kept f32 and added to every output row after the adapter's product, before RoPE and the
 * residual (Linear::project_2d, graph/src/lib.rs:128-139); with cfg.trainable_base it is trained
 * and listed after `<linear>.weight` (Linear::params, graph/src/lib.rs:180-188). A biased
 * projection takes separate bias and RoPE kernels instead of the fused GEMM epilogues. */
int ft_model_set_tensor(ft_model* m, const char* hf_name, const float* data, const size_t* shape, int ndim);
/* Attaches a LoRA adapter (LoRAAdapter, graph/src/lib.rs:28-98) to the linear
 * named `prefix` (`model.layers.N.self_attn.q_proj`, `lm_head`, ...):
 * a [in, rank], b [rank, out], both copied. */
int ft_model_set_lora(ft_model* m, const char* prefix, const float* a, const float* b, size_t rank, float alpha);
/* lora_seed (model_builder.rs:739-759): the seed of the adapter of `module_name`
 * ("q_proj", ...) in the layer with seed `layer_seed` (layer index + 1; 0 for
 * lm_head). Pure integer arithmetic, bit-exact with the reference's pinned values. */
uint64_t ft_lora_seed(uint64_t layer_seed, const char* module_name);
/* LoRAAdapter::new_seeded (graph/src/lib.rs:59-92): fills a[in_dim*rank] (host
 * memory) with xorshift64* draws, uniform in +-1/sqrt(in_dim). */
int ft_lora_init_a(float* a_host, size_t in_dim, size_t out_dim, size_t rank, uint64_t seed);
/* ModelBuilder::maybe_add_lora (model_builder.rs:425-446): attaches a freshly
 * initialised adapter (seeded A, zero B) to the linear named `prefix`. */
int ft_model_add_lora(ft_model* m, const char* prefix, size_t rank, float alpha);
/* Switches ft_model_config.head_all_rows after creation: 1 = the head runs on every position, as
 * Lfm2Model::forward_batch_with_dropout does (lfm.rs:597-623); 0 = on the supervised ones only. */
int ft_model_set_head_all_rows(ft_model* m, int all_rows);
/* Number of trainable tensors and their fixture names / sizes, in the order
 * gradients and parameters are reported (`<prefix>.lora_a`, `<prefix>.lora_b`). */
int ft_model_param_count(ft_model* m, size_t* count);
int ft_model_param_info(ft_model* m, size_t index, const char** name, size_t* numel);
/* Copies parameter / gradient `index` to the host (numel f32 values). The
 * gradient is the one the last step left (scaled by 1/grad_accum, unclipped). */
int ft_model_read_param(ft_model* m, size_t index, float* out_host);
/* Overwrites parameter `index` with numel f32 values from the host, in place: what
 * apply_checkpoint does to an existing tensor (ferrotensor-trainer/src/checkpoint.rs:275-283). */
int ft_model_write_param(ft_model* m, size_t index, const float* host);
int ft_model_read_grad(ft_model* m, size_t index, float* out_host);
/* Lfm2Model::forward_batch (lfm.rs:590-623): logits [B*S, vocab] to the host. */
int ft_model_forward_logits(ft_model* m, const uint32_t* rows, size_t B, size_t S, float* logits_host);

/* The forward-only loss of `evaluate` (ferrotensor-cli/src/main.rs:1110-1137: no_grad forward +
 * masked cross-entropy): per sequence, the mean loss over its supervised targets and their count,
 * for B equally long rows (pad as for training). Nothing is kept for backward and no gradient
 * or parameter is touched. */
int ft_model_eval_chunk(ft_model* m, const uint32_t* rows, const uint32_t* targets, const uint8_t* loss_mask,
                        size_t B, size_t S, float* per_sequence_loss, uint32_t* per_sequence_tokens);

/* Trainer::new + with_clip_grad_norm (trainer/src/lib.rs:113-205) with an
 * AdamW (autograd/src/lib.rs:1502-1515). clip_grad_norm <= 0 disables
 * clipping. */
typedef struct ft_trainer_config {
    float lr, beta1, beta2, eps, weight_decay;
    float clip_grad_norm;
    uint32_t grad_accum_steps;   /* 0 = the chunk's number of sequences */
    /* Trainer::with_lr_scheduler (trainer/src/lib.rs:172-176): FT_LR_CONSTANT keeps `lr`;
     * otherwise optimizer step k (1-based) uses ft_lr_schedule(.., k) with peak `lr`
     * (apply_gradients, trainer/src/lib.rs:345-352). A skipped step (non-finite
     * gradient norm) does not advance the schedule. */
    uint32_t lr_schedule;
    uint32_t warmup_steps;
    uint32_t total_steps;
    float min_lr;
} ft_trainer_config;

#define FT_LR_CONSTANT 0u
#define FT_LR_COSINE 1u         /* CosineAnnealingLR (autograd/src/lib.rs:1717-1758) */
#define FT_LR_WARMUP_COSINE 2u  /* WarmupCosineScheduler (autograd/src/lib.rs:1761-1814) */

/* LRScheduler::get_lr after `step` calls of step() (f32 arithmetic as in the
 * reference): cosine from peak to min over total_steps, or linear warm-up from 0
 * to peak over warmup_steps followed by the cosine to min at total_steps. Host
 * only; never touches the GPU. */
float ft_lr_schedule(uint32_t kind, float peak_lr, float min_lr, uint32_t warmup_steps, uint32_t total_steps,
                     uint32_t step);

/* StepStats of a chunk (trainer/src/lib.rs:36-58). */
typedef struct ft_step_stats {
    float loss;            /* sum of the per-sequence mean losses */
    float grad_norm;
    float clip_scale;      /* 1.0 when not clipped */
    uint32_t supervised_tokens;
    int32_t optimizer_step;
    float lr;              /* the rate the optimizer step used (0 when no step was taken) */
} ft_step_stats;

int ft_trainer_create(ft_model* m, const ft_trainer_config* cfg, ft_trainer** out);
int ft_trainer_destroy(ft_trainer* t);
/* Trainer::optimizer_steps / set_optimizer_steps (trainer/src/lib.rs:199-213): the
 * number of optimizer steps taken; setting it (resume) also advances the schedule. */
/* AdamW::state / load_state (autograd/src/lib.rs:1554-1640): the first and second
 * moments of trainable tensor `index` (the order of ft_model_param_info) to / from
 * host memory, and the optimizer's f32 step counter `t`. */
int ft_trainer_read_moments(ft_trainer* t, size_t index, float* m_host, float* v_host);
int ft_trainer_write_moments(ft_trainer* t, size_t index, const float* m_host, const float* v_host);
int ft_trainer_get_adam_t(ft_trainer* t, float* steps);
int ft_trainer_set_adam_t(ft_trainer* t, float steps);
/* The hyperparameters AdamW::load_state restores with the moments (autograd/src/lib.rs:1644-1649:
 * lr, beta1, beta2, eps, weight_decay of the saved optimizer). With a schedule the rate is
 * overwritten before every step (LRScheduler::step), so `lr` is only taken with FT_LR_CONSTANT. */
int ft_trainer_set_adam_hyper(ft_trainer* t, float lr, float beta1, float beta2, float eps,
                              float weight_decay);
int ft_trainer_optimizer_steps(ft_trainer* t, size_t* steps);
int ft_trainer_set_optimizer_steps(ft_trainer* t, size_t steps);
/* ---- Trainer::train_batch and the padding of train_chunk: host-side integer work ----
 * No device is touched; every array is host memory. */

/* Trainer::train_batch, which sequences of a Batch train (trainer/src/lib.rs:377-395). The batch is
 * [batch, padded_len] row-major (padded_input_ids, padded_target_ids, attention_mask, loss_masks).
 * A row is cut where its attention mask first differs from 1; it is dropped (valid_len[b] = 0)
 * when fewer than 2 tokens remain or no position of the cut loss mask is non-zero. `kept` = rows
 * with valid_len > 0. (The ids are not read; they are taken so the call mirrors the loop.) */
int ft_train_batch_select(const uint32_t* input_ids, const uint32_t* target_ids,
                          const uint8_t* attention_mask, const uint8_t* loss_mask, size_t batch,
                          size_t padded_len, size_t* valid_len, size_t* kept);
/* Trainer::train_batch, where the chunks end (trainer/src/lib.rs:408-421): chunk i takes
 * chunk_sizes[i] of the kept sequences, in order; a chunk stops at the accumulation boundary
 * (room = max(grad_accum_steps - step_in_accum, 1)), so the optimizer steps after the same
 * sequence as in the one-at-a-time path. `step_in_accum` is ft_trainer_step_in_accum before the
 * first chunk. grad_accum_steps 0 (the chunk's own size, ft_trainer_config) gives one chunk.
 * chunk_sizes must hold `sequences` entries. */
int ft_train_batch_plan(size_t sequences, size_t grad_accum_steps, size_t step_in_accum,
                        size_t* chunk_sizes, size_t* chunks);
/* Trainer::train_chunk, the common row length (trainer/src/lib.rs:431-436): the longest
 * min(input, target) length rounded up to a multiple of length_bucket (Trainer::length_bucket,
 * 32 by default, :132). */
int ft_chunk_padded_len(const size_t* input_lens, const size_t* target_lens, size_t count,
                        size_t length_bucket, size_t* padded_len);
/* Trainer::train_chunk, the padding (trainer/src/lib.rs:437-450): sequence s is cut to
 * min(input_lens[s], target_lens[s]) tokens and right-padded to padded_len with its last input
 * token (inputs and targets alike), loss mask 0; a loss mask shorter than the sequence counts as 0
 * past its end. rows / targets / masks are [count, padded_len], ready for ft_trainer_train_chunk. */
int ft_pad_chunk(const uint32_t* const* input_ids, const uint32_t* const* target_ids,
                 const uint8_t* const* loss_masks, const size_t* input_lens,
                 const size_t* target_lens, const size_t* mask_lens, size_t count, size_t padded_len,
                 uint32_t* rows, uint32_t* targets, uint8_t* masks);

/* Trainer::step_in_accum (trainer/src/lib.rs:463-466): sequences counted into the open
 * accumulation window. train_batch cuts its chunks at grad_accum_steps minus this, so the
 * optimizer steps after the same sequence as in the one-at-a-time path (:413-423). */
int ft_trainer_step_in_accum(ft_trainer* t, size_t* sequences);
/* Trainer::train_chunk (trainer/src/lib.rs:426-502) for B equally long rows
 * (already padded: ft_pad_chunk): forward, masked cross-entropy, backward
 * with seed 1/grad_accum_steps, gradient norm, clip, AdamW. rows/targets are
 * [B,S] u32 and loss_mask [B,S] u8 in host memory; per_sequence_loss (B
 * values) may be NULL. `apply` = 0 stops after backward (gradients readable,
 * no optimizer step). The final norm, the vocabulary head and the loss run on
 * the supervised positions only (a position without a target has zero loss and
 * a zero logits gradient, kernels.wgsl:684-711; see ft_model_config.head_all_rows);
 * ft_model_forward_logits still returns the logits of every position.
 * Accumulation follows the reference: the sequences of a chunk count towards
 * grad_accum_steps; the chunk that fills the window takes the norm / clip /
 * optimizer step; a chunk without a supervised token runs no backward, and a
 * window in which no chunk had one takes no step (apply_gradients returns early,
 * trainer/src/lib.rs:301-307: grad_norm 0, optimizer_step 0). */
int ft_trainer_train_chunk(ft_trainer* t, const uint32_t* rows, const uint32_t* targets,
                           const uint8_t* loss_mask, size_t B, size_t S, int apply,
                           ft_step_stats* stats, float* per_sequence_loss);

#ifdef __cplusplus
}
#endif
#endif /* FERROTENSOR_HIP_H */
