// Host driver of one LoRA training step over the kernels of this library: the
// part of the reference that sits above ComputeEngine on the hot path.
//
//   model     Lfm2Model / Lfm2Block / Attention / MLP / Linear(+LoRAAdapter)
//             ferrotensor-graph/src/lfm.rs:116-139, 597-623;
//             ferrotensor-graph/src/lib.rs:112-142, 367-414, 504-510
//   builder   transpose [out,in] -> [in,out], f16 storage, tied head
//             ferrotensor-graph/src/model_builder.rs:400-424, 653-689
//   loss      masked_cross_entropy_batch, ferrotensor-trainer/src/lib.rs:676-752
//   backward  the node rules of ferrotensor-autograd/src/lib.rs (MatMulNode
//             :262-290, AddNode, ScaleNode, RoPENode :509-533, RMSNormNode
//             :575-595, SiLUGateNode, FlashAttentionNode :1328-1390)
//   step      Trainer::train_chunk / apply_gradients / global_grad_norm,
//             trainer/src/lib.rs:296-360, 426-534; AdamW::apply_step,
//             autograd/src/lib.rs:1522-1552
//
// The reference records a tape and walks it; the step's graph is static, so
// forward and backward are written out here and every buffer is allocated once
// per (batch, sequence) shape and kept. A chunk's host arrays go up in one copy
// from pinned memory before the first kernel, and nothing waits for the GPU until
// the per-row losses and the gradient norm come back in one copy at its end.
#include "ft_common.h"
#include "ft_thin.h"

#include <cmath>
#include <cstring>
#include <memory>
#include <string>

// Defined in ft_rowops.hip.
struct ft_segment {
    float* w;
    float* g;
    float* m;
    float* v;
    uint32_t n;
};
int ft_internal_multi_grad_norm(ft_context* ctx, const ft_segment* segs_dev, size_t nseg, float* partials_dev,
                                float max_norm, float* control_dev);
int ft_internal_rms_norm_backward_add(ft_context* ctx, const float* x, const float* w, const float* g,
                                      const float* add, float* gx, size_t rows, size_t size, float eps);
int ft_internal_rope_table(ft_context* ctx, float* table, size_t seq, size_t head_dim, size_t pos, float theta);
int ft_internal_rope_pair(ft_context* ctx, const float* a_src, float* a_dst, size_t heads_a, const float* b_src,
                          float* b_dst, size_t heads_b, const float* table, size_t batch, size_t seq,
                          size_t head_dim, int inverse);
bool ft_internal_norm_can_sum(size_t rows, size_t size);
int ft_internal_rms_norm_sum(ft_context* ctx, const ft_deferred_sum* d, float* x_out, const float* w, float* out,
                             size_t rows, size_t size, float eps);
int ft_internal_rms_norm_backward_sum(ft_context* ctx, const float* x, const float* w, const ft_deferred_sum* d,
                                      const float* add, float* gx, size_t rows, size_t size, float eps);
int ft_internal_row_bias_add(ft_context* ctx, float* y, const float* bias, size_t rows, size_t cols);
int ft_internal_col_sum(ft_context* ctx, const float* g, float* out, size_t rows, size_t cols, int accumulate);
bool ft_internal_attention_rope_fusable(const float* q, const float* k, const float* v, const float* out,
                                        const float* d_out, size_t Sq, size_t Sk, size_t D);
int ft_internal_attention_backward_rope(ft_context* ctx, const float* q, const float* k, const float* v,
                                        const float* out, const float* d_out, float* dq, float* dk, float* dv,
                                        float* stats, size_t B, size_t S, size_t H, size_t Hkv,
                                        const ft_attention_options* opts, const float* rope_table);
int ft_internal_multi_adamw(ft_context* ctx, const ft_segment* segs_dev, size_t nseg, const ft_adam_params* p,
                            float grad_scale, const float* control_dev);

namespace {

constexpr float kF32Epsilon = 1.1920929e-07f;

struct LinearW {
    std::string prefix;
    size_t in = 0, out = 0;
    void* w = nullptr;
    int dtype = FT_DTYPE_F32;
    size_t r = 0;
    float alpha = 0.0f;
    float* a = nullptr;   // [in, r]
    float* b = nullptr;   // [r, out]
    float* ga = nullptr;
    float* gb = nullptr;
    float* gw = nullptr;  // gradient of w [in, out] when the base trains
    float* bias = nullptr;   // [out], f32 (graph/src/lib.rs:105-106: Qwen2 query, key and value projections)
    float* gbias = nullptr;  // its gradient when the base trains
    bool has_lora() const { return r > 0; }
    // graph/src/lib.rs:119-122: the scale is alpha / rank, skipped when it is exactly 1.
    float scale() const {
        const float s = alpha / (float)r;
        return std::fabs(s - 1.0f) > kF32Epsilon ? s : 1.0f;
    }
};

struct Layer {
    float* norm1 = nullptr;
    float* norm2 = nullptr;
    float* gnorm1 = nullptr;  // gradients of the norm scales when the base trains
    float* gnorm2 = nullptr;
    LinearW q, k, v, o, gate, up, down;
    LinearW* all[7] = {&q, &k, &v, &o, &gate, &up, &down};
};

struct ParamRef {
    std::string name;
    float* w;
    float* g;
    size_t n;
};

// Activations of one layer kept for backward.
struct LayerActs {
    float *x, *h1, *q, *k, *v, *attn, *stats, *h, *h2, *gate, *up, *act;
    float *tq, *tk, *tv, *to, *tgate, *tup, *tdown;
};

}  // namespace

struct ft_model {
    ft_context* ctx = nullptr;
    ft_model_config cfg{};
    float* embed = nullptr;
    std::vector<Layer> layers;
    float* norm_f = nullptr;
    float* gnorm_f = nullptr;
    LinearW lm_head;
    std::vector<ParamRef> params;
    bool params_dirty = true;
    // Bumped whenever an adapter's buffers are (re)allocated: a trainer holds raw pointers into
    // them and sizes its moments from them, so it is only valid for the generation it was made in.
    uint64_t param_generation = 0;

    // Step buffers, valid for (ws_B, ws_S).
    size_t ws_B = 0, ws_S = 0;
    std::vector<void*> ws_allocs;
    std::vector<LayerActs> acts;
    float *x_final = nullptr, *hf = nullptr, *thead = nullptr, *logits = nullptr;
    // Everything a chunk sends to the device (token ids, head row indices both ways, targets, row
    // weights: 5 arrays of T words) is written into one pinned staging buffer and goes up in one
    // copy before the first kernel; the per-row losses and the trainer's control block (3 words at
    // step_out + T) come back in one copy into pinned memory at the end: the step's only wait.
    uint32_t *io_host = nullptr, *io_dev = nullptr;
    float *out_host = nullptr, *step_out = nullptr;
    uint32_t *ids_dev = nullptr, *targets_dev = nullptr;
    float *weights_dev = nullptr, *row_loss = nullptr, *control = nullptr;
    // Head on the supervised rows only: head_idx[k] = k-th supervised row, head_inv[row] = its k
    // (or head_rows for an unsupervised row, which gathers as a zero row), xc = those rows of x_final.
    uint32_t *head_idx_dev = nullptr, *head_inv_dev = nullptr;
    float* xc = nullptr;
    size_t head_rows = 0;        // rows the head ran on in the last forward
    bool head_compact = false;   // whether they are a gathered subset
    // backward scratch
    float *g0 = nullptr, *g1 = nullptr, *d_act = nullptr, *d_gate = nullptr, *d_up = nullptr, *d_h2 = nullptr,
          *d_attn = nullptr, *dq = nullptr, *dk = nullptr, *dv = nullptr, *d_h1 = nullptr, *dt = nullptr,
          *dt2 = nullptr, *dt3 = nullptr, *gtmp = nullptr, *rope_table = nullptr;
    // Factor gradients (dA, dB) waiting for their launch: the products of a block's adapted linears
    // go out together in batched launches (flush_cols), before anything they read is rewritten.
    // Each waiting linear keeps its own dT buffer from dt_pool until then.
    static constexpr int kDtPool = 8;
    float* dt_pool[kDtPool] = {};
    int dt_used = 0;
    std::vector<ft_thin_problem> pending_cols;
    // The down projection of the block before, when its K shares were left for this block's first norm to add.
    ft_deferred_sum pending_x;

    size_t head_dim() const { return cfg.hidden_size / cfg.num_attention_heads; }
};

struct ft_trainer {
    ft_model* model = nullptr;
    ft_trainer_config cfg{};
    uint64_t generation = 0;        // the model's param_generation this trainer was built for
    std::vector<size_t> numel;      // elements of m[i] / v[i]
    float t = 0.0f;                 // AdamW step counter (f32, as in the reference)
    size_t optimizer_steps = 0;     // steps taken = position of the LR schedule
    size_t step_in_accum = 0;
    bool window_has_grads = false;  // a backward pass has written the gradient buffers in this window
    std::vector<float*> m, v;       // per parameter
    ft_segment* segs_dev = nullptr;
    size_t nseg = 0;
    float* partials = nullptr;
};

namespace {

int alloc_f(ft_context* ctx, size_t n, float** out) { return ft_alloc(ctx, n * sizeof(float), (void**)out); }

int ws_alloc(ft_model* m, size_t n, float** out) {
    FT_TRY(alloc_f(m->ctx, n, out));
    m->ws_allocs.push_back(*out);
    return FT_OK;
}

void ws_free(ft_model* m) {
    for (void* p : m->ws_allocs) (void)ft_free(m->ctx, p);
    m->ws_allocs.clear();
    if (m->io_host) (void)hipHostFree(m->io_host);
    if (m->out_host) (void)hipHostFree(m->out_host);
    m->io_host = nullptr;
    m->out_host = nullptr;
    m->control = nullptr;
    m->step_out = nullptr;
    m->acts.clear();
    m->ws_B = m->ws_S = 0;
}

int ensure_workspace(ft_model* m, size_t B, size_t S) {
    if (m->ws_B == B && m->ws_S == S) return FT_OK;
    ws_free(m);
    const ft_model_config& c = m->cfg;
    const size_t T = B * S, H = c.hidden_size, F = c.intermediate_size, V = c.vocab_size;
    const size_t D = m->head_dim(), QD = c.num_attention_heads * D, KD = c.num_key_value_heads * D;
    size_t rmax = m->lm_head.r;
    m->acts.resize(c.num_hidden_layers);
    // Block checkpointing (Lfm2Model::with_block_checkpointing, lfm.rs:338-355): only each
    // block's input is kept; every block shares one set of internal buffers, refilled by
    // recomputing the block's forward right before its backward.
    const bool ckpt = c.checkpoint_blocks != 0 && c.num_hidden_layers > 0;
    LayerActs shared{};
    for (size_t l = 0; l < c.num_hidden_layers; l++)
        for (int i = 0; i < 7; i++)
            if (m->layers[l].all[i]->r > rmax) rmax = m->layers[l].all[i]->r;
    for (size_t l = 0; l < c.num_hidden_layers; l++) {
        LayerActs& a = m->acts[l];
        Layer& L = m->layers[l];
        if (ckpt && l > 0) {
            a = shared;
            FT_TRY(ws_alloc(m, T * H, &a.x));
            continue;
        }
        FT_TRY(ws_alloc(m, T * H, &a.x));
        FT_TRY(ws_alloc(m, T * H, &a.h1));
        FT_TRY(ws_alloc(m, T * QD, &a.q));
        FT_TRY(ws_alloc(m, T * KD, &a.k));
        FT_TRY(ws_alloc(m, T * KD, &a.v));
        FT_TRY(ws_alloc(m, T * QD, &a.attn));
        FT_TRY(ws_alloc(m, B * c.num_attention_heads * S * 2, &a.stats));
        FT_TRY(ws_alloc(m, T * H, &a.h));
        FT_TRY(ws_alloc(m, T * H, &a.h2));
        FT_TRY(ws_alloc(m, T * F, &a.gate));
        FT_TRY(ws_alloc(m, T * F, &a.up));
        FT_TRY(ws_alloc(m, T * F, &a.act));
        float** ts[7] = {&a.tq, &a.tk, &a.tv, &a.to, &a.tgate, &a.tup, &a.tdown};
        for (int i = 0; i < 7; i++) {
            *ts[i] = nullptr;
            if (ckpt) {
                if (rmax > 0) FT_TRY(ws_alloc(m, T * rmax, ts[i]));  // any layer may have an adapter here
            } else if (L.all[i]->has_lora()) {
                FT_TRY(ws_alloc(m, T * L.all[i]->r, ts[i]));
            }
        }
        if (ckpt) shared = a;
    }
    FT_TRY(ws_alloc(m, T * H, &m->x_final));
    FT_TRY(ws_alloc(m, T * H, &m->hf));
    m->thead = nullptr;
    if (m->lm_head.has_lora()) FT_TRY(ws_alloc(m, T * m->lm_head.r, &m->thead));
    FT_TRY(ws_alloc(m, T * V, &m->logits));
    FT_TRY(ws_alloc(m, 5 * T, (float**)&m->io_dev));
    m->ids_dev = m->io_dev;
    m->head_idx_dev = m->io_dev + T;
    m->head_inv_dev = m->io_dev + 2 * T;
    m->targets_dev = m->io_dev + 3 * T;
    m->weights_dev = reinterpret_cast<float*>(m->io_dev + 4 * T);
    FT_TRY(ws_alloc(m, T + 4, &m->step_out));
    m->row_loss = m->step_out;
    m->control = m->step_out + T;
    FT_HIP(hipHostMalloc((void**)&m->io_host, 5 * T * sizeof(uint32_t), hipHostMallocDefault));
    FT_HIP(hipHostMalloc((void**)&m->out_host, (T + 4) * sizeof(float), hipHostMallocDefault));
    FT_TRY(ws_alloc(m, T * H, &m->xc));
    FT_TRY(ws_alloc(m, T * H, &m->g0));
    FT_TRY(ws_alloc(m, T * H, &m->g1));
    FT_TRY(ws_alloc(m, T * F, &m->d_act));
    FT_TRY(ws_alloc(m, T * F, &m->d_gate));
    FT_TRY(ws_alloc(m, T * F, &m->d_up));
    FT_TRY(ws_alloc(m, T * H, &m->d_h2));
    FT_TRY(ws_alloc(m, T * QD, &m->d_attn));
    FT_TRY(ws_alloc(m, T * QD, &m->dq));
    FT_TRY(ws_alloc(m, T * KD, &m->dk));
    FT_TRY(ws_alloc(m, T * KD, &m->dv));
    FT_TRY(ws_alloc(m, T * H, &m->d_h1));
    // (cos, sin) table of the rotary embedding; the vector kernel needs head_dim % 8 == 0
    m->rope_table = nullptr;
    if (m->head_dim() % 8 == 0) {
        FT_TRY(ws_alloc(m, S * m->head_dim(), &m->rope_table));
        FT_TRY(ft_internal_rope_table(m->ctx, m->rope_table, S, m->head_dim(), 0, c.rope_theta));
    }
    for (int i = 0; i < ft_model::kDtPool; i++) FT_TRY(ws_alloc(m, T * (rmax ? rmax : 1), &m->dt_pool[i]));
    m->dt = m->dt_pool[0];
    m->dt2 = m->dt_pool[1];
    m->dt3 = m->dt_pool[2];
    m->dt_used = 0;
    m->pending_cols.clear();
    size_t gmax = 1;
    for (auto& p : m->params) gmax = p.n > gmax ? p.n : gmax;
    FT_TRY(ws_alloc(m, gmax, &m->gtmp));
    m->ws_B = B;
    m->ws_S = S;
    return FT_OK;
}

// The trainable tensors in reporting order. With a trainable base (model_builder.rs:353-357) the
// linear weights and the norm scales are in it too, and their gradient buffers are made here.
int rebuild_params(ft_model* m) {
    m->params.clear();
    const bool base = m->cfg.trainable_base != 0;
    const size_t H = m->cfg.hidden_size;
    auto grad_buf = [&](float** g, size_t n) -> int {
        if (*g) return FT_OK;
        FT_TRY(alloc_f(m->ctx, n, g));
        return ft_zero(m->ctx, *g, n * 4);
    };
    auto add_norm = [&](const std::string& name, float* w, float** g) -> int {
        if (!base || !w) return FT_OK;
        FT_TRY(grad_buf(g, H));
        m->params.push_back({name, w, *g, H});
        return FT_OK;
    };
    auto add = [&](LinearW& l) -> int {
        if (base && l.w && l.dtype == FT_DTYPE_F32) {
            FT_TRY(grad_buf(&l.gw, l.in * l.out));
            m->params.push_back({l.prefix + ".weight", (float*)l.w, l.gw, l.in * l.out});
        }
        // Linear::params (graph/src/lib.rs:180-188): weight, bias, then the adapter
        if (base && l.bias) {
            FT_TRY(grad_buf(&l.gbias, l.out));
            m->params.push_back({l.prefix + ".bias", l.bias, l.gbias, l.out});
        }
        if (!l.has_lora()) return FT_OK;
        m->params.push_back({l.prefix + ".lora_a", l.a, l.ga, l.in * l.r});
        m->params.push_back({l.prefix + ".lora_b", l.b, l.gb, l.r * l.out});
        return FT_OK;
    };
    for (size_t li = 0; li < m->layers.size(); li++) {
        Layer& L = m->layers[li];
        const std::string p = "model.layers." + std::to_string(li);
        FT_TRY(add_norm(p + ".input_layernorm.weight", L.norm1, &L.gnorm1));
        for (auto* l : L.all) FT_TRY(add(*l));
        FT_TRY(add_norm(p + ".post_attention_layernorm.weight", L.norm2, &L.gnorm2));
    }
    FT_TRY(add_norm("model.norm.weight", m->norm_f, &m->gnorm_f));
    FT_TRY(add(m->lm_head));
    m->params_dirty = false;
    return FT_OK;
}

// t_i = scale_i * x @ A_i for up to 3 linears that read the same x: one
// launch when the adapters share a rank the vector kernel supports.
int lora_down_group(ft_context* ctx, LinearW* const* ls, float* const* ts, int n, const float* x, size_t T) {
    ft_thin_problem probs[3];
    int cnt = 0;
    bool batch = true;
    for (int i = 0; i < n; i++) {
        if (!ls[i]->has_lora()) continue;
        const LinearW& l = *ls[i];
        probs[cnt] = ft_thin_problem{x, l.a, ts[i], (int)T, (int)l.in, 0, (int)l.r, (long)l.in, (long)l.r, (long)l.r,
                                     l.scale(), 0, 0, 0, 0};
        batch = batch && ft_thin_rowwise_ok(probs[cnt]) && l.r == ls[0]->r;
        cnt++;
    }
    if (cnt == 0) return FT_OK;
    if (batch && cnt > 1) return ft_thin_rowwise(ctx, probs, cnt);
    for (int i = 0; i < n; i++)
        if (ls[i]->has_lora()) FT_TRY(ft_lora_down(ctx, x, ls[i]->a, ts[i], T, ls[i]->in, ls[i]->r, ls[i]->scale()));
    return FT_OK;
}

// y = x @ W (+ t @ B) with t = scale * x @ A already computed.
int linear_gemm(ft_context* ctx, const LinearW& l, const float* x, const float* t, float* y, size_t T,
                const float* residual = nullptr) {
    FT_CHECK_ARG(l.w, "linear %s has no weight", l.prefix.c_str());
    if (l.has_lora()) return ft_lora_linear(ctx, x, l.w, l.dtype, t, l.b, residual, y, T, l.in, l.out, l.r);
    return ft_lora_linear(ctx, x, l.w, l.dtype, nullptr, nullptr, residual, y, T, l.in, l.out, 0);
}

// y_i = x @ W_i (+ t_i @ B_i) for linears that share x, in one launch when they can be batched.
// The first `n_rope` outputs are rotated through RoPE in the GEMM epilogue when `rope_table` is given.
int linear_gemm_group(ft_context* ctx, LinearW* const* ls, const float* const* ts, float* const* ys, int n,
                      const float* x, size_t T, const float* rope_table = nullptr, size_t rope_seq = 0,
                      int n_rope = 0) {
    ft_lora_linear_desc d[3];
    for (int i = 0; i < n; i++) {
        const LinearW& l = *ls[i];
        FT_CHECK_ARG(l.w, "linear %s has no weight", l.prefix.c_str());
        FT_CHECK_ARG(l.in == ls[0]->in, "grouped linears must share their input width");
        d[i] = ft_lora_linear_desc{l.w, l.dtype, l.has_lora() ? ts[i] : nullptr, l.has_lora() ? l.b : nullptr,
                                   nullptr, ys[i], l.out, l.has_lora() ? l.r : 0,
                                   i < n_rope ? rope_table : nullptr, i < n_rope ? rope_seq : 0};
    }
    return ft_lora_linear_group(ctx, x, d, (size_t)n, T, ls[0]->in);
}

// y += bias on every row, for a linear that has one (graph/src/lib.rs:128-139: added after the adapter).
int linear_bias(ft_context* ctx, const LinearW& l, float* y, size_t T) {
    if (!l.bias) return FT_OK;
    return ft_internal_row_bias_add(ctx, y, l.bias, T, l.out);
}

// Offers the next GEMM launch on `ctx` the chance to leave its K shares unadded (the caller's next
// kernel is a norm that adds them while it reads the row). `d->pending()` afterwards: it did.
struct DeferScope {
    ft_context* ctx;
    DeferScope(ft_context* c, ft_deferred_sum* d, bool enable) : ctx(c) {
        *d = ft_deferred_sum{};
        c->defer = enable ? d : nullptr;
    }
    ~DeferScope() { ctx->defer = nullptr; }
};

// y = x @ W (+ (scale * x @ A) @ B) (+ bias) (+ residual), keeping t = scale * x @ A for backward.
// `defer` (optional): the product may leave its K shares unadded for the caller's next kernel.
int linear_forward(ft_context* ctx, LinearW& l, const float* x, float* t, float* y, size_t T,
                   const float* residual = nullptr, ft_deferred_sum* defer = nullptr) {
    LinearW* ls[1] = {&l};
    float* ts[1] = {t};
    FT_TRY(lora_down_group(ctx, ls, ts, 1, x, T));
    ft_deferred_sum unused;
    if (!l.bias) {
        DeferScope scope(ctx, defer ? defer : &unused, defer != nullptr);
        return linear_gemm(ctx, l, x, t, y, T, residual);
    }
    if (defer) *defer = ft_deferred_sum{};
    // the bias belongs to the linear's output, the residual is added to that sum afterwards
    FT_TRY(linear_gemm(ctx, l, x, t, y, T));
    FT_TRY(linear_bias(ctx, l, y, T));
    if (residual) FT_TRY(ft_add(ctx, residual, y, y, T * l.out));
    return FT_OK;
}

// Launches the waiting factor-gradient products in batches of equal rank; afterwards every dT
// buffer is free again (launches of one stream run in order).
int flush_cols(ft_model* m) {
    int rc = FT_OK;
    size_t i = 0;
    while (i < m->pending_cols.size() && rc == FT_OK) {
        size_t n = 1;
        while (i + n < m->pending_cols.size() && n < (size_t)FT_THIN_MAX_BATCH &&
               m->pending_cols[i + n].C == m->pending_cols[i].C)
            n++;
        rc = ft_thin_colwise(m->ctx, &m->pending_cols[i], (int)n);
        i += n;
    }
    m->pending_cols.clear();
    m->dt_used = 0;
    return rc;
}

// A dT buffer no waiting product reads.
int take_dt(ft_model* m, float** dt) {
    if (m->dt_used == ft_model::kDtPool) FT_TRY(flush_cols(m));
    *dt = m->dt_pool[m->dt_used++];
    return FT_OK;
}

// Gradients of one linear given dy: LoRA factor gradients (written, or added
// when `accumulate`), and dx when wanted (added to what dx holds when `dx_add`).
int linear_backward(ft_model* m, LinearW& l, const float* x, const float* t, const float* dy, float* dx, size_t T,
                    bool accumulate, bool dx_add = false) {
    ft_context* ctx = m->ctx;
    // the bias gradient is ones^T @ dy, the output gradient summed over the rows
    if (l.gbias) FT_TRY(ft_internal_col_sum(ctx, dy, l.gbias, T, l.out, accumulate ? 1 : 0));
    if (l.gw) {
        // trainable base: dW[in, out] = x^T @ dy (MatMulNode::backward, autograd/src/lib.rs:280-287)
        float* dst = accumulate ? m->gtmp : l.gw;
        FT_TRY(ft_matmul_at(ctx, x, dy, dst, l.in, T, l.out));
        if (accumulate) FT_TRY(ft_gradient_accumulate(ctx, l.gw, m->gtmp, l.in * l.out));
    }
    if (l.has_lora()) {
        float* dt = nullptr;
        // room for this linear's two products first: a flush frees every dT buffer
        if (m->pending_cols.size() + 2 > (size_t)FT_THIN_MAX_BATCH) FT_TRY(flush_cols(m));
        FT_TRY(take_dt(m, &dt));
        FT_TRY(ft_lora_grad_down(ctx, dy, l.b, dt, T, l.out, l.r, l.scale()));
        // dB = t^T dy and dA = x^T dt in one sliced launch when possible (added to the
        // gradients of the earlier micro-batches when `accumulate`).
        const int acc = accumulate ? 1 : 0;
        ft_thin_problem pb[2] = {
            {dy, t, l.gb, (int)T, 0, (int)l.out, (int)l.r, (long)l.out, (long)l.r, (long)l.out, 1.0f, 0, 1, 0, acc},
            {x, dt, l.ga, (int)T, 0, (int)l.in, (int)l.r, (long)l.in, (long)l.r, (long)l.r, 1.0f, 0, 0, 0, acc}};
        if (ft_thin_colwise_ok(pb[0]) && ft_thin_colwise_ok(pb[1])) {
            // Only the optimizer reads dA and dB: they wait for the block's batched launch.
            m->pending_cols.push_back(pb[0]);
            m->pending_cols.push_back(pb[1]);
        } else if (accumulate) {
            FT_TRY(ft_lora_grad_b(ctx, t, dy, m->gtmp, T, l.out, l.r));
            FT_TRY(ft_gradient_accumulate(ctx, l.gb, m->gtmp, l.r * l.out));
            FT_TRY(ft_lora_grad_a(ctx, x, dt, m->gtmp, T, l.in, l.r));
            FT_TRY(ft_gradient_accumulate(ctx, l.ga, m->gtmp, l.in * l.r));
        } else {
            FT_TRY(ft_lora_grad_b(ctx, t, dy, l.gb, T, l.out, l.r));
            FT_TRY(ft_lora_grad_a(ctx, x, dt, l.ga, T, l.in, l.r));
        }
        if (dx)
            FT_TRY(ft_lora_linear_dx(ctx, dy, l.w, l.dtype, dt, l.a, dx_add ? dx : nullptr, dx, T, l.in, l.out,
                                     l.r));
    } else if (dx) {
        FT_TRY(ft_lora_linear_dx(ctx, dy, l.w, l.dtype, nullptr, nullptr, dx_add ? dx : nullptr, dx, T, l.in, l.out,
                                 0));
    }
    return FT_OK;
}

// The same for up to 3 linears that share their input x (q/k/v, gate/up): the
// dT, dA and dB products of all of them go into two batched launches. The input
// gradients are summed into dx (NULL: not wanted) by one GEMM whose K loop runs
// over all the output gradients. Falls back to one linear at a time when the
// adapters cannot be batched.
// `defer` (optional): the summed input gradient may be left as K shares for the norm backward that reads it next.
int linear_backward_group(ft_model* m, LinearW* const* ls, const float* const* ts, const float* const* dys,
                          float* dx, int n, const float* x, size_t T, bool accumulate, bool flush,
                          ft_deferred_sum* defer = nullptr) {
    ft_context* ctx = m->ctx;
    ft_deferred_sum unused;
    if (defer) *defer = ft_deferred_sum{};
    bool batch = n <= 3;
    bool any_gw = false;
    for (int i = 0; i < n; i++) {
        batch = batch && ls[i]->has_lora() && ls[i]->r == ls[0]->r && !ls[i]->gw && !ls[i]->gbias;
        any_gw = any_gw || ls[i]->gw != nullptr || ls[i]->gbias != nullptr;
    }
    float* dts[3] = {nullptr, nullptr, nullptr};
    if (batch) {
        // room for this group's products and dT buffers first: a flush frees every dT buffer
        if (m->dt_used + n > ft_model::kDtPool || m->pending_cols.size() + 2 * (size_t)n > (size_t)FT_THIN_MAX_BATCH)
            FT_TRY(flush_cols(m));
        for (int i = 0; i < n; i++) FT_TRY(take_dt(m, &dts[i]));
    }
    const int acc = accumulate ? 1 : 0;
    ft_thin_problem rows[3], cols[6];
    for (int i = 0; i < n && batch; i++) {
        const LinearW& l = *ls[i];
        rows[i] = ft_thin_problem{dys[i], l.b, dts[i], (int)T, (int)l.out, 0, (int)l.r, (long)l.out, (long)l.out,
                                  (long)l.r, l.scale(), 1, 0, 0, 0};
        cols[2 * i] = ft_thin_problem{dys[i], ts[i], l.gb, (int)T, 0, (int)l.out, (int)l.r, (long)l.out, (long)l.r,
                                      (long)l.out, 1.0f, 0, 1, 0, acc};
        cols[2 * i + 1] = ft_thin_problem{x, dts[i], l.ga, (int)T, 0, (int)l.in, (int)l.r, (long)l.in, (long)l.r,
                                          (long)l.r, 1.0f, 0, 0, 0, acc};
        batch = ft_thin_rowwise_ok(rows[i]) && ft_thin_colwise_ok(cols[2 * i]) && ft_thin_colwise_ok(cols[2 * i + 1]);
    }
    if (!batch) {
        bool any_lora = false;
        for (int i = 0; i < n; i++) any_lora = any_lora || ls[i]->has_lora();
        if (any_lora || any_gw || n > 3) {
            for (int i = 0; i < n; i++)
                FT_TRY(linear_backward(m, *ls[i], x, ts[i], dys[i], dx, T, accumulate, i > 0));
            if (flush) FT_TRY(flush_cols(m));
            return FT_OK;
        }
        // frozen linears: only the summed input gradient is wanted
        if (flush) FT_TRY(flush_cols(m));
        if (!dx) return FT_OK;
        ft_lora_dx_desc d[3];
        for (int i = 0; i < n; i++) d[i] = ft_lora_dx_desc{dys[i], ls[i]->w, ls[i]->dtype, nullptr, nullptr, ls[i]->out, 0};
        DeferScope scope(ctx, defer ? defer : &unused, defer != nullptr);
        return ft_lora_linear_dx_group(ctx, d, (size_t)n, nullptr, dx, T, ls[0]->in);
    }
    FT_TRY(ft_thin_rowwise(ctx, rows, n));
    for (int i = 0; i < 2 * n; i++) m->pending_cols.push_back(cols[i]);
    if (flush) FT_TRY(flush_cols(m));
    if (dx) {
        ft_lora_dx_desc d[3];
        for (int i = 0; i < n; i++)
            d[i] = ft_lora_dx_desc{dys[i], ls[i]->w, ls[i]->dtype, dts[i], ls[i]->a, ls[i]->out, ls[i]->r};
        DeferScope scope(ctx, defer ? defer : &unused, defer != nullptr);
        FT_TRY(ft_lora_linear_dx_group(ctx, d, (size_t)n, nullptr, dx, T, ls[0]->in));
    }
    return FT_OK;
}

// One transformer block: acts[l].x -> acts[l + 1].x (or x_final), filling acts[l].
// `defer_tail`: the next kernel after this block is the next block's first norm (the plain forward pass, not a
// recomputation), so the down projection may leave its K shares to it (m->pending_x).
int layer_forward(ft_model* m, size_t l, size_t B, size_t S, bool defer_tail = false) {
    ft_context* ctx = m->ctx;
    const ft_model_config& c = m->cfg;
    const size_t T = B * S, H = c.hidden_size, F = c.intermediate_size;
    const size_t D = m->head_dim(), nh = c.num_attention_heads, nkv = c.num_key_value_heads;
    ft_attention_options opts{};
    opts.causal = 1;
    {
        Layer& L = m->layers[l];
        LayerActs& a = m->acts[l];
        float* x_next = l + 1 < m->layers.size() ? m->acts[l + 1].x : m->x_final;
        if (m->pending_x.pending()) {
            FT_TRY(ft_internal_rms_norm_sum(ctx, &m->pending_x, a.x, L.norm1, a.h1, T, H, c.rms_norm_eps));
            m->pending_x = ft_deferred_sum{};
        } else {
            FT_TRY(ft_rms_norm_eps(ctx, a.x, L.norm1, a.h1, T, H, c.rms_norm_eps));
        }
        {
            LinearW* ls[3] = {&L.q, &L.k, &L.v};
            float* ts[3] = {a.tq, a.tk, a.tv};
            FT_TRY(lora_down_group(ctx, ls, ts, 3, a.h1, T));
        }
        bool fused_rope = false;
        {
            LinearW* ls[3] = {&L.q, &L.k, &L.v};
            const float* ts[3] = {a.tq, a.tk, a.tv};
            float* ys[3] = {a.q, a.k, a.v};
            // head_dim 64: q and k leave the GEMM already rotated (a biased projection is rotated after
            // its bias, so it takes the separate kernel)
            fused_rope = m->rope_table && D == 64 && !L.q.bias && !L.k.bias;
            FT_TRY(linear_gemm_group(ctx, ls, ts, ys, 3, a.h1, T, fused_rope ? m->rope_table : nullptr, S,
                                     fused_rope ? 2 : 0));
            for (int i = 0; i < 3; i++) FT_TRY(linear_bias(ctx, *ls[i], ys[i], T));
        }
        if (fused_rope) {
        } else if (m->rope_table) {
            FT_TRY(ft_internal_rope_pair(ctx, a.q, a.q, nh, a.k, a.k, nkv, m->rope_table, B, S, D, 0));
        } else {
            FT_TRY(ft_rope_theta(ctx, a.q, B, S, nh * D, D, 0, c.rope_theta));
            FT_TRY(ft_rope_theta(ctx, a.k, B, S, nkv * D, D, 0, c.rope_theta));
        }
        FT_TRY(ft_flash_attention_v2_with_stats(ctx, a.q, a.k, a.v, a.attn, a.stats, B, S, S, nh, nkv, D, &opts));
        // h = x + o_proj(attn): the residual is added in the GEMM epilogue, or, when the product's K is shared
        // out over workgroups, by the norm kernel that reads h next
        const bool can_sum = ft_internal_norm_can_sum(T, H);
        {
            ft_deferred_sum d;
            FT_TRY(linear_forward(ctx, L.o, a.attn, a.to, a.h, T, a.x, can_sum ? &d : nullptr));
            if (d.pending())
                FT_TRY(ft_internal_rms_norm_sum(ctx, &d, a.h, L.norm2, a.h2, T, H, c.rms_norm_eps));
            else
                FT_TRY(ft_rms_norm_eps(ctx, a.h, L.norm2, a.h2, T, H, c.rms_norm_eps));
        }
        {
            LinearW* ls[2] = {&L.up, &L.gate};
            float* ts[2] = {a.tup, a.tgate};
            FT_TRY(lora_down_group(ctx, ls, ts, 2, a.h2, T));
        }
        if (!L.up.has_lora() && !L.gate.has_lora() && L.up.dtype == L.gate.dtype && !L.up.bias && !L.gate.bias) {
            FT_TRY(ft_mlp_gate_up(ctx, a.h2, L.gate.w, L.up.w, L.up.dtype, a.gate, a.up, a.act, T, H, F));
        } else {
            LinearW* ls[2] = {&L.up, &L.gate};
            const float* ts[2] = {a.tup, a.tgate};
            float* ys[2] = {a.up, a.gate};
            FT_TRY(linear_gemm_group(ctx, ls, ts, ys, 2, a.h2, T));
            for (int i = 0; i < 2; i++) FT_TRY(linear_bias(ctx, *ls[i], ys[i], T));
            FT_TRY(ft_silu_gate_fused(ctx, a.gate, a.up, a.act, T * F));
        }
        m->pending_x = ft_deferred_sum{};
        FT_TRY(linear_forward(ctx, L.down, a.act, a.tdown, x_next, T, a.h,
                              defer_tail && can_sum && l + 1 < m->layers.size() ? &m->pending_x : nullptr));
    }
    return FT_OK;
}

// Stages a chunk's host arrays and sends them to the device in one copy.
// `head` (optional): the rows whose logits are needed, ascending, with their targets and weights.
// The final norm and the vocabulary head then run on those rows only (logits, row losses and
// d_logits are [head->size(), V]): a row without a supervised target has zero loss and a zero
// logits gradient whatever its logits are (masked_cross_entropy, kernels.wgsl:684-711), so leaving
// it out changes no bit of the result. With `head_all_rows` (or no `head`) every row goes through
// the head, unsupervised ones with MASKED_CE_SKIP and weight 0.
int stage_chunk(ft_model* m, const uint32_t* rows_host, size_t B, size_t S, const std::vector<uint32_t>* head,
                const std::vector<uint32_t>* tg, const std::vector<float>* wt) {
    ft_context* ctx = m->ctx;
    const ft_model_config& c = m->cfg;
    FT_CHECK_ARG(m->embed && m->norm_f && m->lm_head.w, "model is missing embed_tokens, norm or lm_head weights");
    for (auto& L : m->layers) {
        FT_CHECK_ARG(L.norm1 && L.norm2, "a layer is missing its norm weights");
        for (auto* l : L.all) FT_CHECK_ARG(l->w, "linear %s has no weight", l->prefix.c_str());
    }
    if (m->params_dirty) {
        FT_TRY(rebuild_params(m));
        ws_free(m);
    }
    FT_TRY(ensure_workspace(m, B, S));
    const size_t T = B * S;
    uint32_t* ids = m->io_host;
    uint32_t* idx = ids + T;
    uint32_t* inv = ids + 2 * T;
    uint32_t* tgs = ids + 3 * T;
    float* wts = reinterpret_cast<float*>(ids + 4 * T);
    std::memcpy(ids, rows_host, T * sizeof(uint32_t));
    m->head_rows = T;
    m->head_compact = head != nullptr && head->size() < T && !c.head_all_rows;
    if (m->head_compact) {
        m->head_rows = head->size();
        for (size_t r = 0; r < T; r++) inv[r] = (uint32_t)head->size();
        for (size_t k = 0; k < head->size(); k++) {
            FT_CHECK_ARG((*head)[k] < T && (k == 0 || (*head)[k] > (*head)[k - 1]), "head rows must ascend within the chunk");
            idx[k] = (*head)[k];
            inv[(*head)[k]] = (uint32_t)k;
            tgs[k] = (*tg)[k];
            wts[k] = (*wt)[k];
        }
    } else {
        for (size_t r = 0; r < T; r++) {
            tgs[r] = FT_MASKED_CE_SKIP;
            wts[r] = 0.0f;
        }
        if (head)
            for (size_t k = 0; k < head->size(); k++) {
                FT_CHECK_ARG((*head)[k] < T, "head rows must lie within the chunk");
                tgs[(*head)[k]] = (*tg)[k];
                wts[(*head)[k]] = (*wt)[k];
            }
    }
    FT_HIP(hipMemcpyAsync(m->io_dev, m->io_host, 5 * T * sizeof(uint32_t), hipMemcpyHostToDevice, ctx->stream));
    return FT_OK;
}

// Forward over the staged chunk: embedding, blocks, and the head on m->head_rows rows.
int model_forward(ft_model* m, size_t B, size_t S) {
    ft_context* ctx = m->ctx;
    const ft_model_config& c = m->cfg;
    const size_t T = B * S, H = c.hidden_size;
    FT_TRY(ft_embedding(ctx, m->embed, c.vocab_size, H, m->ids_dev, T, m->acts.empty() ? m->x_final : m->acts[0].x));
    m->pending_x = ft_deferred_sum{};
    for (size_t l = 0; l < m->layers.size(); l++) FT_TRY(layer_forward(m, l, B, S, true));
    const float* xf = m->x_final;
    if (m->head_compact) {
        // gather: row k of xc = row head[k] of x_final
        FT_TRY(ft_embedding(ctx, m->x_final, T, H, m->head_idx_dev, m->head_rows, m->xc));
        xf = m->xc;
    }
    if (m->head_rows == 0) return FT_OK;
    FT_TRY(ft_rms_norm_eps(ctx, xf, m->norm_f, m->hf, m->head_rows, H, c.rms_norm_eps));
    FT_TRY(linear_forward(ctx, m->lm_head, m->hf, m->thead, m->logits, m->head_rows));
    return FT_OK;
}

// Brings the row losses and the control block to the host (one copy, then the stream is idle).
int fetch_step_out(ft_model* m) {
    const size_t T = m->ws_B * m->ws_S;
    FT_HIP(hipMemcpyAsync(m->out_host, m->step_out, (T + 4) * sizeof(float), hipMemcpyDeviceToHost, m->ctx->stream));
    FT_HIP(hipStreamSynchronize(m->ctx->stream));
    return FT_OK;
}

// gx = rms_norm_backward(x, w, g) (+ add). With a trainable norm scale (`gw`) its gradient is
// computed too (RMSNormNode::backward, autograd/src/lib.rs:575-595), added to the earlier
// micro-batches' when `accumulate`; `tmp` [rows, H] is scratch for that unfused form and must not
// alias x, g or add.
// `g_sum` (optional, only without `gw`): g arrives as the K shares of the GEMM that produced it.
int norm_backward(ft_model* m, const float* x, const float* w, float* gw, const float* g, const float* add,
                  float* gx, float* tmp, size_t rows, bool accumulate, const ft_deferred_sum* g_sum = nullptr) {
    ft_context* ctx = m->ctx;
    const size_t H = m->cfg.hidden_size;
    const float eps = m->cfg.rms_norm_eps;
    if (g_sum && g_sum->pending()) {
        FT_CHECK_ARG(!gw, "norm_backward: a deferred gradient with a trainable norm scale");
        return ft_internal_rms_norm_backward_sum(ctx, x, w, g_sum, add, gx, rows, H, eps);
    }
    if (!gw) {
        if (add) return ft_internal_rms_norm_backward_add(ctx, x, w, g, add, gx, rows, H, eps);
        return ft_rms_norm_backward(ctx, x, w, g, gx, nullptr, rows, H, eps);
    }
    float* out = add ? tmp : gx;
    FT_TRY(ft_rms_norm_backward(ctx, x, w, g, out, accumulate ? m->gtmp : gw, rows, H, eps));
    if (accumulate) FT_TRY(ft_gradient_accumulate(ctx, gw, m->gtmp, H));
    if (add) FT_TRY(ft_add(ctx, add, tmp, gx, rows * H));
    return FT_OK;
}

// Backward from d_logits (in m->logits) to the gradient of every trainable tensor.
int model_backward(ft_model* m, size_t B, size_t S, bool accumulate) {
    ft_context* ctx = m->ctx;
    const ft_model_config& c = m->cfg;
    const size_t T = B * S, H = c.hidden_size, F = c.intermediate_size;
    const size_t D = m->head_dim(), nh = c.num_attention_heads, nkv = c.num_key_value_heads;
    ft_attention_options opts{};
    opts.causal = 1;
    // lm_head and final norm, on the rows the head ran on
    float* g = m->g0;
    float* g_other = m->g1;
    const size_t Th = m->head_rows;
    FT_TRY(linear_backward(m, m->lm_head, m->hf, m->thead, m->logits, m->d_h2, Th, accumulate));
    if (m->head_compact) {
        FT_TRY(norm_backward(m, m->xc, m->norm_f, m->gnorm_f, m->d_h2, nullptr, g_other, nullptr, Th, accumulate));
        // scatter: row r of g = row head_inv[r] of the compact gradient, zero where the head did not run
        FT_TRY(ft_embedding(ctx, g_other, Th, H, m->head_inv_dev, T, g));
    } else {
        FT_TRY(norm_backward(m, m->x_final, m->norm_f, m->gnorm_f, m->d_h2, nullptr, g, nullptr, T, accumulate));
    }
    const bool can_sum = ft_internal_norm_can_sum(T, H);
    for (size_t li = m->layers.size(); li-- > 0;) {
        Layer& L = m->layers[li];
        LayerActs& a = m->acts[li];
        ft_deferred_sum dsum;  // an input gradient left as K shares for the norm backward that follows it
        // The factor gradients of a block read its activations, output gradients and dT buffers; they
        // are launched (flush_cols) at the block's end, before g, the buffers of the next block's
        // gradients and, with checkpointing, the shared block buffers are rewritten.
        if (c.checkpoint_blocks && li + 1 < m->layers.size()) {
            // Recompute this block's forward. (The last block's internals are still there from the
            // forward pass.)
            FT_TRY(layer_forward(m, li, B, S));
        }
        // x_next = h + down(silu(gate) * up)
        if (!L.down.has_lora() && !L.down.gw && !L.down.gbias) {
            FT_TRY(ft_mlp_down_backward(ctx, g, L.down.w, L.down.dtype, a.gate, a.up, m->d_gate, m->d_up, m->d_act, T,
                                        F, H));
        } else {
            FT_TRY(linear_backward(m, L.down, a.act, a.tdown, g, m->d_act, T, accumulate));
            FT_TRY(ft_silu_gate_backward(ctx, a.gate, a.up, m->d_act, m->d_gate, m->d_up, T * F));
        }
        {
            LinearW* ls[2] = {&L.up, &L.gate};
            const float* ts[2] = {a.tup, a.tgate};
            const float* dys[2] = {m->d_up, m->d_gate};
            dsum = ft_deferred_sum{};
            FT_TRY(linear_backward_group(m, ls, ts, dys, m->d_h2, 2, a.h2, T, accumulate, false,
                                         can_sum && !L.gnorm2 ? &dsum : nullptr));
        }
        // g_h = g + norm2_backward(d_h2) (into g_other)
        FT_TRY(norm_backward(m, a.h, L.norm2, L.gnorm2, m->d_h2, g, g_other, m->d_h1, T, accumulate, &dsum));
        // h = x + o_proj(attn)
        FT_TRY(linear_backward(m, L.o, a.attn, a.to, g_other, m->d_attn, T, accumulate));
        if (m->rope_table &&
            ft_internal_attention_rope_fusable(a.q, a.k, a.v, a.attn, m->d_attn, S, S, D)) {
            // dq and dk come out of the attention kernels already rotated back through RoPE
            FT_TRY(ft_internal_attention_backward_rope(ctx, a.q, a.k, a.v, a.attn, m->d_attn, m->dq, m->dk, m->dv,
                                                       a.stats, B, S, nh, nkv, &opts, m->rope_table));
        } else {
            FT_TRY(ft_flash_attention_v2_backward_with_stats(ctx, a.q, a.k, a.v, a.attn, m->d_attn, m->dq, m->dk,
                                                             m->dv, a.stats, B, S, S, nh, nkv, D, &opts));
            if (m->rope_table) {
                FT_TRY(ft_internal_rope_pair(ctx, m->dq, m->dq, nh, m->dk, m->dk, nkv, m->rope_table, B, S, D, 1));
            } else {
                FT_TRY(ft_rope_theta_inverse(ctx, m->dq, B, S, nh * D, D, 0, c.rope_theta));
                FT_TRY(ft_rope_theta_inverse(ctx, m->dk, B, S, nkv * D, D, 0, c.rope_theta));
            }
        }
        // The first block's input is the frozen embedding: its norm output needs
        // no gradient, so the three input-gradient GEMMs are skipped
        // (MatMulNode::backward, autograd/src/lib.rs:268-287).
        // A trainable input norm still needs its output's gradient for its own scale.
        const bool need_dx = li > 0 || L.gnorm1 != nullptr;
        {
            LinearW* ls[3] = {&L.q, &L.k, &L.v};
            const float* ts[3] = {a.tq, a.tk, a.tv};
            const float* dys[3] = {m->dq, m->dk, m->dv};
            // d_h1 = dx_q + dx_k + dx_v
            // the block's last adapters: everything that waited is launched now
            dsum = ft_deferred_sum{};
            FT_TRY(linear_backward_group(m, ls, ts, dys, need_dx ? m->d_h1 : nullptr, 3, a.h1, T, accumulate, true,
                                         can_sum && !L.gnorm1 ? &dsum : nullptr));
        }
        if (!need_dx) break;
        // g = g_h + norm1_backward(d_h1)
        FT_TRY(norm_backward(m, a.x, L.norm1, L.gnorm1, m->d_h1, g_other, g, m->d_h2, T, accumulate, &dsum));
    }
    return flush_cols(m);
}

LinearW* find_linear(ft_model* m, const std::string& prefix) {
    if (prefix == "lm_head") return &m->lm_head;
    for (auto& L : m->layers)
        for (auto* l : L.all)
            if (l->prefix == prefix) return l;
    return nullptr;
}

int set_linear_weight(ft_model* m, LinearW& l, const float* hf_out_in, size_t out, size_t in) {
    FT_CHECK_ARG(out == l.out && in == l.in, "%s.weight is [%zu, %zu], expected [%zu, %zu]", l.prefix.c_str(), out, in,
                 l.out, l.in);
    // upload_linear (model_builder.rs:325-340): f32 when the base trains, else f16 when asked
    const int dtype = (m->cfg.f16_linears && !m->cfg.trainable_base) ? FT_DTYPE_F16 : FT_DTYPE_F32;
    if (!l.w) {
        m->params_dirty = true;   // a new weight may be a new trainable tensor
        m->param_generation++;
        size_t bytes = in * out * (dtype == FT_DTYPE_F16 ? 2 : 4);
        bytes = (bytes + 3) / 4 * 4;
        FT_TRY(ft_alloc(m->ctx, bytes, &l.w));
    }
    l.dtype = dtype;
    // builder rule: HF [out, in] -> [in, out] (model_builder.rs:415-424)
    return ft_upload_f32_transposed(m->ctx, l.w, hf_out_in, out, in, dtype);
}

int set_vector(ft_model* m, float** slot, const float* data, size_t n, size_t want, const char* name) {
    FT_CHECK_ARG(n == want, "%s has %zu values, expected %zu", name, n, want);
    if (!*slot) {
        FT_TRY(alloc_f(m->ctx, n, slot));
        m->params_dirty = true;   // with a trainable base a new norm scale is a new trainable tensor
        m->param_generation++;
    }
    return ft_upload(m->ctx, *slot, data, n * sizeof(float));
}

template <typename Fn>
int guarded(Fn&& fn) {
    try {
        return fn();
    } catch (const std::exception& e) {
        return ft_set_error(FT_ERR_INVALID, "exception: %s", e.what());
    } catch (...) {
        return ft_set_error(FT_ERR_INVALID, "unknown exception");
    }
}

}  // namespace

extern "C" {

int ft_model_create(ft_context* ctx, const ft_model_config* cfg, ft_model** out) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(ctx && cfg && out, "ft_model_create: NULL argument");
        FT_CHECK_ARG(cfg->num_attention_heads > 0 && cfg->hidden_size % cfg->num_attention_heads == 0,
                     "ft_model_create: hidden_size %u is not a multiple of %u heads", cfg->hidden_size,
                     cfg->num_attention_heads);
        FT_CHECK_ARG(cfg->num_key_value_heads > 0 && cfg->num_attention_heads % cfg->num_key_value_heads == 0,
                     "ft_model_create: %u heads is not a multiple of %u kv heads", cfg->num_attention_heads,
                     cfg->num_key_value_heads);
        const size_t D = cfg->hidden_size / cfg->num_attention_heads;
        FT_CHECK_ARG(D <= 128 && D % 2 == 0, "ft_model_create: head_dim %zu must be even and <= 128", D);
        auto m = std::make_unique<ft_model>();
        m->ctx = ctx;
        m->cfg = *cfg;
        const size_t H = cfg->hidden_size, F = cfg->intermediate_size;
        const size_t QD = cfg->num_attention_heads * D, KD = cfg->num_key_value_heads * D;
        m->layers.resize(cfg->num_hidden_layers);
        for (size_t l = 0; l < m->layers.size(); l++) {
            Layer& L = m->layers[l];
            const std::string p = "model.layers." + std::to_string(l);
            auto init = [&](LinearW& w, const char* name, size_t in, size_t o) {
                w.prefix = p + name;
                w.in = in;
                w.out = o;
            };
            init(L.q, ".self_attn.q_proj", H, QD);
            init(L.k, ".self_attn.k_proj", H, KD);
            init(L.v, ".self_attn.v_proj", H, KD);
            init(L.o, ".self_attn.o_proj", QD, H);
            init(L.gate, ".mlp.gate_proj", H, F);
            init(L.up, ".mlp.up_proj", H, F);
            init(L.down, ".mlp.down_proj", F, H);
        }
        m->lm_head.prefix = "lm_head";
        m->lm_head.in = H;
        m->lm_head.out = cfg->vocab_size;
        *out = m.release();
        return FT_OK;
    });
}

int ft_model_destroy(ft_model* m) {
    if (!m) return FT_OK;
    ws_free(m);
    ft_context* ctx = m->ctx;
    auto rel = [&](void* p) {
        if (p) (void)ft_free(ctx, p);
    };
    auto rel_lin = [&](LinearW& l) {
        rel(l.w);
        rel(l.a);
        rel(l.b);
        rel(l.ga);
        rel(l.gb);
        rel(l.gw);
        rel(l.bias);
        rel(l.gbias);
    };
    rel(m->embed);
    rel(m->norm_f);
    rel(m->gnorm_f);
    for (auto& L : m->layers) {
        rel(L.norm1);
        rel(L.norm2);
        rel(L.gnorm1);
        rel(L.gnorm2);
        for (auto* l : L.all) rel_lin(*l);
    }
    rel_lin(m->lm_head);
    delete m;
    return FT_OK;
}

int ft_model_set_tensor(ft_model* m, const char* hf_name, const float* data, const size_t* shape, int ndim) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && hf_name && data && shape, "ft_model_set_tensor: NULL argument");
        const std::string name(hf_name);
        const ft_model_config& c = m->cfg;
        const size_t H = c.hidden_size, V = c.vocab_size;
        size_t n = 1;
        for (int i = 0; i < ndim; i++) n *= shape[i];
        if (name == "model.embed_tokens.weight") {
            FT_CHECK_ARG(ndim == 2 && shape[0] == V && shape[1] == H, "embed_tokens must be [%zu, %zu]", V, H);
            FT_TRY(set_vector(m, &m->embed, data, n, V * H, hf_name));
            // Tied head = embedding transposed (model_builder.rs:653-689).
            if (c.tie_word_embeddings) FT_TRY(set_linear_weight(m, m->lm_head, data, V, H));
            return FT_OK;
        }
        if (name == "model.norm.weight") return set_vector(m, &m->norm_f, data, n, H, hf_name);
        if (name == "lm_head.weight") {
            FT_CHECK_ARG(ndim == 2, "lm_head.weight must be 2-D");
            if (c.tie_word_embeddings) return FT_OK;  // the tied head ignores a separate tensor
            return set_linear_weight(m, m->lm_head, data, shape[0], shape[1]);
        }
        // build_linear (model_builder.rs:454-469): `<prefix>.bias` must be [out]
        auto set_bias = [&](LinearW& l) -> int {
            FT_CHECK_ARG(ndim == 1 && shape[0] == l.out, "%s must be [%zu]", hf_name, l.out);
            return set_vector(m, &l.bias, data, n, l.out, hf_name);
        };
        if (name == "lm_head.bias") {
            if (c.tie_word_embeddings) return FT_OK;  // the tied head is the embedding alone
            return set_bias(m->lm_head);
        }
        const std::string pre = "model.layers.";
        FT_CHECK_ARG(name.compare(0, pre.size(), pre) == 0, "unknown tensor %s", hf_name);
        const size_t dot = name.find('.', pre.size());
        FT_CHECK_ARG(dot != std::string::npos, "unknown tensor %s", hf_name);
        const size_t li = (size_t)std::stoul(name.substr(pre.size(), dot - pre.size()));
        FT_CHECK_ARG(li < m->layers.size(), "%s: layer %zu of %zu", hf_name, li, m->layers.size());
        Layer& L = m->layers[li];
        const std::string rest = name.substr(dot);
        if (rest == ".input_layernorm.weight") return set_vector(m, &L.norm1, data, n, H, hf_name);
        if (rest == ".post_attention_layernorm.weight") return set_vector(m, &L.norm2, data, n, H, hf_name);
        const std::string bias_suffix = ".bias";
        if (rest.size() > bias_suffix.size() &&
            rest.compare(rest.size() - bias_suffix.size(), bias_suffix.size(), bias_suffix) == 0) {
            LinearW* l = find_linear(m, name.substr(0, name.size() - bias_suffix.size()));
            FT_CHECK_ARG(l, "unknown tensor %s", hf_name);
            return set_bias(*l);
        }
        const std::string suffix = ".weight";
        FT_CHECK_ARG(rest.size() > suffix.size() && rest.compare(rest.size() - suffix.size(), suffix.size(), suffix) == 0,
                     "unknown tensor %s", hf_name);
        LinearW* l = find_linear(m, name.substr(0, name.size() - suffix.size()));
        FT_CHECK_ARG(l, "unknown tensor %s", hf_name);
        FT_CHECK_ARG(ndim == 2, "%s must be 2-D", hf_name);
        return set_linear_weight(m, *l, data, shape[0], shape[1]);
    });
}

int ft_model_set_lora(ft_model* m, const char* prefix, const float* a, const float* b, size_t rank, float alpha) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && prefix && a && b, "ft_model_set_lora: NULL argument");
        FT_CHECK_ARG(rank >= 1 && rank <= 32, "ft_model_set_lora: rank %zu is outside 1..32", rank);
        LinearW* l = find_linear(m, prefix);
        FT_CHECK_ARG(l, "ft_model_set_lora: no linear named %s", prefix);
        if (l->r != rank) {
            for (float** p : {&l->a, &l->b, &l->ga, &l->gb}) {
                if (*p) FT_TRY(ft_free(m->ctx, *p));
                *p = nullptr;
            }
            FT_TRY(alloc_f(m->ctx, l->in * rank, &l->a));
            FT_TRY(alloc_f(m->ctx, rank * l->out, &l->b));
            FT_TRY(alloc_f(m->ctx, l->in * rank, &l->ga));
            FT_TRY(alloc_f(m->ctx, rank * l->out, &l->gb));
            FT_TRY(ft_zero(m->ctx, l->ga, l->in * rank * 4));
            FT_TRY(ft_zero(m->ctx, l->gb, rank * l->out * 4));
            l->r = rank;
            m->params_dirty = true;
            m->param_generation++;
        }
        l->alpha = alpha;
        FT_TRY(ft_upload(m->ctx, l->a, a, l->in * rank * sizeof(float)));
        FT_TRY(ft_upload(m->ctx, l->b, b, rank * l->out * sizeof(float)));
        return FT_OK;
    });
}

uint64_t ft_lora_seed(uint64_t layer_seed, const char* module_name) {
    // FNV-1a over the name bytes, then the seed's little-endian bytes, then the splitmix64 finalizer.
    uint64_t h = 0xcbf29ce484222325ull;
    auto mix = [&](uint8_t byte) {
        h ^= (uint64_t)byte;
        h *= 0x00000100000001b3ull;
    };
    for (const char* c = module_name ? module_name : ""; *c; c++) mix((uint8_t)*c);
    for (int i = 0; i < 8; i++) mix((uint8_t)(layer_seed >> (8 * i)));
    h ^= h >> 30;
    h *= 0xbf58476d1ce4e5b9ull;
    h ^= h >> 27;
    h *= 0x94d049bb133111ebull;
    return h ^ (h >> 31);
}

int ft_lora_init_a(float* a_host, size_t in_dim, size_t out_dim, size_t rank, uint64_t seed) {
    FT_CHECK_ARG(a_host || in_dim * rank == 0, "ft_lora_init_a: NULL argument");
    const float bound = 1.0f / std::sqrt((float)(in_dim > 0 ? in_dim : 1));
    uint64_t state =
        (seed * 0x9E3779B97F4A7C15ull + (((uint64_t)in_dim << 32) | ((uint64_t)out_dim << 8) | (uint64_t)rank)) | 1ull;
    for (size_t i = 0; i < in_dim * rank; i++) {
        // xorshift64*
        state ^= state >> 12;
        state ^= state << 25;
        state ^= state >> 27;
        const uint64_t bits = (state * 0x2545F4914F6CDD1Dull) >> 40;
        const float unit = (float)bits / (float)(1ull << 24);
        a_host[i] = (unit * 2.0f - 1.0f) * bound;
    }
    return FT_OK;
}

int ft_model_add_lora(ft_model* m, const char* prefix, size_t rank, float alpha) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && prefix, "ft_model_add_lora: NULL argument");
        LinearW* l = find_linear(m, prefix);
        FT_CHECK_ARG(l, "ft_model_add_lora: no linear named %s", prefix);
        // layer seed = layer index + 1, 0 for lm_head; module name = last component of the prefix
        const std::string pre(prefix);
        uint64_t layer_seed = 0;
        const size_t at = pre.find("layers.");
        if (at != std::string::npos) layer_seed = (uint64_t)std::strtoull(pre.c_str() + at + 7, nullptr, 10) + 1;
        const size_t dot = pre.rfind('.');
        const std::string module = dot == std::string::npos ? pre : pre.substr(dot + 1);
        std::vector<float> a(l->in * rank), b(rank * l->out, 0.0f);
        FT_TRY(ft_lora_init_a(a.data(), l->in, l->out, rank, ft_lora_seed(layer_seed, module.c_str())));
        return ft_model_set_lora(m, prefix, a.data(), b.data(), rank, alpha);
    });
}

int ft_model_set_head_all_rows(ft_model* m, int all_rows) {
    FT_CHECK_ARG(m, "ft_model_set_head_all_rows: NULL argument");
    m->cfg.head_all_rows = all_rows ? 1 : 0;
    return FT_OK;
}

int ft_model_param_count(ft_model* m, size_t* count) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && count, "ft_model_param_count: NULL argument");
        if (m->params_dirty) {
            FT_TRY(rebuild_params(m));
            ws_free(m);
        }
        *count = m->params.size();
        return FT_OK;
    });
}

int ft_model_param_info(ft_model* m, size_t index, const char** name, size_t* numel) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m, "ft_model_param_info: NULL argument");
        if (m->params_dirty) {
            FT_TRY(rebuild_params(m));
            ws_free(m);
        }
        FT_CHECK_ARG(index < m->params.size(), "ft_model_param_info: index %zu of %zu", index, m->params.size());
        if (name) *name = m->params[index].name.c_str();
        if (numel) *numel = m->params[index].n;
        return FT_OK;
    });
}

int ft_model_read_param(ft_model* m, size_t index, float* out_host) {
    FT_CHECK_ARG(m && out_host && !m->params_dirty && index < m->params.size(), "ft_model_read_param: bad argument");
    return ft_download(m->ctx, out_host, m->params[index].w, m->params[index].n * sizeof(float));
}

int ft_model_write_param(ft_model* m, size_t index, const float* host) {
    FT_CHECK_ARG(m && host && !m->params_dirty && index < m->params.size(), "ft_model_write_param: bad argument");
    // The buffer keeps its address: optimizer moments and trainers built for it stay valid.
    return ft_upload(m->ctx, m->params[index].w, host, m->params[index].n * sizeof(float));
}

int ft_model_read_grad(ft_model* m, size_t index, float* out_host) {
    FT_CHECK_ARG(m && out_host && !m->params_dirty && index < m->params.size(), "ft_model_read_grad: bad argument");
    return ft_download(m->ctx, out_host, m->params[index].g, m->params[index].n * sizeof(float));
}

int ft_model_forward_logits(ft_model* m, const uint32_t* rows, size_t B, size_t S, float* logits_host) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && rows && logits_host && B > 0 && S > 0, "ft_model_forward_logits: bad argument");
        FT_TRY(stage_chunk(m, rows, B, S, nullptr, nullptr, nullptr));
        FT_TRY(model_forward(m, B, S));
        return ft_download(m->ctx, logits_host, m->logits, B * S * m->cfg.vocab_size * sizeof(float));
    });
}

int ft_trainer_create(ft_model* m, const ft_trainer_config* cfg, ft_trainer** out) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && cfg && out, "ft_trainer_create: NULL argument");
        if (m->params_dirty) {
            FT_TRY(rebuild_params(m));
            ws_free(m);
        }
        FT_CHECK_ARG(!m->params.empty(), "ft_trainer_create: the model has no LoRA adapter to train");
        auto t = std::make_unique<ft_trainer>();
        t->model = m;
        t->cfg = *cfg;
        t->generation = m->param_generation;
        ft_context* ctx = m->ctx;
        std::vector<ft_segment> segs;
        for (auto& p : m->params) {
            t->numel.push_back(p.n);
            float *pm = nullptr, *pv = nullptr;
            FT_TRY(alloc_f(ctx, p.n, &pm));
            FT_TRY(alloc_f(ctx, p.n, &pv));
            FT_TRY(ft_zero(ctx, pm, p.n * 4));   // moments start at zero (AdamW::apply_step)
            FT_TRY(ft_zero(ctx, pv, p.n * 4));
            t->m.push_back(pm);
            t->v.push_back(pv);
            for (size_t off = 0; off < p.n; off += FT_SUM_SQUARES_CHUNK) {
                const size_t n = p.n - off < FT_SUM_SQUARES_CHUNK ? p.n - off : FT_SUM_SQUARES_CHUNK;
                segs.push_back(ft_segment{p.w + off, p.g + off, pm + off, pv + off, (uint32_t)n});
            }
        }
        t->nseg = segs.size();
        FT_TRY(ft_alloc(ctx, segs.size() * sizeof(ft_segment), (void**)&t->segs_dev));
        FT_TRY(ft_upload(ctx, t->segs_dev, segs.data(), segs.size() * sizeof(ft_segment)));
        FT_TRY(alloc_f(ctx, segs.size(), &t->partials));
        *out = t.release();
        return FT_OK;
    });
}

int ft_trainer_destroy(ft_trainer* t) {
    if (!t) return FT_OK;
    ft_context* ctx = t->model->ctx;
    for (float* p : t->m) (void)ft_free(ctx, p);
    for (float* p : t->v) (void)ft_free(ctx, p);
    if (t->segs_dev) (void)ft_free(ctx, t->segs_dev);
    if (t->partials) (void)ft_free(ctx, t->partials);
    delete t;
    return FT_OK;
}

}  // extern "C"

namespace {

// Host half of masked_cross_entropy_batch (trainer/src/lib.rs:689-722): per-row target or
// MASKED_CE_SKIP, weight 1 / supervised tokens of the row's sequence; kept for the supervised rows
// only (`head`, ascending), in that order. Returns the total.
size_t build_targets(const uint32_t* targets, const uint8_t* loss_mask, size_t B, size_t S, size_t V,
                     std::vector<uint32_t>& tg, std::vector<float>& wt, std::vector<size_t>& tokens,
                     std::vector<uint32_t>& head) {
    const size_t T = B * S;
    tg.clear();
    wt.clear();
    head.clear();
    tokens.assign(B, 0);
    auto supervised = [&](size_t r) { return loss_mask[r] != 0 && (size_t)targets[r] < V; };
    size_t total = 0;
    for (size_t s = 0; s < B; s++) {
        for (size_t i = 0; i < S; i++) tokens[s] += supervised(s * S + i) ? 1 : 0;
        total += tokens[s];
    }
    for (size_t r = 0; r < T; r++) {
        if (supervised(r)) {
            head.push_back((uint32_t)r);
            tg.push_back(targets[r]);
            wt.push_back(1.0f / (float)tokens[r / S]);
        }
    }
    return total;
}

// Per-sequence mean losses from the device row losses of the head rows (f64 sums in row order, as the
// reference's host code; the rows left out are the ones that would add 0).
int read_sequence_losses(ft_model* m, size_t B, size_t S, const std::vector<size_t>& tokens,
                         const std::vector<uint32_t>& head, float* per_sequence, float* total_out) {
    const float* losses = m->out_host;   // filled by fetch_step_out
    std::vector<double> sums(B, 0.0);
    for (size_t k = 0; k < head.size(); k++) sums[head[k] / S] += (double)losses[m->head_compact ? k : head[k]];
    float total = 0.0f;
    for (size_t s = 0; s < B; s++) {
        const float mean = (float)(sums[s] / (double)(tokens[s] ? tokens[s] : 1));
        if (per_sequence) per_sequence[s] = mean;
        total += mean;
    }
    if (total_out) *total_out = total;
    return FT_OK;
}

}  // namespace

extern "C" {

int ft_model_eval_chunk(ft_model* m, const uint32_t* rows, const uint32_t* targets, const uint8_t* loss_mask,
                        size_t B, size_t S, float* per_sequence_loss, uint32_t* per_sequence_tokens) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(m && rows && targets && loss_mask && per_sequence_loss && per_sequence_tokens,
                     "ft_model_eval_chunk: NULL argument");
        FT_CHECK_ARG(B > 0 && S > 0, "ft_model_eval_chunk: empty chunk");
        const size_t V = m->cfg.vocab_size;
        std::vector<uint32_t> tg;
        std::vector<float> wt;
        std::vector<size_t> tokens;
        std::vector<uint32_t> head;
        const size_t total = build_targets(targets, loss_mask, B, S, V, tg, wt, tokens, head);
        for (size_t s = 0; s < B; s++) {
            per_sequence_tokens[s] = (uint32_t)tokens[s];
            per_sequence_loss[s] = 0.0f;
        }
        if (total == 0) return FT_OK;
        FT_TRY(stage_chunk(m, rows, B, S, &head, &tg, &wt));
        FT_TRY(model_forward(m, B, S));
        // forward only: the gradient the kernel writes (in place of the logits) is discarded
        FT_TRY(ft_masked_cross_entropy_weighted(m->ctx, m->logits, m->targets_dev, m->weights_dev, m->logits,
                                                m->row_loss, m->head_rows, V, 1.0f));
        FT_TRY(fetch_step_out(m));
        return read_sequence_losses(m, B, S, tokens, head, per_sequence_loss, nullptr);
    });
}

float ft_lr_schedule(uint32_t kind, float peak_lr, float min_lr, uint32_t warmup_steps, uint32_t total_steps,
                     uint32_t step) {
    const float pi = 3.14159265358979323846f;
    if (kind == FT_LR_COSINE) {
        if (step >= total_steps) return min_lr;
        const float progress = (float)step / (float)total_steps;
        const float cosine = (1.0f + cosf(pi * progress)) / 2.0f;
        return min_lr + (peak_lr - min_lr) * cosine;
    }
    if (kind == FT_LR_WARMUP_COSINE) {
        if (step < warmup_steps) return peak_lr * ((float)step / (float)warmup_steps);
        if (step >= total_steps) return min_lr;
        const float progress = (float)(step - warmup_steps) / (float)(total_steps - warmup_steps);
        const float cosine = (1.0f + cosf(pi * progress)) / 2.0f;
        return min_lr + (peak_lr - min_lr) * cosine;
    }
    return peak_lr;
}

int ft_trainer_optimizer_steps(ft_trainer* t, size_t* steps) {
    FT_CHECK_ARG(t && steps, "ft_trainer_optimizer_steps: NULL argument");
    *steps = t->optimizer_steps;
    return FT_OK;
}

// A trainer built before an adapter was added or changed rank points into buffers the model has
// freed since: refuse to use it.
#define FT_CHECK_TRAINER_CURRENT(t, what)                                                                     \
    FT_CHECK_ARG((t)->generation == (t)->model->param_generation,                                            \
                 what ": the model's adapters changed (a rank, or a new adapter) after this trainer was "     \
                      "created; create a new trainer")

int ft_trainer_read_moments(ft_trainer* t, size_t index, float* m_host, float* v_host) {
    FT_CHECK_ARG(t && m_host && v_host, "ft_trainer_read_moments: NULL argument");
    FT_CHECK_TRAINER_CURRENT(t, "ft_trainer_read_moments");
    FT_CHECK_ARG(index < t->m.size(), "ft_trainer_read_moments: index %zu of %zu", index, t->m.size());
    const size_t bytes = t->numel[index] * sizeof(float);
    FT_TRY(ft_download(t->model->ctx, m_host, t->m[index], bytes));
    return ft_download(t->model->ctx, v_host, t->v[index], bytes);
}

int ft_trainer_write_moments(ft_trainer* t, size_t index, const float* m_host, const float* v_host) {
    FT_CHECK_ARG(t && m_host && v_host, "ft_trainer_write_moments: NULL argument");
    FT_CHECK_TRAINER_CURRENT(t, "ft_trainer_write_moments");
    FT_CHECK_ARG(index < t->m.size(), "ft_trainer_write_moments: index %zu of %zu", index, t->m.size());
    const size_t bytes = t->numel[index] * sizeof(float);
    FT_TRY(ft_upload(t->model->ctx, t->m[index], m_host, bytes));
    return ft_upload(t->model->ctx, t->v[index], v_host, bytes);
}

int ft_trainer_get_adam_t(ft_trainer* t, float* steps) {
    FT_CHECK_ARG(t && steps, "ft_trainer_get_adam_t: NULL argument");
    *steps = t->t;
    return FT_OK;
}

int ft_trainer_set_adam_t(ft_trainer* t, float steps) {
    FT_CHECK_ARG(t && steps >= 0.0f, "ft_trainer_set_adam_t: bad argument");
    t->t = steps;
    return FT_OK;
}

int ft_trainer_set_adam_hyper(ft_trainer* t, float lr, float beta1, float beta2, float eps, float weight_decay) {
    FT_CHECK_ARG(t, "ft_trainer_set_adam_hyper: NULL argument");
    FT_CHECK_ARG(std::isfinite(lr) && beta1 >= 0.0f && beta1 < 1.0f && beta2 >= 0.0f && beta2 < 1.0f && eps >= 0.0f &&
                     std::isfinite(weight_decay),
                 "ft_trainer_set_adam_hyper: lr %g, betas (%g, %g), eps %g, weight decay %g", lr, beta1, beta2, eps,
                 weight_decay);
    // With a schedule the optimizer's rate is overwritten before every step (LRScheduler::step), so a
    // restored rate only lasts where there is none.
    if (t->cfg.lr_schedule == FT_LR_CONSTANT) t->cfg.lr = lr;
    t->cfg.beta1 = beta1;
    t->cfg.beta2 = beta2;
    t->cfg.eps = eps;
    t->cfg.weight_decay = weight_decay;
    return FT_OK;
}

// ---- Trainer::train_batch / train_chunk, the host half (integer work, no device) ----

int ft_train_batch_select(const uint32_t* input_ids, const uint32_t* target_ids, const uint8_t* attention_mask,
                          const uint8_t* loss_mask, size_t batch, size_t padded_len, size_t* valid_len,
                          size_t* kept) {
    FT_CHECK_ARG(valid_len && kept && (batch == 0 || padded_len == 0 || (input_ids && target_ids && attention_mask && loss_mask)),
                 "ft_train_batch_select: NULL argument");
    (void)input_ids;
    (void)target_ids;
    size_t n = 0;
    for (size_t b = 0; b < batch; b++) {
        const uint8_t* attn = attention_mask + b * padded_len;
        const uint8_t* mask = loss_mask + b * padded_len;
        size_t len = 0;
        while (len < padded_len && attn[len] == 1) len++;  // take_while(flag == 1)
        bool supervised = false;
        for (size_t i = 0; i < len && !supervised; i++) supervised = mask[i] != 0;
        // fewer than two tokens, or no supervised position: the sequence does not train
        if (len < 2 || !supervised) len = 0;
        valid_len[b] = len;
        if (len) n++;
    }
    *kept = n;
    return FT_OK;
}

int ft_train_batch_plan(size_t sequences, size_t grad_accum_steps, size_t step_in_accum, size_t* chunk_sizes,
                        size_t* chunks) {
    FT_CHECK_ARG(chunks && (sequences == 0 || chunk_sizes), "ft_train_batch_plan: NULL argument");
    size_t n = 0, rest = sequences;
    while (rest > 0) {
        size_t room = rest;  // grad_accum_steps 0: the whole batch is one window (ft_trainer_config)
        if (grad_accum_steps) {
            room = grad_accum_steps > step_in_accum ? grad_accum_steps - step_in_accum : 0;  // saturating_sub
            if (room < 1) room = 1;
            if (room > rest) room = rest;
            step_in_accum += room;
            if (step_in_accum >= grad_accum_steps) step_in_accum = 0;  // the chunk that fills the window steps
        }
        chunk_sizes[n++] = room;
        rest -= room;
    }
    *chunks = n;
    return FT_OK;
}

int ft_chunk_padded_len(const size_t* input_lens, const size_t* target_lens, size_t count, size_t length_bucket,
                        size_t* padded_len) {
    FT_CHECK_ARG(padded_len && (count == 0 || (input_lens && target_lens)), "ft_chunk_padded_len: NULL argument");
    FT_CHECK_ARG(length_bucket >= 1, "ft_chunk_padded_len: length_bucket must be at least 1");
    size_t longest = 0;
    for (size_t i = 0; i < count; i++) {
        const size_t len = input_lens[i] < target_lens[i] ? input_lens[i] : target_lens[i];
        if (len > longest) longest = len;
    }
    *padded_len = (longest + length_bucket - 1) / length_bucket * length_bucket;
    return FT_OK;
}

int ft_pad_chunk(const uint32_t* const* input_ids, const uint32_t* const* target_ids, const uint8_t* const* loss_masks,
                 const size_t* input_lens, const size_t* target_lens, const size_t* mask_lens, size_t count,
                 size_t padded_len, uint32_t* rows, uint32_t* targets, uint8_t* masks) {
    FT_CHECK_ARG(count == 0 || (input_ids && target_ids && loss_masks && input_lens && target_lens && mask_lens),
                 "ft_pad_chunk: NULL argument");
    FT_CHECK_ARG(count == 0 || padded_len == 0 || (rows && targets && masks), "ft_pad_chunk: NULL output");
    for (size_t s = 0; s < count; s++) {
        const size_t len = input_lens[s] < target_lens[s] ? input_lens[s] : target_lens[s];
        FT_CHECK_ARG(len <= padded_len, "ft_pad_chunk: sequence %zu has %zu tokens, the rows have %zu", s, len, padded_len);
        FT_CHECK_ARG(len == 0 || (input_ids[s] && target_ids[s]), "ft_pad_chunk: sequence %zu is NULL", s);
        const uint32_t pad = len ? input_ids[s][len - 1] : 0;  // the row's last token, for inputs and targets alike
        uint32_t* r = rows + s * padded_len;
        uint32_t* t = targets + s * padded_len;
        uint8_t* m = masks + s * padded_len;
        for (size_t i = 0; i < len; i++) {
            r[i] = input_ids[s][i];
            t[i] = target_ids[s][i];
            m[i] = i < mask_lens[s] && loss_masks[s] ? loss_masks[s][i] : 0;  // loss_mask.get(i).unwrap_or(0)
        }
        for (size_t i = len; i < padded_len; i++) {
            r[i] = pad;
            t[i] = pad;
            m[i] = 0;
        }
    }
    return FT_OK;
}

int ft_trainer_step_in_accum(ft_trainer* t, size_t* sequences) {
    FT_CHECK_ARG(t && sequences, "ft_trainer_step_in_accum: NULL argument");
    *sequences = t->step_in_accum;
    return FT_OK;
}

int ft_trainer_set_optimizer_steps(ft_trainer* t, size_t steps) {
    FT_CHECK_ARG(t, "ft_trainer_set_optimizer_steps: NULL argument");
    t->optimizer_steps = steps;
    return FT_OK;
}

int ft_trainer_train_chunk(ft_trainer* t, const uint32_t* rows, const uint32_t* targets, const uint8_t* loss_mask,
                           size_t B, size_t S, int apply, ft_step_stats* stats, float* per_sequence_loss) {
    return guarded([&]() -> int {
        FT_CHECK_ARG(t && rows && targets && loss_mask && stats, "ft_trainer_train_chunk: NULL argument");
        FT_CHECK_ARG(B > 0 && S > 0, "ft_trainer_train_chunk: empty chunk");
        FT_CHECK_TRAINER_CURRENT(t, "ft_trainer_train_chunk");
        ft_model* m = t->model;
        ft_context* ctx = m->ctx;
        const size_t T = B * S, V = m->cfg.vocab_size;
        const size_t accum = t->cfg.grad_accum_steps ? t->cfg.grad_accum_steps : B;
        std::memset(stats, 0, sizeof(*stats));
        stats->clip_scale = 1.0f;

        std::vector<uint32_t> tg;
        std::vector<float> wt;
        std::vector<size_t> tokens;
        std::vector<uint32_t> head;
        const size_t total_tokens = build_targets(targets, loss_mask, B, S, V, tg, wt, tokens, head);
        stats->supervised_tokens = (uint32_t)total_tokens;
        if (total_tokens == 0) {
            // masked_cross_entropy_batch returns None: no forward result is used, no backward.
            t->step_in_accum += B;
            if (per_sequence_loss)
                for (size_t s = 0; s < B; s++) per_sequence_loss[s] = 0.0f;
        } else {
            FT_TRY(stage_chunk(m, rows, B, S, &head, &tg, &wt));
            FT_TRY(model_forward(m, B, S));
            // Loss + d loss / d logits in place, with the backward seed
            // 1 / grad_accum_steps folded in (trainer/src/lib.rs:474-480, 553-572).
            const float seed = 1.0f / (float)accum;
            const float gscale = std::fabs(seed - 1.0f) > kF32Epsilon ? seed : 1.0f;
            FT_TRY(ft_masked_cross_entropy_weighted(ctx, m->logits, m->targets_dev, m->weights_dev, m->logits,
                                                    m->row_loss, m->head_rows, V, gscale));
            // The first backward of a window overwrites the gradient buffers (the reference's
            // zero_grad after every optimizer step); later ones add to them.
            FT_TRY(model_backward(m, B, S, t->window_has_grads));
            t->window_has_grads = true;
            t->step_in_accum += B;
        }

        const bool window_full = t->step_in_accum >= accum;
        // A window without any supervised token has no gradients: apply_gradients returns
        // before the norm and the optimizer (trainer/src/lib.rs:301-307).
        const bool have_grads = t->window_has_grads;
        bool launched_update = false;
        // Step k (1-based) uses the schedule's value at k (trainer/src/lib.rs:345-352).
        const float lr = ft_lr_schedule(t->cfg.lr_schedule, t->cfg.lr, t->cfg.min_lr, t->cfg.warmup_steps,
                                        t->cfg.total_steps, (uint32_t)(t->optimizer_steps + 1));
        ft_adam_params ap{lr, t->cfg.beta1, t->cfg.beta2, t->cfg.eps, t->cfg.weight_decay, t->t + 1.0f};
        if (window_full) {
            t->step_in_accum = 0;
            t->window_has_grads = false;
            if (have_grads) {
                FT_CHECK_ARG(m->control, "ft_trainer_train_chunk: gradients without a workspace");
                FT_TRY(ft_internal_multi_grad_norm(ctx, t->segs_dev, t->nseg, t->partials, t->cfg.clip_grad_norm,
                                                   m->control));
                if (apply) {
                    FT_TRY(ft_internal_multi_adamw(ctx, t->segs_dev, t->nseg, &ap, 1.0f, m->control));
                    launched_update = true;
                }
            }
        }

        // The step's only wait: row losses and the control block, in one copy.
        if (total_tokens > 0 || (window_full && have_grads)) FT_TRY(fetch_step_out(m));
        if (total_tokens > 0) FT_TRY(read_sequence_losses(m, B, S, tokens, head, per_sequence_loss, &stats->loss));
        if (window_full && have_grads) {
            const float* control = m->out_host + m->ws_B * m->ws_S;
            int applied;
            std::memcpy(&applied, &control[2], 4);
            stats->grad_norm = control[0];
            stats->clip_scale = control[1];
            if (launched_update && applied) {
                // A skipped step leaves both counters alone, so the schedule does not advance either.
                t->t += 1.0f;
                t->optimizer_steps += 1;
                stats->optimizer_step = 1;
                stats->lr = lr;
            }
        }
        return FT_OK;
    });
}

}  // extern "C"
