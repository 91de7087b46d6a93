//! MI355X flavour of the reference's kernel boundary: the same type and method names as
//! `ferrotensor_backend::{WgpuContext, UnifiedTensor, ComputeEngine, AdamParams, AttentionOptions,
//! DType, MASKED_CE_SKIP, SUM_SQUARES_CHUNK}` (ferrotensor-backend/src/lib.rs:38-46), every method
//! forwarding to the entry point of `include/ferrotensor_hip.h` that cites it. `ferrotensor-autograd`,
//! `-graph` and `-trainer` use only these methods, so re-exporting this crate's types from
//! `ferrotensor_backend` (behind a cargo feature) switches them to the HIP library unchanged.
//!
//! Contract kept from the reference: every method enqueues on one in-order stream and returns;
//! outputs are caller-allocated and written, not accumulated; shape and dtype violations panic
//! (the reference `assert!`s, engine/attention.rs:461-500, engine/matmul.rs:140,153);
//! `to_vec` / `synchronize` are the synchronisation points; a tensor's buffer returns to an
//! exact-size pool on its last drop (tensor.rs:106-115).
//!
//! The step driver (`Lfm2Model`, `Trainer`, `train_batch`) is in `step`.
//!
//! Not compiled in this repository's build image (it has no Rust toolchain): the signatures come
//! from the generated `ferrotensor-hip-sys`, whose completeness against the header is tested.
use ferrotensor_hip_sys as sys;

pub mod step;
pub use step::{AdamW, Batch, Lfm2Model, LrSchedule, ModelConfig, StepStats, TrainError, Trainer};
use std::ffi::CStr;
use std::os::raw::c_void;
use std::sync::Arc;

pub const MASKED_CE_SKIP: u32 = sys::FT_MASKED_CE_SKIP; // engine/training.rs:7
pub const SUM_SQUARES_CHUNK: usize = sys::FT_SUM_SQUARES_CHUNK;

/// tensor.rs:18-40 (Q4 is not part of the HIP path).
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum DType {
    FP32,
    FP16,
}

impl DType {
    pub fn size_bytes(&self) -> usize {
        match self {
            DType::FP32 => 4,
            DType::FP16 => 2,
        }
    }
    fn raw(&self) -> i32 {
        match self {
            DType::FP32 => sys::FT_DTYPE_F32,
            DType::FP16 => sys::FT_DTYPE_F16,
        }
    }
}

/// engine/training.rs:13-32.
#[derive(Clone, Copy, Debug)]
pub struct AdamParams {
    pub lr: f32,
    pub beta1: f32,
    pub beta2: f32,
    pub eps: f32,
    pub weight_decay: f32,
    pub t: f32,
}

/// engine/attention.rs:575-594. `window` and `dropout_prob` must be 0 on this path.
#[derive(Clone, Copy, Debug, Default)]
pub struct AttentionOptions {
    pub causal: bool,
    pub causal_offset: u32,
    pub window: u32,
    pub dropout_prob: f32,
    pub seed: u64,
}

impl AttentionOptions {
    fn raw(&self) -> sys::FtAttentionOptions {
        sys::FtAttentionOptions {
            causal: self.causal as i32,
            causal_offset: self.causal_offset,
            window: self.window,
            dropout_prob: self.dropout_prob,
            seed: self.seed,
        }
    }
}

/// The reference panics on shape errors; a failing library call panics with the library's message.
fn check(rc: i32) {
    if rc != sys::FT_OK {
        let msg = unsafe { CStr::from_ptr(sys::ft_last_error()) }.to_string_lossy().into_owned();
        panic!("ferrotensor_hip: {msg}");
    }
}

/// `WgpuContext` (context.rs:50-60): one device, one in-order stream, the buffer pool.
pub struct WgpuContext {
    raw: *mut sys::FtContext,
}
/// The name the rest of the workspace would import on this path.
pub type HipContext = WgpuContext;

unsafe impl Send for WgpuContext {}
unsafe impl Sync for WgpuContext {}

impl WgpuContext {
    /// context.rs:96-156 returns `Result<_, ContextError>`; a missing gfx950 device is the error here.
    pub fn new(device: i32) -> Result<Arc<Self>, String> {
        let mut raw = std::ptr::null_mut();
        let rc = unsafe { sys::ft_context_create(device, &mut raw) };
        if rc != sys::FT_OK {
            return Err(unsafe { CStr::from_ptr(sys::ft_last_error()) }.to_string_lossy().into_owned());
        }
        Ok(Arc::new(Self { raw }))
    }
    /// context.rs:373-378: submit recorded work. Launches are submitted as they are made.
    pub fn flush(&self) {
        check(unsafe { sys::ft_flush(self.raw) });
    }
    /// context.rs:380-391.
    pub fn synchronize(&self) {
        check(unsafe { sys::ft_synchronize(self.raw) });
    }
    pub fn raw(&self) -> *mut sys::FtContext {
        self.raw
    }
}

impl Drop for WgpuContext {
    fn drop(&mut self) {
        unsafe { sys::ft_context_destroy(self.raw) };
    }
}

/// The `Arc<TensorData>` of tensor.rs:53-65.
struct TensorData {
    ctx: Arc<WgpuContext>,
    ptr: *mut c_void,
    bytes: usize,
}
unsafe impl Send for TensorData {}
unsafe impl Sync for TensorData {}

impl Drop for TensorData {
    fn drop(&mut self) {
        // back to the exact-size pool (tensor.rs:106-115); safe without a wait: one in-order stream
        unsafe { sys::ft_free(self.ctx.raw, self.ptr) };
    }
}

/// `UnifiedTensor` (tensor.rs:53-65): device buffer + shape + dtype; clones and views share the buffer.
#[derive(Clone)]
pub struct UnifiedTensor {
    data: Arc<TensorData>,
    pub shape: Vec<usize>,
    pub dtype: DType,
}

impl UnifiedTensor {
    fn alloc(ctx: &Arc<WgpuContext>, shape: &[usize], dtype: DType) -> Self {
        let n: usize = shape.iter().product();
        let bytes = ((n * dtype.size_bytes() + 3) / 4 * 4).max(4); // whole words, as storage bindings need
        let mut ptr = std::ptr::null_mut();
        check(unsafe { sys::ft_alloc(ctx.raw, bytes, &mut ptr) });
        Self { data: Arc::new(TensorData { ctx: ctx.clone(), ptr, bytes }), shape: shape.to_vec(), dtype }
    }
    pub fn ptr(&self) -> *mut c_void {
        self.data.ptr
    }
    fn f32(&self) -> *mut f32 {
        self.data.ptr as *mut f32
    }
    pub fn numel(&self) -> usize {
        self.shape.iter().product()
    }
    /// tensor.rs:124.
    pub fn size_in_bytes(&self) -> u64 {
        self.data.bytes as u64
    }
    /// tensor.rs:146-155.
    pub fn write_data(&self, context: &WgpuContext, data: &[u8]) {
        assert!(data.len() <= self.data.bytes, "write_data: {} bytes into a {}-byte buffer", data.len(), self.data.bytes);
        check(unsafe { sys::ft_upload(context.raw, self.data.ptr, data.as_ptr() as *const c_void, data.len()) });
    }
    /// tensor.rs:157-183.
    pub fn new(context: &Arc<WgpuContext>, data: &[f32], shape: &[usize]) -> Self {
        assert_eq!(data.len(), shape.iter().product::<usize>(), "UnifiedTensor::new: data does not fill {shape:?}");
        let t = Self::alloc(context, shape, DType::FP32);
        check(unsafe { sys::ft_upload(context.raw, t.ptr(), data.as_ptr() as *const c_void, data.len() * 4) });
        t
    }
    /// tensor.rs:185-188: uninitialised.
    pub fn empty(context: &Arc<WgpuContext>, shape: &[usize]) -> Self {
        Self::alloc(context, shape, DType::FP32)
    }
    /// tensor.rs:190-210.
    pub fn empty_with_dtype(context: &Arc<WgpuContext>, shape: &[usize], dtype: DType) -> Self {
        Self::alloc(context, shape, dtype)
    }
    /// tensor.rs:302-305.
    pub fn empty_fp16(context: &Arc<WgpuContext>, shape: &[usize]) -> Self {
        Self::alloc(context, shape, DType::FP16)
    }
    /// tensor.rs:213-218.
    pub fn zeros(context: &Arc<WgpuContext>, shape: &[usize]) -> Self {
        let t = Self::alloc(context, shape, DType::FP32);
        check(unsafe { sys::ft_zero(context.raw, t.ptr(), t.data.bytes) });
        t
    }
    /// tensor.rs:220-223: raw words (e.g. u32 targets) in an FP32-typed buffer.
    pub fn from_bytes(context: &Arc<WgpuContext>, data: &[u8], shape: &[usize]) -> Self {
        let t = Self::alloc(context, shape, DType::FP32);
        t.write_data(context, data);
        t
    }
    /// tensor.rs:261-269: round to nearest even, little endian, two per word, low half first.
    pub fn from_f32_as_f16(context: &Arc<WgpuContext>, data: &[f32], shape: &[usize]) -> Self {
        assert_eq!(data.len(), shape.iter().product::<usize>());
        let t = Self::alloc(context, shape, DType::FP16);
        check(unsafe { sys::ft_upload_f32_as_f16(context.raw, t.ptr(), data.as_ptr(), data.len()) });
        t
    }
    /// tensor.rs:385-406: `data` is `[rows, cols]`; the tensor holds `[cols, rows]`.
    pub fn from_f32_transposed(context: &Arc<WgpuContext>, data: &[f32], rows: usize, cols: usize, dtype: DType) -> Self {
        assert_eq!(data.len(), rows * cols, "from_f32_transposed: data does not fill [{rows}, {cols}]");
        let t = Self::alloc(context, &[cols, rows], dtype);
        check(unsafe { sys::ft_upload_f32_transposed(context.raw, t.ptr(), data.as_ptr(), rows, cols, dtype.raw()) });
        t
    }
    /// tensor.rs:307-330: a view with the same element count.
    pub fn reshaped(&self, new_shape: &[usize]) -> Self {
        assert_eq!(new_shape.iter().product::<usize>(), self.numel(), "reshaped: {new_shape:?} does not hold {} elements", self.numel());
        Self { data: self.data.clone(), shape: new_shape.to_vec(), dtype: self.dtype }
    }
    /// tensor.rs:333-369 (async in the reference; the wait happens inside the library here).
    pub async fn to_vec(&self, context: &WgpuContext) -> Vec<f32> {
        assert_eq!(self.dtype, DType::FP32, "to_vec reads f32 tensors");
        let mut out = vec![0.0f32; self.numel()];
        check(unsafe { sys::ft_download(context.raw, out.as_mut_ptr() as *mut c_void, self.data.ptr, out.len() * 4) });
        out
    }
}

fn rows_of(t: &UnifiedTensor) -> (usize, usize) {
    let size = *t.shape.last().unwrap_or(&1);
    (t.numel() / size.max(1), size)
}

/// `[batch, seq, hidden]` of a 2-D or 3-D tensor (engine/attention.rs:46-60).
fn rope_dims(t: &UnifiedTensor) -> (usize, usize, usize) {
    match t.shape.len() {
        3 => (t.shape[0], t.shape[1], t.shape[2]),
        2 => (1, t.shape[0], t.shape[1]),
        _ => panic!("RoPE expects 2D or 3D tensor, got {:?}", t.shape),
    }
}

struct AttnDims {
    b: usize,
    sq: usize,
    sk: usize,
    h: usize,
    hkv: usize,
    d: usize,
}

/// engine/attention.rs:461-500.
fn attn_dims(q: &UnifiedTensor, k: &UnifiedTensor, mask: Option<&UnifiedTensor>) -> AttnDims {
    assert!(mask.is_none(), "additive attention masks are not supported on the HIP path");
    assert_eq!(q.shape.len(), 4, "q must be [batch, seq, heads, head_dim]");
    assert_eq!(k.shape.len(), 4, "k must be [batch, seq, kv_heads, head_dim]");
    let (b, sq, h, d) = (q.shape[0], q.shape[1], q.shape[2], q.shape[3]);
    let (sk, hkv) = (k.shape[1], k.shape[2]);
    assert!(d <= 128, "flash attention supports head_dim <= 128, got {d}");
    assert!(hkv > 0 && h % hkv == 0, "num_heads ({h}) must be a multiple of num_kv_heads ({hkv})");
    AttnDims { b, sq, sk, h, hkv, d }
}

/// `ComputeEngine` (engine/mod.rs:215-274): the hot subset, argument for argument.
pub struct ComputeEngine;

impl ComputeEngine {
    /// engine/mod.rs:289-346 compiles pipelines; the HIP kernels are in the library already.
    pub fn new(_ctx: &WgpuContext) -> Self {
        Self
    }

    // ---- engine/matmul.rs:94-156 ----
    pub fn matmul(&self, ctx: &WgpuContext, a: &UnifiedTensor, b: &UnifiedTensor, out: &UnifiedTensor) {
        let (m, k, n) = (a.shape[0], a.shape[1], b.shape[1]);
        assert_eq!(b.shape[0], k, "matmul: inner dimensions differ");
        check(unsafe { sys::ft_matmul(ctx.raw, a.f32(), b.f32(), out.f32(), m, k, n) });
    }
    pub fn matmul_bt(&self, ctx: &WgpuContext, a: &UnifiedTensor, b: &UnifiedTensor, out: &UnifiedTensor) {
        let (m, k, n) = (a.shape[0], a.shape[1], b.shape[0]);
        assert_eq!(b.shape[1], k, "matmul_bt: inner dimensions differ");
        check(unsafe { sys::ft_matmul_bt(ctx.raw, a.f32(), b.f32(), out.f32(), m, k, n) });
    }
    pub fn matmul_at(&self, ctx: &WgpuContext, a: &UnifiedTensor, b: &UnifiedTensor, out: &UnifiedTensor) {
        let (k, m, n) = (a.shape[0], a.shape[1], b.shape[1]);
        assert_eq!(b.shape[0], k, "matmul_at: inner dimensions differ");
        check(unsafe { sys::ft_matmul_at(ctx.raw, a.f32(), b.f32(), out.f32(), m, k, n) });
    }
    pub fn matmul_f16b(&self, ctx: &WgpuContext, a: &UnifiedTensor, b: &UnifiedTensor, out: &UnifiedTensor) {
        assert_eq!(b.dtype, DType::FP16, "matmul_f16b: b must be FP16");
        let (m, k, n) = (a.shape[0], a.shape[1], b.shape[1]);
        check(unsafe { sys::ft_matmul_f16b(ctx.raw, a.f32(), b.ptr() as *const u16, out.f32(), m, k, n) });
    }
    pub fn matmul_bt_f16b(&self, ctx: &WgpuContext, a: &UnifiedTensor, b: &UnifiedTensor, out: &UnifiedTensor) {
        assert_eq!(b.dtype, DType::FP16, "matmul_bt_f16b: b must be FP16");
        let (m, k, n) = (a.shape[0], a.shape[1], b.shape[0]);
        check(unsafe { sys::ft_matmul_bt_f16b(ctx.raw, a.f32(), b.ptr() as *const u16, out.f32(), m, k, n) });
    }

    // ---- engine/norm.rs:9-99 ----
    pub fn rms_norm(&self, ctx: &WgpuContext, input: &UnifiedTensor, weight: &UnifiedTensor, out: &UnifiedTensor) {
        self.rms_norm_eps(ctx, input, weight, out, 1e-5);
    }
    pub fn rms_norm_eps(&self, ctx: &WgpuContext, input: &UnifiedTensor, weight: &UnifiedTensor, out: &UnifiedTensor, eps: f32) {
        let (rows, size) = rows_of(input);
        check(unsafe { sys::ft_rms_norm_eps(ctx.raw, input.f32(), weight.f32(), out.f32(), rows, size, eps) });
    }
    #[allow(clippy::too_many_arguments)]
    pub fn rms_norm_backward(&self, ctx: &WgpuContext, input: &UnifiedTensor, weight: &UnifiedTensor, grad_out: &UnifiedTensor,
                             grad_input: &UnifiedTensor, grad_weight: &UnifiedTensor, eps: f32) {
        let (rows, size) = rows_of(input);
        if rows == 0 || size == 0 {
            return;
        }
        check(unsafe {
            sys::ft_rms_norm_backward(ctx.raw, input.f32(), weight.f32(), grad_out.f32(), grad_input.f32(), grad_weight.f32(), rows, size, eps)
        });
    }

    // ---- engine/attention.rs:15-83 ----
    pub fn rope(&self, ctx: &WgpuContext, tensor: &UnifiedTensor, head_dim: usize, pos: usize) {
        self.rope_theta(ctx, tensor, head_dim, pos, 10000.0);
    }
    pub fn rope_theta(&self, ctx: &WgpuContext, tensor: &UnifiedTensor, head_dim: usize, pos: usize, theta: f32) {
        let (b, s, h) = rope_dims(tensor);
        check(unsafe { sys::ft_rope_theta(ctx.raw, tensor.f32(), b, s, h, head_dim, pos, theta) });
    }
    pub fn rope_theta_inverse(&self, ctx: &WgpuContext, tensor: &UnifiedTensor, head_dim: usize, pos: usize, theta: f32) {
        let (b, s, h) = rope_dims(tensor);
        check(unsafe { sys::ft_rope_theta_inverse(ctx.raw, tensor.f32(), b, s, h, head_dim, pos, theta) });
    }

    // ---- engine/attention.rs:139-177, 312-358 ----
    #[allow(clippy::too_many_arguments)]
    pub fn flash_attention_v2_with(&self, ctx: &WgpuContext, q: &UnifiedTensor, k: &UnifiedTensor, v: &UnifiedTensor,
                                   out: &UnifiedTensor, opts: &AttentionOptions, mask: Option<&UnifiedTensor>) {
        let d = attn_dims(q, k, mask);
        let o = opts.raw();
        check(unsafe {
            sys::ft_flash_attention_v2_with_stats(ctx.raw, q.f32(), k.f32(), v.f32(), out.f32(), std::ptr::null_mut(),
                                                  d.b, d.sq, d.sk, d.h, d.hkv, d.d, &o)
        });
    }
    #[allow(clippy::too_many_arguments)]
    pub fn flash_attention_v2_with_stats(&self, ctx: &WgpuContext, q: &UnifiedTensor, k: &UnifiedTensor, v: &UnifiedTensor,
                                         out: &UnifiedTensor, stats: &UnifiedTensor, opts: &AttentionOptions,
                                         mask: Option<&UnifiedTensor>) {
        let d = attn_dims(q, k, mask);
        assert_eq!(stats.numel(), d.b * d.h * d.sq * 2, "attention stats must be [batch * heads * seq, 2]");
        let o = opts.raw();
        check(unsafe {
            sys::ft_flash_attention_v2_with_stats(ctx.raw, q.f32(), k.f32(), v.f32(), out.f32(), stats.f32(),
                                                  d.b, d.sq, d.sk, d.h, d.hkv, d.d, &o)
        });
    }
    #[allow(clippy::too_many_arguments)]
    pub fn flash_attention_v2_backward_with_stats(&self, ctx: &WgpuContext, q: &UnifiedTensor, k: &UnifiedTensor, v: &UnifiedTensor,
                                                  out: &UnifiedTensor, grad_out: &UnifiedTensor, grad_q: &UnifiedTensor,
                                                  grad_k: &UnifiedTensor, grad_v: &UnifiedTensor, stats: &UnifiedTensor,
                                                  opts: &AttentionOptions, mask: Option<&UnifiedTensor>) {
        let d = attn_dims(q, k, mask);
        assert_eq!(stats.numel(), d.b * d.h * d.sq * 2, "attention stats must be [batch * heads * seq, 2]");
        let o = opts.raw();
        check(unsafe {
            sys::ft_flash_attention_v2_backward_with_stats(ctx.raw, q.f32(), k.f32(), v.f32(), out.f32(), grad_out.f32(),
                                                           grad_q.f32(), grad_k.f32(), grad_v.f32(), stats.f32(),
                                                           d.b, d.sq, d.sk, d.h, d.hkv, d.d, &o)
        });
    }

    // ---- engine/elementwise.rs:8-17, 57-75, 183-216 ----
    pub fn add(&self, ctx: &WgpuContext, a: &UnifiedTensor, b: &UnifiedTensor, out: &UnifiedTensor) {
        assert_eq!(a.numel(), b.numel());
        check(unsafe { sys::ft_add(ctx.raw, a.f32(), b.f32(), out.f32(), a.numel()) });
    }
    pub fn add_backward(&self, ctx: &WgpuContext, grad_out: &UnifiedTensor, grad_a: &UnifiedTensor, grad_b: &UnifiedTensor) {
        check(unsafe { sys::ft_add_backward(ctx.raw, grad_out.f32(), grad_a.f32(), grad_b.f32(), grad_out.numel()) });
    }
    /// out = silu(first) * second; the reference names the two `up`, `gate` and calls it `(gate, up)`.
    pub fn silu_gate_fused(&self, ctx: &WgpuContext, up: &UnifiedTensor, gate: &UnifiedTensor, out: &UnifiedTensor) {
        check(unsafe { sys::ft_silu_gate_fused(ctx.raw, up.f32(), gate.f32(), out.f32(), out.numel()) });
    }
    pub fn silu_gate_backward(&self, ctx: &WgpuContext, up: &UnifiedTensor, gate: &UnifiedTensor, grad_out: &UnifiedTensor,
                              grad_up: &UnifiedTensor, grad_gate: &UnifiedTensor) {
        check(unsafe {
            sys::ft_silu_gate_backward(ctx.raw, up.f32(), gate.f32(), grad_out.f32(), grad_up.f32(), grad_gate.f32(), grad_out.numel())
        });
    }

    // ---- engine/training.rs:54-76, 161-283 ----
    pub fn adamw_update(&self, ctx: &WgpuContext, weight: &UnifiedTensor, grad: &UnifiedTensor, m: &UnifiedTensor,
                        v: &UnifiedTensor, params: &AdamParams) {
        let p = sys::FtAdamParams { lr: params.lr, beta1: params.beta1, beta2: params.beta2, eps: params.eps,
                                    weight_decay: params.weight_decay, t: params.t };
        check(unsafe { sys::ft_adamw_update(ctx.raw, weight.f32(), grad.f32(), m.f32(), v.f32(), weight.numel(), &p) });
    }
    pub fn clip_grad_by_norm(&self, ctx: &WgpuContext, grad: &UnifiedTensor, scale: f32) {
        check(unsafe { sys::ft_clip_grad_by_norm(ctx.raw, grad.f32(), grad.numel(), scale) });
    }
    pub fn gradient_accumulate(&self, ctx: &WgpuContext, accum: &UnifiedTensor, grad: &UnifiedTensor) {
        check(unsafe { sys::ft_gradient_accumulate(ctx.raw, accum.f32(), grad.f32(), accum.numel()) });
    }
    pub fn gradient_scale(&self, ctx: &WgpuContext, grad: &UnifiedTensor, scale: f32) {
        check(unsafe { sys::ft_gradient_scale(ctx.raw, grad.f32(), grad.numel(), scale) });
    }
    /// engine/training.rs:207-225: one weight `inv_tokens` for every row.
    pub fn masked_cross_entropy(&self, ctx: &Arc<WgpuContext>, logits: &UnifiedTensor, targets: &UnifiedTensor, inv_tokens: f32,
                                grad: &UnifiedTensor, row_loss: &UnifiedTensor) {
        let (rows, _) = rows_of(logits);
        let weights = UnifiedTensor::new(ctx, &vec![inv_tokens; rows], &[rows]);
        self.masked_cross_entropy_weighted(ctx, logits, targets, &weights, grad, row_loss);
    }
    pub fn masked_cross_entropy_weighted(&self, ctx: &WgpuContext, logits: &UnifiedTensor, targets: &UnifiedTensor,
                                         weights: &UnifiedTensor, grad: &UnifiedTensor, row_loss: &UnifiedTensor) {
        let (rows, vocab) = rows_of(logits);
        if rows == 0 || vocab == 0 {
            return;
        }
        check(unsafe {
            sys::ft_masked_cross_entropy_weighted(ctx.raw, logits.f32(), targets.ptr() as *const u32, weights.f32(), grad.f32(),
                                                  row_loss.f32(), rows, vocab, 1.0)
        });
    }
    pub fn sum_squares_partial(&self, ctx: &WgpuContext, input: &UnifiedTensor, out: &UnifiedTensor, offset: usize) -> usize {
        let mut chunks = 0usize;
        check(unsafe { sys::ft_sum_squares_partial(ctx.raw, input.f32(), input.numel(), out.f32(), offset, &mut chunks) });
        chunks
    }

    /// engine/mod.rs:399-415.
    pub fn copy_tensor(&self, ctx: &WgpuContext, src: &UnifiedTensor, dst: &UnifiedTensor, dst_offset: usize) {
        check(unsafe { sys::ft_copy_tensor(ctx.raw, src.ptr(), src.numel() * src.dtype.size_bytes(), dst.ptr(), dst_offset) });
    }

    // ---- fused entry points without a single counterpart (what `Linear::project_2d`,
    //      graph/src/lib.rs:112-126, and its backward call when built for this path) ----

    /// t = scale * x @ a.
    pub fn lora_down(&self, ctx: &WgpuContext, x: &UnifiedTensor, a: &UnifiedTensor, t: &UnifiedTensor, scale: f32) {
        let (m, k, r) = (x.shape[0], x.shape[1], a.shape[1]);
        check(unsafe { sys::ft_lora_down(ctx.raw, x.f32(), a.f32(), t.f32(), m, k, r, scale) });
    }
    /// y = x @ w (+ t @ b) (+ residual).
    #[allow(clippy::too_many_arguments)]
    pub fn lora_linear(&self, ctx: &WgpuContext, x: &UnifiedTensor, w: &UnifiedTensor, t: Option<&UnifiedTensor>,
                       b: Option<&UnifiedTensor>, residual: Option<&UnifiedTensor>, y: &UnifiedTensor) {
        let (m, k, n) = (x.shape[0], x.shape[1], w.shape[1]);
        let r = b.map_or(0, |b| b.shape[0]);
        let p = |t: Option<&UnifiedTensor>| t.map_or(std::ptr::null(), |t| t.f32() as *const f32);
        check(unsafe { sys::ft_lora_linear(ctx.raw, x.f32(), w.ptr(), w.dtype.raw(), p(t), p(b), p(residual), y.f32(), m, k, n, r) });
    }
    /// dt = scale * dy @ b^T.
    pub fn lora_grad_down(&self, ctx: &WgpuContext, dy: &UnifiedTensor, b: &UnifiedTensor, dt: &UnifiedTensor, scale: f32) {
        let (m, n, r) = (dy.shape[0], dy.shape[1], b.shape[0]);
        check(unsafe { sys::ft_lora_grad_down(ctx.raw, dy.f32(), b.f32(), dt.f32(), m, n, r, scale) });
    }
    /// dx = dy @ w^T (+ dt @ a^T) (+ residual).
    #[allow(clippy::too_many_arguments)]
    pub fn lora_linear_dx(&self, ctx: &WgpuContext, dy: &UnifiedTensor, w: &UnifiedTensor, dt: Option<&UnifiedTensor>,
                          a: Option<&UnifiedTensor>, residual: Option<&UnifiedTensor>, dx: &UnifiedTensor) {
        let (m, n, k) = (dy.shape[0], dy.shape[1], w.shape[0]);
        let r = a.map_or(0, |a| a.shape[1]);
        let p = |t: Option<&UnifiedTensor>| t.map_or(std::ptr::null(), |t| t.f32() as *const f32);
        check(unsafe { sys::ft_lora_linear_dx(ctx.raw, dy.f32(), w.ptr(), w.dtype.raw(), p(dt), p(a), p(residual), dx.f32(), m, k, n, r) });
    }
    /// db = t^T @ dy, da = x^T @ dt.
    pub fn lora_grad_b(&self, ctx: &WgpuContext, t: &UnifiedTensor, dy: &UnifiedTensor, db: &UnifiedTensor) {
        let (m, r, n) = (t.shape[0], t.shape[1], dy.shape[1]);
        check(unsafe { sys::ft_lora_grad_b(ctx.raw, t.f32(), dy.f32(), db.f32(), m, n, r) });
    }
    pub fn lora_grad_a(&self, ctx: &WgpuContext, x: &UnifiedTensor, dt: &UnifiedTensor, da: &UnifiedTensor) {
        let (m, k, r) = (x.shape[0], x.shape[1], dt.shape[1]);
        check(unsafe { sys::ft_lora_grad_a(ctx.raw, x.f32(), dt.f32(), da.f32(), m, k, r) });
    }
    /// out = rows `ids` of `table` (zero rows for ids >= vocab): the host gather of
    /// `Tensor::embedding` (autograd/src/lib.rs:1159-1179) on the device.
    pub fn embedding(&self, ctx: &WgpuContext, table: &UnifiedTensor, ids: &UnifiedTensor, out: &UnifiedTensor) {
        let (vocab, hidden) = (table.shape[0], table.shape[1]);
        check(unsafe { sys::ft_embedding(ctx.raw, table.f32(), vocab, hidden, ids.ptr() as *const u32, ids.numel(), out.f32()) });
    }
}
