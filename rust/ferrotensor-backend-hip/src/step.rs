//! The fast path of the training step behind the reference's own names: `Lfm2Model`
//! (ferrotensor-graph/src/lfm.rs), `Trainer`, `StepStats`, `TrainError`
//! (ferrotensor-trainer/src/lib.rs:42-111, 371-502) and `Batch`
//! (ferrotensor-trainer/src/data.rs:323-339), over the `ft_model_*` / `ft_trainer_*` entry
//! points of `include/ferrotensor_hip.h`. The model, loss, backward pass and optimizer step
//! run inside the library as one fixed sequence of fused launches; this module owns the
//! handles and reproduces the host side of `train_batch` (which sequences train, where the
//! chunks end, how rows are padded) through the library's integer routines.
//!
//! Differences a caller sees: the optimizer is the library's AdamW (`AdamW` below holds its
//! settings, as `AdamW::new(lr)` + fields do in ferrotensor-autograd/src/lib.rs:1482-1515);
//! the trainable parameters are the model's own list (LoRA factors, and the base weights of a
//! `trainable_base` model), so `train_batch` takes no `train_params`.
//!
//! Not compiled in this repository's build image (it has no Rust toolchain).
use crate::{sys, WgpuContext};
use std::ffi::{CStr, CString};
use std::sync::Arc;

fn last_error() -> String {
    unsafe { CStr::from_ptr(sys::ft_last_error()) }.to_string_lossy().into_owned()
}

/// Error from a training step (ferrotensor-trainer/src/lib.rs:60-70).
#[derive(Debug)]
pub struct TrainError(pub String);

impl std::fmt::Display for TrainError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        f.write_str(&self.0)
    }
}

impl std::error::Error for TrainError {}

fn ok(rc: i32) -> Result<(), TrainError> {
    if rc == sys::FT_OK {
        Ok(())
    } else {
        Err(TrainError(last_error()))
    }
}

/// Result of one chunk (ferrotensor-trainer/src/lib.rs:42-58). `loss` is the sum of the chunk's
/// per-sequence mean losses, as `train_chunk` reports it; `clip_scale` is extra.
#[derive(Clone, Copy, Debug, PartialEq)]
pub struct StepStats {
    pub loss: f32,
    pub tokens: usize,
    pub optimizer_step: bool,
    pub grad_norm: Option<f32>,
    pub lr: Option<f32>,
    pub clip_scale: f32,
}

/// Batch of training data (ferrotensor-trainer/src/data.rs:323-339).
pub struct Batch {
    pub input_ids: Vec<Vec<u32>>,
    pub target_ids: Vec<Vec<u32>>,
    pub padded_input_ids: Vec<Vec<u32>>,
    pub padded_target_ids: Vec<Vec<u32>>,
    pub attention_mask: Vec<Vec<u8>>,
    pub loss_masks: Vec<Vec<u8>>,
    pub batch_size: usize,
}

/// The fields of `Lfm2Config` the step needs (ferrotensor-loader/src/lib.rs:74-142) and the
/// builder's switches (model_builder.rs:325-357, lfm.rs:347-350).
#[derive(Clone, Copy, Debug)]
pub struct ModelConfig {
    pub vocab_size: u32,
    pub hidden_size: u32,
    pub intermediate_size: u32,
    pub num_hidden_layers: u32,
    pub num_attention_heads: u32,
    pub num_key_value_heads: u32,
    pub rms_norm_eps: f32,
    pub rope_theta: f32,
    pub tie_word_embeddings: bool,
    pub f16_linears: bool,
    pub checkpoint_blocks: bool,
    pub trainable_base: bool,
}

/// `Lfm2Model` for all-attention (Llama / SmolLM2) checkpoints.
pub struct Lfm2Model {
    ctx: Arc<WgpuContext>,
    raw: *mut sys::FtModel,
}

unsafe impl Send for Lfm2Model {}

impl Lfm2Model {
    /// `Lfm2ModelBuilder::build` (model_builder.rs:623-709): an empty model; the weights arrive
    /// through `set_tensor`.
    pub fn new(ctx: Arc<WgpuContext>, config: &ModelConfig) -> Result<Self, TrainError> {
        let cfg = sys::FtModelConfig {
            vocab_size: config.vocab_size,
            hidden_size: config.hidden_size,
            intermediate_size: config.intermediate_size,
            num_hidden_layers: config.num_hidden_layers,
            num_attention_heads: config.num_attention_heads,
            num_key_value_heads: config.num_key_value_heads,
            rms_norm_eps: config.rms_norm_eps,
            rope_theta: config.rope_theta,
            tie_word_embeddings: config.tie_word_embeddings as i32,
            f16_linears: config.f16_linears as i32,
            checkpoint_blocks: config.checkpoint_blocks as i32,
            head_all_rows: 0,
            trainable_base: config.trainable_base as i32,
        };
        let mut raw = std::ptr::null_mut();
        ok(unsafe { sys::ft_model_create(ctx.raw(), &cfg, &mut raw) })?;
        Ok(Self { ctx, raw })
    }
    pub fn ctx(&self) -> &Arc<WgpuContext> {
        &self.ctx
    }
    /// One Hugging Face tensor by name, `[out, in]` for linears (model_builder.rs:400-424, 653-689).
    pub fn set_tensor(&mut self, hf_name: &str, data: &[f32], shape: &[usize]) -> Result<(), TrainError> {
        assert_eq!(data.len(), shape.iter().product::<usize>(), "set_tensor: data does not fill {shape:?}");
        let name = CString::new(hf_name).map_err(|e| TrainError(e.to_string()))?;
        ok(unsafe { sys::ft_model_set_tensor(self.raw, name.as_ptr(), data.as_ptr(), shape.as_ptr(), shape.len() as i32) })
    }
    /// `ModelBuilder::maybe_add_lora` (model_builder.rs:425-446): seeded A, zero B.
    pub fn add_lora(&mut self, prefix: &str, rank: usize, alpha: f32) -> Result<(), TrainError> {
        let name = CString::new(prefix).map_err(|e| TrainError(e.to_string()))?;
        ok(unsafe { sys::ft_model_add_lora(self.raw, name.as_ptr(), rank, alpha) })
    }
    /// An adapter with given factors, `a [in, rank]`, `b [rank, out]` (graph/src/lib.rs:28-56).
    pub fn set_lora(&mut self, prefix: &str, a: &[f32], b: &[f32], rank: usize, alpha: f32) -> Result<(), TrainError> {
        let name = CString::new(prefix).map_err(|e| TrainError(e.to_string()))?;
        ok(unsafe { sys::ft_model_set_lora(self.raw, name.as_ptr(), a.as_ptr(), b.as_ptr(), rank, alpha) })
    }
    /// `named_lora_params` (lfm.rs:756-770) and, with a trainable base, the weights: name and size.
    pub fn named_params(&self) -> Result<Vec<(String, usize)>, TrainError> {
        let mut count = 0usize;
        ok(unsafe { sys::ft_model_param_count(self.raw, &mut count) })?;
        let mut out = Vec::with_capacity(count);
        for index in 0..count {
            let mut name = std::ptr::null();
            let mut numel = 0usize;
            ok(unsafe { sys::ft_model_param_info(self.raw, index, &mut name, &mut numel) })?;
            out.push((unsafe { CStr::from_ptr(name) }.to_string_lossy().into_owned(), numel));
        }
        Ok(out)
    }
    pub fn read_param(&self, index: usize, numel: usize) -> Result<Vec<f32>, TrainError> {
        let mut out = vec![0.0f32; numel];
        ok(unsafe { sys::ft_model_read_param(self.raw, index, out.as_mut_ptr()) })?;
        Ok(out)
    }
    pub fn write_param(&mut self, index: usize, values: &[f32]) -> Result<(), TrainError> {
        ok(unsafe { sys::ft_model_write_param(self.raw, index, values.as_ptr()) })
    }
    pub fn read_grad(&self, index: usize, numel: usize) -> Result<Vec<f32>, TrainError> {
        let mut out = vec![0.0f32; numel];
        ok(unsafe { sys::ft_model_read_grad(self.raw, index, out.as_mut_ptr()) })?;
        Ok(out)
    }
    /// `Lfm2Model::forward_batch` (lfm.rs:590-623): logits `[B * S, vocab]` of equally long rows.
    pub fn forward_batch(&self, rows: &[&[u32]], vocab_size: usize) -> Result<Vec<f32>, TrainError> {
        let b = rows.len();
        let s = rows.first().map_or(0, |r| r.len());
        assert!(rows.iter().all(|r| r.len() == s), "forward_batch: rows of different lengths");
        let flat: Vec<u32> = rows.iter().flat_map(|r| r.iter().copied()).collect();
        let mut logits = vec![0.0f32; b * s * vocab_size];
        ok(unsafe { sys::ft_model_forward_logits(self.raw, flat.as_ptr(), b, s, logits.as_mut_ptr()) })?;
        Ok(logits)
    }
    /// The forward-only loss of `evaluate` (ferrotensor-cli/src/main.rs:1110-1137): per sequence,
    /// the mean loss over its supervised targets and their count.
    pub fn eval_chunk(&self, rows: &[u32], targets: &[u32], loss_mask: &[u8], b: usize, s: usize)
                      -> Result<(Vec<f32>, Vec<u32>), TrainError> {
        assert!(rows.len() == b * s && targets.len() == b * s && loss_mask.len() == b * s, "eval_chunk: not [B, S]");
        let (mut loss, mut tokens) = (vec![0.0f32; b], vec![0u32; b]);
        ok(unsafe {
            sys::ft_model_eval_chunk(self.raw, rows.as_ptr(), targets.as_ptr(), loss_mask.as_ptr(), b, s,
                                     loss.as_mut_ptr(), tokens.as_mut_ptr())
        })?;
        Ok((loss, tokens))
    }
}

impl Drop for Lfm2Model {
    fn drop(&mut self) {
        unsafe { sys::ft_model_destroy(self.raw) };
    }
}

/// The settings of `AdamW` (ferrotensor-autograd/src/lib.rs:1482-1515): `AdamW::new(lr)` has
/// betas (0.9, 0.999), eps 1e-8, weight decay 0.01; the CLI's train command sets decay 0.
#[derive(Clone, Copy, Debug)]
pub struct AdamW {
    pub lr: f32,
    pub beta1: f32,
    pub beta2: f32,
    pub eps: f32,
    pub weight_decay: f32,
}

impl AdamW {
    pub fn new(lr: f32) -> Self {
        Self { lr, beta1: 0.9, beta2: 0.999, eps: 1e-8, weight_decay: 0.01 }
    }
}

/// `LRScheduler` choices (ferrotensor-autograd/src/lib.rs:1708-1814); the optimizer's `lr` is the peak.
#[derive(Clone, Copy, Debug)]
pub enum LrSchedule {
    Constant,
    CosineAnnealing { total_steps: u32, min_lr: f32 },
    WarmupCosine { warmup_steps: u32, total_steps: u32, min_lr: f32 },
}

/// Runs optimization steps on a model (ferrotensor-trainer/src/lib.rs:72-111).
pub struct Trainer {
    pub model: Lfm2Model,
    pub optimizer: AdamW,
    pub clip_grad_norm: Option<f32>,
    pub grad_accum_steps: usize,
    pub lr_scheduler: LrSchedule,
    pub length_bucket: usize,
    raw: *mut sys::FtTrainer,
}

unsafe impl Send for Trainer {}

impl Trainer {
    /// A trainer with no clipping, accumulation or schedule (`Trainer::new`, :113-135).
    pub fn new(model: Lfm2Model, optimizer: AdamW) -> Self {
        Self {
            model,
            optimizer,
            clip_grad_norm: None,
            grad_accum_steps: 1,
            lr_scheduler: LrSchedule::Constant,
            length_bucket: 32,
            raw: std::ptr::null_mut(),
        }
    }
    /// :154-157.
    pub fn with_grad_accum_steps(mut self, steps: usize) -> Self {
        self.grad_accum_steps = steps.max(1);
        self
    }
    /// :159-163.
    pub fn with_clip_grad_norm(mut self, max_norm: f32) -> Self {
        self.clip_grad_norm = Some(max_norm);
        self
    }
    /// :172-176.
    pub fn with_lr_scheduler(mut self, schedule: LrSchedule) -> Self {
        self.lr_scheduler = schedule;
        self
    }
    /// :195-199. 1 disables padding.
    pub fn with_length_bucket(mut self, tokens: usize) -> Self {
        self.length_bucket = tokens.max(1);
        self
    }

    /// The library-side trainer is made at the first step, once the builder calls are over.
    fn handle(&mut self) -> Result<*mut sys::FtTrainer, TrainError> {
        if self.raw.is_null() {
            let (lr_schedule, warmup_steps, total_steps, min_lr) = match self.lr_scheduler {
                LrSchedule::Constant => (sys::FT_LR_CONSTANT, 0, 0, 0.0),
                LrSchedule::CosineAnnealing { total_steps, min_lr } => (sys::FT_LR_COSINE, 0, total_steps, min_lr),
                LrSchedule::WarmupCosine { warmup_steps, total_steps, min_lr } => {
                    (sys::FT_LR_WARMUP_COSINE, warmup_steps, total_steps, min_lr)
                }
            };
            let cfg = sys::FtTrainerConfig {
                lr: self.optimizer.lr,
                beta1: self.optimizer.beta1,
                beta2: self.optimizer.beta2,
                eps: self.optimizer.eps,
                weight_decay: self.optimizer.weight_decay,
                clip_grad_norm: self.clip_grad_norm.unwrap_or(0.0),
                grad_accum_steps: self.grad_accum_steps as u32,
                lr_schedule,
                warmup_steps,
                total_steps,
                min_lr,
            };
            ok(unsafe { sys::ft_trainer_create(self.model.raw, &cfg, &mut self.raw) })?;
        }
        Ok(self.raw)
    }

    /// Sequences counted into the open accumulation window (`step_in_accum`, :86-89).
    pub fn step_in_accum(&mut self) -> Result<usize, TrainError> {
        let t = self.handle()?;
        let mut n = 0usize;
        ok(unsafe { sys::ft_trainer_step_in_accum(t, &mut n) })?;
        Ok(n)
    }
    /// :201-204.
    pub fn optimizer_steps(&mut self) -> Result<usize, TrainError> {
        let t = self.handle()?;
        let mut n = 0usize;
        ok(unsafe { sys::ft_trainer_optimizer_steps(t, &mut n) })?;
        Ok(n)
    }
    /// Resume (:206-213): the step counter is also the position of the learning-rate schedule.
    pub fn set_optimizer_steps(&mut self, steps: usize) -> Result<(), TrainError> {
        let t = self.handle()?;
        ok(unsafe { sys::ft_trainer_set_optimizer_steps(t, steps) })
    }

    /// One sequence (`train_step_masked`, :228-294): a chunk of one.
    pub fn train_step_masked(&mut self, input_ids: &[u32], target_ids: &[u32], loss_mask: Option<&[u8]>)
                             -> Result<StepStats, TrainError> {
        let ones;
        let mask = match loss_mask {
            Some(m) => m,
            None => {
                ones = vec![1u8; input_ids.len().min(target_ids.len())];
                &ones[..]
            }
        };
        self.train_chunk(&[(input_ids, target_ids, mask)])
    }

    /// `Trainer::train_batch` (:371-423): rows are cut at their attention mask, rows that cannot
    /// train are dropped, the rest run in chunks that end at the accumulation boundary. One
    /// `StepStats` per chunk.
    pub fn train_batch(&mut self, batch: &Batch) -> Result<Vec<StepStats>, TrainError> {
        let n = batch.batch_size;
        let padded_len = batch.padded_input_ids.first().map_or(0, |r| r.len());
        let flat32 = |rows: &Vec<Vec<u32>>| rows.iter().flat_map(|r| r.iter().copied()).collect::<Vec<u32>>();
        let flat8 = |rows: &Vec<Vec<u8>>| rows.iter().flat_map(|r| r.iter().copied()).collect::<Vec<u8>>();
        let (ids, tgs) = (flat32(&batch.padded_input_ids), flat32(&batch.padded_target_ids));
        let (attn, mask) = (flat8(&batch.attention_mask), flat8(&batch.loss_masks));
        assert!(ids.len() == n * padded_len && tgs.len() == n * padded_len && attn.len() == n * padded_len
                    && mask.len() == n * padded_len, "train_batch: the batch is not [batch_size, padded_len]");
        let mut valid = vec![0usize; n.max(1)];
        let mut kept = 0usize;
        ok(unsafe {
            sys::ft_train_batch_select(ids.as_ptr(), tgs.as_ptr(), attn.as_ptr(), mask.as_ptr(), n, padded_len,
                                       valid.as_mut_ptr(), &mut kept)
        })?;
        let mut seqs: Vec<(&[u32], &[u32], &[u8])> = Vec::with_capacity(kept);
        for b in 0..n {
            let len = valid[b];
            if len > 0 {
                seqs.push((&batch.padded_input_ids[b][..len], &batch.padded_target_ids[b][..len],
                           &batch.loss_masks[b][..len]));
            }
        }
        let in_accum = self.step_in_accum()?;
        let mut sizes = vec![0usize; seqs.len().max(1)];
        let mut chunks = 0usize;
        ok(unsafe {
            sys::ft_train_batch_plan(seqs.len(), self.grad_accum_steps, in_accum, sizes.as_mut_ptr(), &mut chunks)
        })?;
        let mut out = Vec::with_capacity(chunks);
        let mut rest = seqs.as_slice();
        for &size in &sizes[..chunks] {
            let (chunk, tail) = rest.split_at(size);
            out.push(self.train_chunk(chunk)?);
            rest = tail;
        }
        Ok(out)
    }

    /// `Trainer::train_chunk` (:426-502): pad to a common bucketed length, then forward, loss,
    /// backward and, when the accumulation window is full, gradient norm, clip and AdamW.
    pub fn train_chunk(&mut self, chunk: &[(&[u32], &[u32], &[u8])]) -> Result<StepStats, TrainError> {
        let t = self.handle()?;
        let count = chunk.len();
        let ids: Vec<*const u32> = chunk.iter().map(|s| s.0.as_ptr()).collect();
        let tgs: Vec<*const u32> = chunk.iter().map(|s| s.1.as_ptr()).collect();
        let mks: Vec<*const u8> = chunk.iter().map(|s| s.2.as_ptr()).collect();
        let il: Vec<usize> = chunk.iter().map(|s| s.0.len()).collect();
        let tl: Vec<usize> = chunk.iter().map(|s| s.1.len()).collect();
        let ml: Vec<usize> = chunk.iter().map(|s| s.2.len()).collect();
        let mut padded_len = 0usize;
        ok(unsafe { sys::ft_chunk_padded_len(il.as_ptr(), tl.as_ptr(), count, self.length_bucket, &mut padded_len) })?;
        let mut rows = vec![0u32; count * padded_len];
        let mut targets = vec![0u32; count * padded_len];
        let mut masks = vec![0u8; count * padded_len];
        ok(unsafe {
            sys::ft_pad_chunk(ids.as_ptr(), tgs.as_ptr(), mks.as_ptr(), il.as_ptr(), tl.as_ptr(), ml.as_ptr(), count,
                              padded_len, rows.as_mut_ptr(), targets.as_mut_ptr(), masks.as_mut_ptr())
        })?;
        let mut st = sys::FtStepStats { loss: 0.0, grad_norm: 0.0, clip_scale: 1.0, supervised_tokens: 0, optimizer_step: 0, lr: 0.0 };
        ok(unsafe {
            sys::ft_trainer_train_chunk(t, rows.as_ptr(), targets.as_ptr(), masks.as_ptr(), count, padded_len, 1, &mut st,
                                        std::ptr::null_mut())
        })?;
        let stepped = st.optimizer_step != 0;
        Ok(StepStats {
            loss: st.loss,
            tokens: st.supervised_tokens as usize,
            optimizer_step: stepped,
            grad_norm: if stepped { Some(st.grad_norm) } else { None },
            lr: if stepped { Some(st.lr) } else { None },
            clip_scale: st.clip_scale,
        })
    }

    /// AdamW moments of parameter `index`, for the optimizer-state file (`AdamW::save_state`,
    /// ferrotensor-autograd/src/lib.rs:1577-1628).
    pub fn read_moments(&mut self, index: usize, numel: usize) -> Result<(Vec<f32>, Vec<f32>), TrainError> {
        let t = self.handle()?;
        let (mut m, mut v) = (vec![0.0f32; numel], vec![0.0f32; numel]);
        ok(unsafe { sys::ft_trainer_read_moments(t, index, m.as_mut_ptr(), v.as_mut_ptr()) })?;
        Ok((m, v))
    }
    /// `AdamW::load_state` (:1630-1662): hyperparameters and step counter first, then the moments.
    pub fn load_state(&mut self, saved: &AdamW, t_steps: f32, moments: &[(usize, Vec<f32>, Vec<f32>)])
                      -> Result<(), TrainError> {
        let t = self.handle()?;
        ok(unsafe { sys::ft_trainer_set_adam_hyper(t, saved.lr, saved.beta1, saved.beta2, saved.eps, saved.weight_decay) })?;
        ok(unsafe { sys::ft_trainer_set_adam_t(t, t_steps) })?;
        for (index, m, v) in moments {
            ok(unsafe { sys::ft_trainer_write_moments(t, *index, m.as_ptr(), v.as_ptr()) })?;
        }
        self.optimizer = *saved;
        Ok(())
    }
    pub fn adam_t(&mut self) -> Result<f32, TrainError> {
        let t = self.handle()?;
        let mut steps = 0.0f32;
        ok(unsafe { sys::ft_trainer_get_adam_t(t, &mut steps) })?;
        Ok(steps)
    }
}

impl Drop for Trainer {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { sys::ft_trainer_destroy(self.raw) };
        }
    }
}
