"""Python mirror of the reference's model and trainer over the library's step driver.

`Lfm2Model` follows `ferrotensor_graph::lfm::Lfm2Model` + `Lfm2ModelBuilder`
(ferrotensor-graph/src/lfm.rs:590-623, model_builder.rs:623-709) and `Trainer`
follows `ferrotensor_trainer::Trainer` (ferrotensor-trainer/src/lib.rs:74-135,
371-502). The work happens in libferrotensor_hip.so (`ft_model_*`,
`ft_trainer_*`); this file only marshals host arrays.
"""
import ctypes as C
import weakref
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import _lib
from ._lib import check
from .engine import HipContext


@dataclass
class ModelConfig:
    """The `Lfm2Config` fields the step uses (ferrotensor-loader/src/lib.rs:74-142)."""
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    f16_linears: bool = False
    checkpoint_blocks: bool = False
    head_all_rows: bool = False
    trainable_base: bool = False

    def c(self):
        return _lib.ModelConfigC(self.vocab_size, self.hidden_size, self.intermediate_size, self.num_hidden_layers,
                                 self.num_attention_heads, self.num_key_value_heads, self.rms_norm_eps,
                                 self.rope_theta, 1 if self.tie_word_embeddings else 0, 1 if self.f16_linears else 0,
                                 1 if self.checkpoint_blocks else 0, 1 if self.head_all_rows else 0,
                                 1 if self.trainable_base else 0)


@dataclass
class LoRaConfig:
    """model_builder.rs `LoRaConfig`: rank, alpha, target module names."""
    rank: int = 8
    alpha: float = 16.0
    target_modules: Tuple[str, ...] = ("q_proj", "k_proj", "v_proj", "o_proj")


@dataclass
class StepStats:
    """trainer/src/lib.rs:36-58 for one chunk."""
    loss: float
    tokens: int
    optimizer_step: bool
    grad_norm: Optional[float]
    clip_scale: float
    per_sequence: List[float]
    lr: Optional[float] = None


class Lfm2Model:
    def __init__(self, ctx: HipContext, config: ModelConfig):
        self.ctx = ctx
        self.config = config
        self._lib = ctx._lib
        h = C.c_void_p()
        cfg = config.c()
        check(self._lib.ft_model_create(ctx.handle, C.byref(cfg), C.byref(h)))
        self.handle = h
        self._trainers = []
        ctx._adopt(self)

    def set_tensor(self, hf_name: str, data):
        """One Hugging Face tensor ([out, in] for linears); the library applies the builder's layout rules."""
        data = np.ascontiguousarray(data, np.float32)
        shape = (C.c_size_t * data.ndim)(*data.shape)
        check(self._lib.ft_model_set_tensor(self.handle, hf_name.encode(), data.ctypes.data_as(C.c_void_p), shape,
                                            data.ndim))

    def load_tensors(self, tensors: Dict[str, np.ndarray]):
        for name, value in tensors.items():
            self.set_tensor(name, value)

    def set_lora(self, prefix: str, a, b, alpha: float):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        assert a.ndim == 2 and b.ndim == 2 and a.shape[1] == b.shape[0]
        check(self._lib.ft_model_set_lora(self.handle, prefix.encode(), a.ctypes.data_as(C.c_void_p),
                                          b.ctypes.data_as(C.c_void_p), a.shape[1], alpha))

    def add_lora(self, prefix: str, rank: int, alpha: float):
        """`ModelBuilder::maybe_add_lora`: a fresh adapter, A seeded from (layer, module name), B zero."""
        check(self._lib.ft_model_add_lora(self.handle, prefix.encode(), rank, alpha))

    def set_head_all_rows(self, all_rows: bool):
        """True: final norm, vocabulary head and loss on every position (the reference's behaviour); False: on
        the supervised positions only (same results, less work)."""
        check(self._lib.ft_model_set_head_all_rows(self.handle, 1 if all_rows else 0))
        self.config.head_all_rows = bool(all_rows)

    def linear_prefixes(self, targets: Sequence[str]) -> List[str]:
        out = []
        for l in range(self.config.num_hidden_layers):
            for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
                if n in targets:
                    out.append(f"model.layers.{l}.self_attn.{n}")
            for n in ("gate_proj", "up_proj", "down_proj"):
                if n in targets:
                    out.append(f"model.layers.{l}.mlp.{n}")
        if "lm_head" in targets:
            out.append("lm_head")
        return out

    def linear_dims(self, prefix: str) -> Tuple[int, int]:
        c = self.config
        d = c.hidden_size // c.num_attention_heads
        table = {"q_proj": (c.hidden_size, c.num_attention_heads * d),
                 "k_proj": (c.hidden_size, c.num_key_value_heads * d),
                 "v_proj": (c.hidden_size, c.num_key_value_heads * d),
                 "o_proj": (c.num_attention_heads * d, c.hidden_size),
                 "gate_proj": (c.hidden_size, c.intermediate_size),
                 "up_proj": (c.hidden_size, c.intermediate_size),
                 "down_proj": (c.intermediate_size, c.hidden_size),
                 "lm_head": (c.hidden_size, c.vocab_size)}
        return table[prefix.split(".")[-1]]

    def named_params(self) -> List[Tuple[str, int]]:
        n = C.c_size_t()
        check(self._lib.ft_model_param_count(self.handle, C.byref(n)))
        out = []
        for i in range(n.value):
            name, numel = C.c_char_p(), C.c_size_t()
            check(self._lib.ft_model_param_info(self.handle, i, C.byref(name), C.byref(numel)))
            out.append((name.value.decode(), numel.value))
        return out

    def write_param(self, index: int, values):
        """Overwrites trainable tensor `index` (the order of `named_params`) in place."""
        numel = self.named_params()[index][1]
        v = np.ascontiguousarray(values, np.float32).reshape(-1)
        assert v.size == numel, "write_param: %d values for a parameter of %d" % (v.size, numel)
        check(self._lib.ft_model_write_param(self.handle, index, v.ctypes.data_as(C.c_void_p)))

    def _read(self, fn, index, numel):
        out = np.empty(numel, np.float32)
        check(fn(self.handle, index, out.ctypes.data_as(C.c_void_p)))
        return out

    def params(self) -> Dict[str, np.ndarray]:
        return {n: self._read(self._lib.ft_model_read_param, i, k) for i, (n, k) in enumerate(self.named_params())}

    def grads(self) -> Dict[str, np.ndarray]:
        return {n: self._read(self._lib.ft_model_read_grad, i, k) for i, (n, k) in enumerate(self.named_params())}

    def forward_batch(self, rows) -> np.ndarray:
        """`Lfm2Model::forward_batch`: logits [B, S, vocab] on the host."""
        rows = np.ascontiguousarray(rows, np.uint32)
        assert rows.ndim == 2, "forward_batch: rows must have the same length"
        B, S = rows.shape
        out = np.empty((B, S, self.config.vocab_size), np.float32)
        check(self._lib.ft_model_forward_logits(self.handle, rows.ctypes.data_as(C.c_void_p), B, S,
                                                out.ctypes.data_as(C.c_void_p)))
        return out

    def evaluate(self, seqs, batch: int = 8, length_bucket: int = 32) -> Tuple[float, int]:
        """`evaluate` of the CLI (ferrotensor-cli/src/main.rs:1110-1137): token-weighted mean loss
        over [(input_ids, target_ids, loss_mask)] and the number of supervised tokens; (nan, 0) when
        nothing is supervised. Forward only."""
        loss_sum, tokens = 0.0, 0
        kept = [(i, t, m) for i, t, m in seqs if len(i) > 0 and len(t) > 0]
        for at in range(0, len(kept), batch):
            rows, targets, masks = pad_chunk(kept[at:at + batch], length_bucket)
            B, S = rows.shape
            per, cnt = np.zeros(B, np.float32), np.zeros(B, np.uint32)
            check(self._lib.ft_model_eval_chunk(self.handle, rows.ctypes.data_as(C.c_void_p),
                                                targets.ctypes.data_as(C.c_void_p), masks.ctypes.data_as(C.c_void_p),
                                                B, S, per.ctypes.data_as(C.c_void_p), cnt.ctypes.data_as(C.c_void_p)))
            loss_sum += float((per.astype(np.float64) * cnt).sum())
            tokens += int(cnt.sum())
        return (float("nan"), 0) if tokens == 0 else (loss_sum / tokens, tokens)

    def close(self):
        if self.handle is not None and self.handle.value:
            for ref in self._trainers:
                t = ref()
                if t is not None:
                    t.close()
            self._lib.ft_model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


LR_SCHEDULES = {"constant": 0, "cosine": 1, "warmup_cosine": 2}


def lr_schedule(kind: str, peak_lr: float, min_lr: float, warmup_steps: int, total_steps: int, step: int) -> float:
    """`LRScheduler::get_lr` after `step` calls of `step()` (autograd/src/lib.rs:1705-1814)."""
    return float(_lib.load().ft_lr_schedule(LR_SCHEDULES[kind], peak_lr, min_lr, warmup_steps, total_steps, step))


def lora_seed(layer_seed: int, module_name: str) -> int:
    """`lora_seed` (model_builder.rs:739-759)."""
    return int(_lib.load().ft_lora_seed(layer_seed, module_name.encode()))


def lora_init_a(in_dim: int, out_dim: int, rank: int, seed: int) -> np.ndarray:
    """`LoRAAdapter::new_seeded`'s A matrix [in_dim, rank] (graph/src/lib.rs:59-92)."""
    a = np.empty((in_dim, rank), np.float32)
    check(_lib.load().ft_lora_init_a(a.ctypes.data_as(C.c_void_p), in_dim, out_dim, rank, seed))
    return a


def pad_chunk(seqs, length_bucket=32):
    """`Trainer::train_chunk` padding (trainer/src/lib.rs:431-450) through `ft_chunk_padded_len` and
    `ft_pad_chunk`: right-pad to a multiple of `length_bucket` with each row's last token, loss mask 0."""
    lib = _lib.load()
    n = len(seqs)
    ids = [np.ascontiguousarray(i, np.uint32) for i, _, _ in seqs]
    tgs = [np.ascontiguousarray(t, np.uint32) for _, t, _ in seqs]
    mks = [np.ascontiguousarray(m, np.uint8) for _, _, m in seqs]
    sizes = lambda arrs: (C.c_size_t * n)(*[a.size for a in arrs])
    ptrs = lambda arrs: (C.c_void_p * n)(*[a.ctypes.data for a in arrs])
    il, tl, ml = sizes(ids), sizes(tgs), sizes(mks)
    padded = C.c_size_t()
    check(lib.ft_chunk_padded_len(il, tl, n, length_bucket, C.byref(padded)))
    S = padded.value
    rows, targets, masks = np.empty((n, S), np.uint32), np.empty((n, S), np.uint32), np.empty((n, S), np.uint8)
    check(lib.ft_pad_chunk(ptrs(ids), ptrs(tgs), ptrs(mks), il, tl, ml, n, S, rows.ctypes.data_as(C.c_void_p),
                           targets.ctypes.data_as(C.c_void_p), masks.ctypes.data_as(C.c_void_p)))
    return rows, targets, masks


def select_sequences(input_ids, target_ids, attention_mask, loss_mask):
    """`Trainer::train_batch`, which rows of a padded `Batch` train (trainer/src/lib.rs:377-395), through
    `ft_train_batch_select`: the valid length of every row, 0 for a row that is dropped."""
    a = [np.ascontiguousarray(x, t) for x, t in ((input_ids, np.uint32), (target_ids, np.uint32),
                                                 (attention_mask, np.uint8), (loss_mask, np.uint8))]
    B, S = a[0].shape
    assert all(x.shape == (B, S) for x in a)
    valid = (C.c_size_t * max(B, 1))()
    kept = C.c_size_t()
    check(_lib.load().ft_train_batch_select(*[x.ctypes.data_as(C.c_void_p) for x in a], B, S, valid, C.byref(kept)))
    out = [valid[b] for b in range(B)]
    assert sum(1 for v in out if v) == kept.value
    return out


def plan_chunks(sequences: int, grad_accum_steps: int, step_in_accum: int = 0):
    """`Trainer::train_batch`, where the chunks end (trainer/src/lib.rs:408-421), through `ft_train_batch_plan`."""
    sizes = (C.c_size_t * max(sequences, 1))()
    n = C.c_size_t()
    check(_lib.load().ft_train_batch_plan(sequences, grad_accum_steps, step_in_accum, sizes, C.byref(n)))
    return [sizes[i] for i in range(n.value)]


class Trainer:
    """`Trainer::new(..).with_grad_accum_steps(..).with_clip_grad_norm(..)` with an AdamW optimizer."""

    def __init__(self, model: Lfm2Model, lr: float, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01,
                 clip_grad_norm: Optional[float] = None, grad_accum_steps: int = 0, length_bucket: int = 32,
                 lr_schedule: str = "constant", warmup_steps: int = 0, total_steps: int = 0, min_lr: float = 0.0):
        """`lr_schedule`: "constant", "cosine" (`CosineAnnealingLR`) or "warmup_cosine"
        (`WarmupCosineScheduler`, what the CLI's train command installs with min_lr = lr / 10,
        ferrotensor-cli/src/main.rs:1686-1695); `lr` is the peak rate."""
        self.model = model
        self.length_bucket = length_bucket
        self.grad_accum_steps = grad_accum_steps
        self._lib = model._lib
        self.hyper = dict(lr=lr, beta1=beta1, beta2=beta2, eps=eps, weight_decay=weight_decay)
        kind = LR_SCHEDULES[lr_schedule]
        self.lr_schedule = lr_schedule
        cfg = _lib.TrainerConfigC(lr, beta1, beta2, eps, weight_decay,
                                  clip_grad_norm if clip_grad_norm else 0.0, grad_accum_steps,
                                  kind, warmup_steps, total_steps, min_lr)
        h = C.c_void_p()
        check(self._lib.ft_trainer_create(model.handle, C.byref(cfg), C.byref(h)))
        self.handle = h
        model._trainers.append(weakref.ref(self))

    def train_chunk(self, rows, targets, masks, apply: bool = True) -> StepStats:
        rows = np.ascontiguousarray(rows, np.uint32)
        targets = np.ascontiguousarray(targets, np.uint32)
        masks = np.ascontiguousarray(masks, np.uint8)
        assert rows.ndim == 2 and rows.shape == targets.shape == masks.shape
        B, S = rows.shape
        st = _lib.StepStatsC()
        per = np.zeros(B, np.float32)
        check(self._lib.ft_trainer_train_chunk(self.handle, rows.ctypes.data_as(C.c_void_p),
                                               targets.ctypes.data_as(C.c_void_p), masks.ctypes.data_as(C.c_void_p),
                                               B, S, 1 if apply else 0, C.byref(st), per.ctypes.data_as(C.c_void_p)))
        return StepStats(loss=st.loss, tokens=st.supervised_tokens, optimizer_step=bool(st.optimizer_step),
                         grad_norm=st.grad_norm, clip_scale=st.clip_scale, per_sequence=per.tolist(),
                         lr=st.lr if st.optimizer_step else None)

    @property
    def optimizer_steps(self) -> int:
        n = C.c_size_t()
        check(self._lib.ft_trainer_optimizer_steps(self.handle, C.byref(n)))
        return n.value

    def set_optimizer_steps(self, steps: int):
        """Resume: restores the step counter, which is also the position of the LR schedule."""
        check(self._lib.ft_trainer_set_optimizer_steps(self.handle, steps))

    @property
    def step_in_accum(self) -> int:
        """Sequences counted into the open accumulation window."""
        n = C.c_size_t()
        check(self._lib.ft_trainer_step_in_accum(self.handle, C.byref(n)))
        return n.value

    def train_batch(self, seqs, apply: bool = True) -> List[StepStats]:
        """`Trainer::train_batch` (trainer/src/lib.rs:371-423) for ragged sequences
        [(input_ids, target_ids, loss_mask)]: those without a supervised token or shorter
        than 2 tokens are dropped; the rest go through `train_chunk` in chunks that end at
        the accumulation boundary, so the optimizer steps after the same sequence as when
        they are trained one at a time. One StepStats per chunk; none when nothing is left."""
        kept = [(i, t, m) for i, t, m in seqs if min(len(i), len(t)) >= 2 and any(m[:min(len(i), len(t))])]
        out = []
        for room in plan_chunks(len(kept), self.grad_accum_steps, self.step_in_accum):
            chunk, kept = kept[:room], kept[room:]
            rows, targets, masks = pad_chunk(chunk, self.length_bucket)
            out.append(self.train_chunk(rows, targets, masks, apply))
        return out

    def train_padded_batch(self, input_ids, target_ids, attention_mask, loss_mask, apply: bool = True) -> List[StepStats]:
        """`Trainer::train_batch` on a `Batch` as the data loader hands it over (trainer/src/lib.rs:371-423):
        [batch, padded_len] ids, targets, attention mask and loss mask. Rows are cut at their attention mask,
        rows that cannot train are dropped (`ft_train_batch_select`), the rest run as `train_batch`."""
        valid = select_sequences(input_ids, target_ids, attention_mask, loss_mask)
        seqs = [(np.asarray(input_ids[b])[:n], np.asarray(target_ids[b])[:n], np.asarray(loss_mask[b])[:n])
                for b, n in enumerate(valid) if n]
        return self.train_batch(seqs, apply)

    def close(self):
        if self.handle is not None and self.handle.value:
            self._lib.ft_trainer_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
