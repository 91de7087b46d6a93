"""CPU restatement of the reference's LoRA training step. Test infrastructure only.

Restates, op for op and in the reference's order, what one optimizer step of
`ferrotensor train` does on a Llama-style model:

* model forward: `Lfm2Model::forward_batch_with_dropout`
  (ferrotensor-graph/src/lfm.rs:597-623), `Lfm2Block::forward_with_dropout`
  (lfm.rs:116-139), `Attention::forward_with_dropout`
  (ferrotensor-graph/src/lib.rs:367-414), `MLP::forward` (lib.rs:504-510),
  `Linear::project_2d` with its LoRA adapter (lib.rs:112-142), host embedding
  gather (ferrotensor-autograd/src/lib.rs:1159-1179);
* loss: `masked_cross_entropy_batch` (ferrotensor-trainer/src/lib.rs:676-752);
* backward: the node rules of ferrotensor-autograd/src/lib.rs (MatMulNode
  :262-290, AddNode :293-310, ScaleNode :340-357, RoPENode :509-533,
  RMSNormNode :575-595, SiLUGateNode :731-749, FlashAttentionNode :1328-1390,
  MaskedCrossEntropyNode trainer/src/lib.rs:548-572);
* step: `Trainer::train_chunk` / `apply_gradients` / `global_grad_norm`
  (trainer/src/lib.rs:296-360, 426-534) and `AdamW::apply_step`
  (autograd/src/lib.rs:1522-1552).

The arithmetic itself is in oracle/kernels.cpp (through oracle.cpu). There is
no autograd tape: the step's graph is static, so backward is written out.
Attention dropout is 0 in every SmolLM2 config and is not restated.

Pinned by tests/test_oracle_fixture.py against the reference's own
PyTorch-autograd fixture (loss, logits, every LoRA / base / norm gradient).
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import cpu

MASKED_CE_SKIP = 0xFFFFFFFF  # ferrotensor-backend/src/engine/training.rs:7
SUM_SQUARES_CHUNK = 4096     # ferrotensor-backend/src/engine/training.rs (sum_squares_partial)
F32_EPSILON = float(np.finfo(np.float32).eps)

ATTN_LINEARS = ("q_proj", "k_proj", "v_proj", "o_proj")
MLP_LINEARS = ("gate_proj", "up_proj", "down_proj")


@dataclass
class ModelConfig:
    """The fields of `Lfm2Config` the step uses (ferrotensor-loader/src/lib.rs:74-142)."""
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False

    @property
    def head_dim(self):
        return self.hidden_size // self.num_attention_heads


@dataclass
class Linear:
    """`Linear` (graph/src/lib.rs:100-110): weight is [in, out]."""
    weight: np.ndarray
    lora_a: Optional[np.ndarray] = None  # [in, rank]
    lora_b: Optional[np.ndarray] = None  # [rank, out]
    alpha: float = 0.0
    rank: int = 0
    bias: Optional[np.ndarray] = None    # [out] (Qwen2 query, key and value projections)

    @property
    def scale(self):
        return np.float32(self.alpha) / np.float32(self.rank)

    def forward(self, x2d, cache):
        """`Linear::project_2d` (graph/src/lib.rs:112-126)."""
        out = cpu.matmul(x2d, self.weight)
        if self.lora_a is not None:
            temp = cpu.matmul(x2d, self.lora_a)
            s = self.scale
            if abs(float(s) - 1.0) > F32_EPSILON:
                temp = cpu.scale(temp, float(s))
            cache["temp"] = temp
            out = cpu.add(out, cpu.matmul(temp, self.lora_b))
        if self.bias is not None:
            # graph/src/lib.rs:128-139: out + ones[rows, 1] @ bias[1, out], i.e. the bias on every row
            ones = np.ones((x2d.shape[0], 1), np.float32)
            out = cpu.add(out, cpu.matmul(ones, self.bias.reshape(1, -1)))
        cache["x"] = x2d
        return out

    def backward(self, g, cache, need_dx, trainable_base, grads, name):
        """MatMulNode / ScaleNode / AddNode rules for the graph above."""
        x = cache["x"]
        dx = None
        if self.bias is not None and trainable_base:
            # backward of ones @ bias_row: ones^T @ g, the output gradient summed over the rows
            ones = np.ones((g.shape[0], 1), np.float32)
            _acc(grads, name + ".bias", cpu.matmul_at(ones, g).reshape(-1))
        if self.lora_a is not None:
            temp = cache["temp"]
            d_temp = cpu.matmul_bt(g, self.lora_b)          # [M, r]
            _acc(grads, name + ".lora_b", cpu.matmul_at(temp, g))
            s = self.scale
            if abs(float(s) - 1.0) > F32_EPSILON:
                d_temp = cpu.scale(d_temp, float(s))
            _acc(grads, name + ".lora_a", cpu.matmul_at(x, d_temp))
            if need_dx:
                dx = cpu.matmul_bt(d_temp, self.lora_a)
        if trainable_base:
            _acc(grads, name + ".weight", cpu.matmul_at(x, g))
        if need_dx:
            dxb = cpu.matmul_bt(g, self.weight)
            dx = dxb if dx is None else cpu.add(dxb, dx)
        return dx


def _acc(grads, name, value):
    """`accumulate_grad` (autograd/src/lib.rs:206-218): first gradient kept, later ones added."""
    if name in grads:
        grads[name] = cpu.add(grads[name], value)
    else:
        grads[name] = value


@dataclass
class Block:
    norm1: np.ndarray
    norm2: np.ndarray
    linears: Dict[str, Linear]


@dataclass
class Model:
    config: ModelConfig
    embed: np.ndarray            # [vocab, hidden]
    blocks: List[Block]
    norm_f: np.ndarray
    lm_head: Linear              # weight [hidden, vocab]

    # ---- construction -------------------------------------------------
    @staticmethod
    def from_hf_tensors(config: ModelConfig, tensors: Dict[str, np.ndarray], f16_linears=False):
        """Builder rules of ferrotensor-graph/src/model_builder.rs:400-424, 653-689:
        HF `[out, in]` weights are transposed to `[in, out]`; with f16 storage
        the values are rounded to f16; a tied head is the transposed embedding."""
        def lin(key):
            w = cpu.transpose(tensors[key])
            if f16_linears:
                w = cpu.round_f16(w)
            # build_linear (model_builder.rs:454-469): `<prefix>.bias` [out] when the checkpoint has it, kept f32
            bias = tensors.get(key[:-len(".weight")] + ".bias")
            return Linear(weight=w, bias=None if bias is None else np.ascontiguousarray(bias, np.float32))

        blocks = []
        for l in range(config.num_hidden_layers):
            p = f"model.layers.{l}"
            ls = {n: lin(f"{p}.self_attn.{n}.weight") for n in ATTN_LINEARS}
            ls.update({n: lin(f"{p}.mlp.{n}.weight") for n in MLP_LINEARS})
            blocks.append(Block(norm1=np.asarray(tensors[f"{p}.input_layernorm.weight"], np.float32),
                                norm2=np.asarray(tensors[f"{p}.post_attention_layernorm.weight"], np.float32),
                                linears=ls))
        embed = np.ascontiguousarray(tensors["model.embed_tokens.weight"], np.float32)
        if config.tie_word_embeddings or "lm_head.weight" not in tensors:
            head_w = cpu.transpose(embed)
            if f16_linears:
                head_w = cpu.round_f16(head_w)
            head = Linear(weight=head_w)
        else:
            head = lin("lm_head.weight")
        return Model(config, embed, blocks, np.asarray(tensors["model.norm.weight"], np.float32), head)

    def named_linears(self) -> List[Tuple[str, Linear]]:
        out = []
        for l, b in enumerate(self.blocks):
            for n in ATTN_LINEARS:
                out.append((f"model.layers.{l}.self_attn.{n}", b.linears[n]))
            for n in MLP_LINEARS:
                out.append((f"model.layers.{l}.mlp.{n}", b.linears[n]))
        out.append(("lm_head", self.lm_head))
        return out

    def set_lora(self, name, a, b, alpha):
        lin = dict(self.named_linears())[name]
        lin.lora_a = np.ascontiguousarray(a, np.float32)
        lin.lora_b = np.ascontiguousarray(b, np.float32)
        lin.rank = lin.lora_a.shape[1]
        lin.alpha = float(alpha)

    def lora_params(self) -> List[Tuple[str, np.ndarray]]:
        out = []
        for name, lin in self.named_linears():
            if lin.lora_a is not None:
                out.append((name + ".lora_a", lin.lora_a))
                out.append((name + ".lora_b", lin.lora_b))
        return out

    # ---- forward ------------------------------------------------------
    def forward(self, rows: np.ndarray, trainable_base=False):
        """rows: [B, S] uint32 -> (logits [B, S, V], cache)."""
        c = self.config
        rows = np.ascontiguousarray(rows, np.uint32)
        B, S = rows.shape
        T = B * S
        H, D = c.hidden_size, c.head_dim
        nh, nkv = c.num_attention_heads, c.num_key_value_heads
        x = cpu.embedding(self.embed, rows).reshape(T, H)
        cache = {"B": B, "S": S, "layers": [], "trainable_base": trainable_base}
        x_req = False  # embedding output is a frozen constant
        for blk in self.blocks:
            lc = {"x": x, "x_req": x_req}
            h1 = cpu.rms_norm(x, blk.norm1, c.rms_norm_eps)
            h1_req = x_req or trainable_base
            lc["h1_req"] = h1_req
            for n in ("q_proj", "k_proj", "v_proj"):
                lc[n] = {}
            q = blk.linears["q_proj"].forward(h1, lc["q_proj"])
            k = blk.linears["k_proj"].forward(h1, lc["k_proj"])
            v = blk.linears["v_proj"].forward(h1, lc["v_proj"])
            q = cpu.rope(q.reshape(B, S, nh * D), D, 0, c.rope_theta)
            k = cpu.rope(k.reshape(B, S, nkv * D), D, 0, c.rope_theta)
            q4 = q.reshape(B, S, nh, D)
            k4 = k.reshape(B, S, nkv, D)
            v4 = v.reshape(B, S, nkv, D)
            o4, _ = cpu.attention(q4, k4, v4, causal=True)
            lc.update(q4=q4, k4=k4, v4=v4, o4=o4)
            lc["o_proj"] = {}
            a = blk.linears["o_proj"].forward(o4.reshape(T, nh * D), lc["o_proj"])
            h = cpu.add(x, a)
            lc["h"] = h
            h2 = cpu.rms_norm(h, blk.norm2, c.rms_norm_eps)
            for n in MLP_LINEARS:
                lc[n] = {}
            up = blk.linears["up_proj"].forward(h2, lc["up_proj"])
            gate = blk.linears["gate_proj"].forward(h2, lc["gate_proj"])
            act = cpu.silu_gate(gate, up)
            lc.update(gate=gate, up=up)
            m = blk.linears["down_proj"].forward(act, lc["down_proj"])
            x = cpu.add(h, m)
            x_req = True  # every block holds trainable LoRA factors in these configs
            cache["layers"].append(lc)
        cache["x_final"] = x
        hf = cpu.rms_norm(x, self.norm_f, c.rms_norm_eps)
        cache["lm_head"] = {}
        logits = self.lm_head.forward(hf, cache["lm_head"])
        return logits.reshape(B, S, c.vocab_size), cache

    # ---- backward -----------------------------------------------------
    def backward(self, d_logits: np.ndarray, cache) -> Dict[str, np.ndarray]:
        """Gradients of every trainable tensor, by fixture name
        (`<prefix>.lora_a`, `<prefix>.lora_b`, and with a trainable base
        `<prefix>.weight` [in, out] and the norm scales)."""
        c = self.config
        B, S = cache["B"], cache["S"]
        T = B * S
        D = c.head_dim
        nh, nkv = c.num_attention_heads, c.num_key_value_heads
        tb = cache["trainable_base"]
        grads: Dict[str, np.ndarray] = {}
        g = np.ascontiguousarray(d_logits, np.float32).reshape(T, c.vocab_size)
        g = self.lm_head.backward(g, cache["lm_head"], True, tb, grads, "lm_head")
        gx, gw = cpu.rms_norm_backward(cache["x_final"], self.norm_f, g, c.rms_norm_eps)
        if tb:
            grads["model.norm.weight"] = gw
        g = gx
        for l in reversed(range(len(self.blocks))):
            blk, lc = self.blocks[l], cache["layers"][l]
            p = f"model.layers.{l}"
            # out = h + mlp(norm2(h)): AddNode sends g to both.
            d_act = blk.linears["down_proj"].backward(g, lc["down_proj"], True, tb, grads, f"{p}.mlp.down_proj")
            d_gate, d_up = cpu.silu_gate_backward(lc["gate"], lc["up"], d_act)
            d_h2 = blk.linears["up_proj"].backward(d_up, lc["up_proj"], True, tb, grads, f"{p}.mlp.up_proj")
            d_h2 = cpu.add(d_h2, blk.linears["gate_proj"].backward(d_gate, lc["gate_proj"], True, tb, grads,
                                                                  f"{p}.mlp.gate_proj"))
            gx, gw = cpu.rms_norm_backward(lc["h"], blk.norm2, d_h2, c.rms_norm_eps)
            if tb:
                grads[f"{p}.post_attention_layernorm.weight"] = gw
            g_h = cpu.add(g, gx)
            # h = x + o_proj(attn)
            d_o = blk.linears["o_proj"].backward(g_h, lc["o_proj"], True, tb, grads, f"{p}.self_attn.o_proj")
            dq4, dk4, dv4 = cpu.attention_backward(lc["q4"], lc["k4"], lc["v4"], lc["o4"],
                                                   d_o.reshape(B, S, nh, D), causal=True)
            dq = cpu.rope(dq4.reshape(B, S, nh * D), D, 0, c.rope_theta, inverse=True).reshape(T, nh * D)
            dk = cpu.rope(dk4.reshape(B, S, nkv * D), D, 0, c.rope_theta, inverse=True).reshape(T, nkv * D)
            dv = dv4.reshape(T, nkv * D)
            need = lc["h1_req"]
            d_h1 = blk.linears["q_proj"].backward(dq, lc["q_proj"], need, tb, grads, f"{p}.self_attn.q_proj")
            t = blk.linears["k_proj"].backward(dk, lc["k_proj"], need, tb, grads, f"{p}.self_attn.k_proj")
            if need:
                d_h1 = cpu.add(d_h1, t)
            t = blk.linears["v_proj"].backward(dv, lc["v_proj"], need, tb, grads, f"{p}.self_attn.v_proj")
            if need:
                d_h1 = cpu.add(d_h1, t)
            if need:
                gx, gw = cpu.rms_norm_backward(lc["x"], blk.norm1, d_h1, c.rms_norm_eps)
                if tb:
                    grads[f"{p}.input_layernorm.weight"] = gw
                g = cpu.add(g_h, gx)
            else:
                g = g_h
            if not lc["x_req"]:
                break  # the embedding output is frozen: nothing upstream needs g
        return grads


# ---------------------------------------------------------------------------
# Loss (trainer/src/lib.rs:676-752)
# ---------------------------------------------------------------------------

def build_targets_and_weights(target_ids, loss_mask, sequences, vocab):
    """Host half of `masked_cross_entropy_batch`: per-row target (or
    MASKED_CE_SKIP) and weight 1 / supervised-tokens-of-its-sequence.
    Integer work: compared bit-exactly."""
    target_ids = np.asarray(target_ids, np.uint32).reshape(-1)
    loss_mask = np.asarray(loss_mask, np.uint8).reshape(-1)
    rows = target_ids.size
    assert rows % sequences == 0
    seq_len = rows // sequences
    sup = (loss_mask != 0) & (target_ids.astype(np.uint64) < vocab)
    tokens = sup.reshape(sequences, seq_len).sum(axis=1).astype(np.int64)
    targets = np.where(sup, target_ids, np.uint32(MASKED_CE_SKIP)).astype(np.uint32)
    per_row_tokens = np.repeat(tokens, seq_len)
    weights = np.zeros(rows, np.float32)
    weights[sup] = (np.float32(1.0) / per_row_tokens[sup].astype(np.float32)).astype(np.float32)
    return targets, weights, tokens


def masked_cross_entropy_batch(logits, target_ids, loss_mask, sequences):
    """-> (total loss f32, per_sequence [(mean, tokens)], grad_logits) or None."""
    vocab = logits.shape[-1]
    targets, weights, tokens = build_targets_and_weights(target_ids, loss_mask, sequences, vocab)
    if not (tokens > 0).any():
        return None
    rows = targets.size
    seq_len = rows // sequences
    grad, row_loss = cpu.masked_cross_entropy(logits.reshape(rows, vocab), targets, weights)
    per_sequence = []
    for s in range(sequences):
        total = float(np.sum(row_loss[s * seq_len:(s + 1) * seq_len].astype(np.float64)))
        per_sequence.append((np.float32(total / max(int(tokens[s]), 1)), int(tokens[s])))
    loss = np.float32(0.0)
    for mean, _ in per_sequence:
        loss = np.float32(loss + mean)
    return loss, per_sequence, grad


# ---------------------------------------------------------------------------
# Optimizer step (trainer/src/lib.rs:296-360, 507-534; autograd:1522-1552)
# ---------------------------------------------------------------------------

def global_grad_norm(grads: Sequence[np.ndarray]) -> np.float32:
    chunks = sum((g.size + SUM_SQUARES_CHUNK - 1) // SUM_SQUARES_CHUNK for g in grads)
    if chunks == 0:
        return np.float32(0.0)
    partials = np.empty(chunks, np.float32)
    off = 0
    for g in grads:
        off += cpu.sum_squares_partial(g, partials, off)
    return np.float32(np.sqrt(np.sum(partials.astype(np.float64))))


@dataclass
class AdamW:
    """`AdamW::new` defaults (autograd/src/lib.rs:1502-1515); the CLI passes weight_decay 0."""
    lr: float
    beta1: float = 0.9
    beta2: float = 0.999
    eps: float = 1e-8
    weight_decay: float = 0.01
    t: float = 0.0
    m: Dict[str, np.ndarray] = field(default_factory=dict)
    v: Dict[str, np.ndarray] = field(default_factory=dict)

    def step(self, params: Sequence[Tuple[str, np.ndarray]], grads: Dict[str, np.ndarray]):
        self.t += 1.0
        for name, w in params:
            g = grads.get(name)
            if g is None:
                continue
            if name not in self.m:
                self.m[name] = np.zeros_like(w)
                self.v[name] = np.zeros_like(w)
            cpu.adamw_update(w, g, self.m[name], self.v[name], self.lr, self.beta1, self.beta2,
                             self.eps, self.weight_decay, self.t)


_M64 = (1 << 64) - 1


def lora_seed(layer_seed: int, module_name: str) -> int:
    """`lora_seed` (model_builder.rs:739-759): FNV-1a over the name bytes and the seed's
    little-endian bytes, then the splitmix64 finalizer. Pinned values at model_builder.rs:870-876."""
    h = 0xcbf29ce484222325
    for byte in module_name.encode() + int(layer_seed).to_bytes(8, "little"):
        h ^= byte
        h = (h * 0x00000100000001b3) & _M64
    h ^= h >> 30
    h = (h * 0xbf58476d1ce4e5b9) & _M64
    h ^= h >> 27
    h = (h * 0x94d049bb133111eb) & _M64
    return h ^ (h >> 31)


def lora_init_a(in_dim: int, out_dim: int, rank: int, seed: int) -> np.ndarray:
    """`LoRAAdapter::new_seeded` (graph/src/lib.rs:59-92): A [in, rank] uniform in +-1/sqrt(in)
    from xorshift64* (shifts 12, 25, 27; multiplier 0x2545F4914F6CDD1D; top 24 bits)."""
    bound = np.float32(1.0) / np.sqrt(np.float32(max(in_dim, 1)))
    state = ((seed * 0x9E3779B97F4A7C15 + ((in_dim << 32) | (out_dim << 8) | rank)) & _M64) | 1
    out = np.empty(in_dim * rank, np.float32)
    for i in range(in_dim * rank):
        state ^= state >> 12
        state = (state ^ (state << 25)) & _M64
        state ^= state >> 27
        bits = ((state * 0x2545F4914F6CDD1D) & _M64) >> 40
        unit = np.float32(bits) / np.float32(1 << 24)
        out[i] = (unit * np.float32(2.0) - np.float32(1.0)) * bound
    return out.reshape(in_dim, rank)


@dataclass
class CosineAnnealingLR:
    """`CosineAnnealingLR` (autograd/src/lib.rs:1717-1758), f32 arithmetic."""
    initial_lr: float
    min_lr: float
    total_steps: int
    current: int = 0

    def get_lr(self) -> float:
        if self.current >= self.total_steps:
            return float(np.float32(self.min_lr))
        progress = np.float32(self.current) / np.float32(self.total_steps)
        cosine = (np.float32(1.0) + np.cos(np.float32(np.pi) * progress, dtype=np.float32)) / np.float32(2.0)
        return float(np.float32(self.min_lr) + (np.float32(self.initial_lr) - np.float32(self.min_lr)) * cosine)

    def step(self):
        self.current += 1


@dataclass
class WarmupCosineScheduler:
    """`WarmupCosineScheduler` (autograd/src/lib.rs:1761-1814), f32 arithmetic."""
    peak_lr: float
    min_lr: float
    warmup_steps: int
    total_steps: int
    current: int = 0

    def get_lr(self) -> float:
        peak, low = np.float32(self.peak_lr), np.float32(self.min_lr)
        if self.current < self.warmup_steps:
            return float(peak * (np.float32(self.current) / np.float32(self.warmup_steps)))
        if self.current >= self.total_steps:
            return float(low)
        progress = np.float32(self.current - self.warmup_steps) / np.float32(self.total_steps - self.warmup_steps)
        cosine = (np.float32(1.0) + np.cos(np.float32(np.pi) * progress, dtype=np.float32)) / np.float32(2.0)
        return float(low + (peak - low) * cosine)

    def step(self):
        self.current += 1


@dataclass
class StepStats:
    loss: float
    per_sequence: List[Tuple[float, int]]
    grad_norm: Optional[float]
    optimizer_step: bool
    clip_scale: Optional[float] = None
    lr: Optional[float] = None


def pad_chunk(seqs, length_bucket=32):
    """`train_chunk` padding (trainer/src/lib.rs:431-450): rows right-padded to
    a multiple of `length_bucket` with their last token, mask 0. Integer work."""
    longest = max(min(len(i), len(t)) for i, t, _ in seqs)
    padded = -(-longest // length_bucket) * length_bucket
    rows, targets, masks = [], [], []
    for ids, tg, mk in seqs:
        n = min(len(ids), len(tg))
        pad = ids[n - 1] if n else 0
        rows.append(list(ids[:n]) + [pad] * (padded - n))
        targets.append(list(tg[:n]) + [pad] * (padded - n))
        masks.append([mk[i] if i < len(mk) else 0 for i in range(n)] + [0] * (padded - n))
    return (np.array(rows, np.uint32), np.array(targets, np.uint32), np.array(masks, np.uint8))


def select_sequences(attention_mask, loss_mask):
    """`Trainer::train_batch`, which rows of a `Batch` train (trainer/src/lib.rs:377-395): a row is cut
    where its attention mask first differs from 1 and dropped when fewer than 2 tokens remain or the cut
    loss mask has no non-zero entry. Returns the valid length per row (0 = dropped). Integer work."""
    out = []
    for attn, mask in zip(attention_mask, loss_mask):
        n = 0
        for flag in attn:
            if flag != 1:
                break
            n += 1
        out.append(n if n >= 2 and any(m != 0 for m in mask[:n]) else 0)
    return out


def plan_chunks(sequences: int, grad_accum_steps: int, step_in_accum: int = 0):
    """`Trainer::train_batch`, where the chunks end (trainer/src/lib.rs:408-421 with the counter of
    :486-489): room = max(grad_accum_steps - step_in_accum, 1); the chunk that fills the window resets
    the counter. Integer work."""
    sizes, rest = [], sequences
    while rest > 0:
        room = min(max(grad_accum_steps - step_in_accum, 1), rest)
        sizes.append(room)
        rest -= room
        step_in_accum += room
        if step_in_accum >= grad_accum_steps:
            step_in_accum = 0
    return sizes


def apply_gradients(params, grads, opt: AdamW, stats: "StepStats", clip_grad_norm: Optional[float] = None,
                    scheduler=None):
    """`Trainer::apply_gradients` (trainer/src/lib.rs:296-360): global norm; a non-finite norm
    skips the step (neither the optimizer's t nor the schedule advances, :332-335); when the norm
    exceeds `clip_grad_norm` every gradient is scaled in place by max / (norm + 1e-6), all in f32
    (:336-343, `clip_grad_by_norm`, engine/training.rs:161-169); then the schedule steps and AdamW
    applies. `grads` (name -> array) is updated with the clipped gradients."""
    glist = [grads[n] for n, _ in params if n in grads]
    if not glist:
        return
    norm = global_grad_norm(glist)
    stats.grad_norm = float(norm)
    if not np.isfinite(norm):
        return
    if clip_grad_norm is not None and norm > np.float32(clip_grad_norm):
        s = np.float32(clip_grad_norm) / (norm + np.float32(1e-6))
        stats.clip_scale = float(s)
        for n, _ in params:
            if n in grads:
                grads[n] = cpu.scale(grads[n], float(s))
    if scheduler is not None:   # step k (1-based) uses the schedule's value at k (:345-352)
        scheduler.step()
        opt.lr = scheduler.get_lr()
        stats.lr = opt.lr
    opt.step(params, grads)
    stats.optimizer_step = True


def train_chunk(model: Model, opt: AdamW, rows, targets, masks, grad_accum_steps=None,
                clip_grad_norm: Optional[float] = None, trainable_base=False, return_grads=False, scheduler=None):
    """One forward + backward over equally long rows and one optimizer step
    (`Trainer::train_chunk` with the chunk filling the accumulation window:
    the CLI sets grad_accum_steps = batch * accum, main.rs:1687-1695)."""
    rows = np.asarray(rows, np.uint32)
    B = rows.shape[0]
    if grad_accum_steps is None:
        grad_accum_steps = B
    logits, cache = model.forward(rows, trainable_base=trainable_base)
    res = masked_cross_entropy_batch(logits, targets, masks, B)
    if res is None:
        return None
    loss, per_seq, grad_logits = res
    seed = np.float32(1.0) / np.float32(grad_accum_steps)
    if abs(float(seed) - 1.0) > F32_EPSILON:   # MaskedCrossEntropyNode::backward
        grad_logits = cpu.scale(grad_logits, float(seed))
    grads = model.backward(grad_logits, cache)
    params = model.lora_params()
    stats = StepStats(float(loss), [(float(a), b) for a, b in per_seq], None, False)
    apply_gradients(params, grads, opt, stats, clip_grad_norm=clip_grad_norm, scheduler=scheduler)
    if return_grads:
        return stats, logits, grads
    return stats
