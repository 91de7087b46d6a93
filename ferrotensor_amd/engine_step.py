"""The LoRA training step composed ONLY of the 1:1 `ComputeEngine` entry points, in the order
`ferrotensor-autograd`'s tape issues them: what the reference's own graph, trainer and optimizer would run
on the HIP library if `ferrotensor_backend`'s types were re-exported from it and nothing else changed.

Per linear `Linear::project_2d` (ferrotensor-graph/src/lib.rs:112-142): matmul_f16b, matmul (x@A), copy +
gradient_scale (`Tensor::scale`, autograd/src/lib.rs:1046-1055), matmul (.@B), add. Block and model as
lfm.rs:116-139, 597-623; RoPE is copy + in-place rotation (autograd:1122-1139); loss and its backward as
trainer/src/lib.rs:548-572, 676-752 (row losses read back; the logits gradient copied, then scaled by
1/accum); `MatMulNode::backward` (autograd:262-290: dX for every operand that needs a gradient, dW only
for trainable ones), `accumulate_grad` (first gradient aliased, later ones summed with `add`, :206-218);
`global_grad_norm` with one `sum_squares_partial` per tensor and a host f64 finish (trainer:507-534);
`clip_grad_by_norm` per tensor (:336-343); `adamw_update` per tensor (autograd:1522-1552).

It exists to be measured next to the fused step driver (`bench.py --path engine-ops`) and is checked
against it in the GPU tests; the product's training path is `ferrotensor_amd.trainer`.
"""
import math
from typing import Dict, List, Optional

import numpy as np

from .engine import AdamParams, AttentionOptions, ComputeEngine, HipContext, UnifiedTensor

SKIP = 0xFFFFFFFF  # MASKED_CE_SKIP (engine/training.rs:7)
LINEARS = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")


class _Lora:
    def __init__(self, ctx, a, b, alpha):
        self.rank = a.shape[1]
        self.scale = float(alpha) / self.rank
        self.a = UnifiedTensor.new(ctx, a, list(a.shape))
        self.b = UnifiedTensor.new(ctx, b, list(b.shape))
        self.ga: Optional[UnifiedTensor] = None
        self.gb: Optional[UnifiedTensor] = None


class _Linear:
    """Frozen base weight [in, out] (f16 storage) + optional adapter."""

    def __init__(self, ctx, w_out_in: np.ndarray, f16: bool):
        w = np.ascontiguousarray(w_out_in.T)
        self.dims = w.shape
        self.f16 = f16
        self.w = UnifiedTensor.from_f32_as_f16(ctx, w, list(w.shape)) if f16 else UnifiedTensor.new(ctx, w, list(w.shape))
        self.lora: Optional[_Lora] = None


class EngineOpsModel:
    """Weights of a Llama-style model as plain engine tensors (Hugging Face names in, builder rules applied:
    linears transposed to [in, out] and rounded to f16, tied head = transposed embedding)."""

    def __init__(self, ctx: HipContext, cfg, tensors: Dict[str, np.ndarray]):
        self.ctx, self.cfg, self.eng = ctx, cfg, ComputeEngine(ctx)
        f16 = bool(cfg.f16_linears)
        self.embed = UnifiedTensor.new(ctx, tensors["model.embed_tokens.weight"], list(tensors["model.embed_tokens.weight"].shape))
        self.norm_f = UnifiedTensor.new(ctx, tensors["model.norm.weight"], [cfg.hidden_size])
        head = tensors.get("lm_head.weight", tensors["model.embed_tokens.weight"])
        self.head = _Linear(ctx, head, f16)
        self.layers: List[dict] = []
        for l in range(cfg.num_hidden_layers):
            p = "model.layers.%d" % l
            layer = {"norm1": UnifiedTensor.new(ctx, tensors[p + ".input_layernorm.weight"], [cfg.hidden_size]),
                     "norm2": UnifiedTensor.new(ctx, tensors[p + ".post_attention_layernorm.weight"], [cfg.hidden_size])}
            for name in LINEARS:
                group = "self_attn" if name in LINEARS[:4] else "mlp"
                layer[name] = _Linear(ctx, tensors["%s.%s.%s.weight" % (p, group, name)], f16)
            self.layers.append(layer)

    def set_lora(self, layer: int, name: str, a: np.ndarray, b: np.ndarray, alpha: float):
        self.layers[layer][name].lora = _Lora(self.ctx, a, b, alpha)

    def loras(self) -> List[_Lora]:
        return [lin.lora for layer in self.layers for name in LINEARS for lin in [layer[name]] if lin.lora]


class EngineOpsTrainer:
    """`Trainer` + `AdamW` over the engine entry points: one optimizer step per `train_chunk` call."""

    def __init__(self, model: EngineOpsModel, lr=2e-4, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01,
                 clip_grad_norm: Optional[float] = None):
        self.m, self.clip = model, clip_grad_norm
        self.hyper = dict(lr=lr, beta1=beta1, beta2=beta2, eps=eps, weight_decay=weight_decay)
        self.t = 0
        self.moments: Dict[int, tuple] = {}
        self.calls = 0  # engine entry points issued by the last step

    # -- helpers: every engine call goes through _e so the step's call count can be reported --
    def _e(self):
        self.calls += 1
        return self.m.eng

    def _empty(self, *shape):
        return UnifiedTensor.empty(self.m.ctx, list(shape))

    def _matmul(self, a, lin_or_b, out_cols, f16):
        out = self._empty(a.shape[0], out_cols)
        (self._e().matmul_f16b if f16 else self._e().matmul)(self.m.ctx, a, lin_or_b, out)
        return out

    def _matmul_bt(self, g, b, out_cols, f16):
        out = self._empty(g.shape[0], out_cols)
        (self._e().matmul_bt_f16b if f16 else self._e().matmul_bt)(self.m.ctx, g, b, out)
        return out

    def _add(self, a, b):
        out = self._empty(*a.shape)
        self._e().add(self.m.ctx, a, b, out)
        return out

    def _scaled_copy(self, t, s):
        """`Tensor::scale` / `ScaleNode`: copy, then gradient_scale (skipped when the factor is exactly 1)."""
        if abs(s - 1.0) <= np.finfo(np.float32).eps:
            return t
        out = self._empty(*t.shape)
        self._e().copy_tensor(self.m.ctx, t, out)
        self._e().gradient_scale(self.m.ctx, out, s)
        return out

    def _accum(self, cur, g):
        """`accumulate_grad`: the first gradient is aliased, later ones are summed into a new buffer."""
        return g if cur is None else self._add(cur, g)

    def _linear_fwd(self, lin: _Linear, x):
        i, o = lin.dims
        y = self._matmul(x, lin.w, o, lin.f16)
        saved = {"x": x}
        if lin.lora:
            t = self._matmul(x, lin.lora.a, lin.lora.rank, False)
            ts = self._scaled_copy(t, lin.lora.scale)
            u = self._matmul(ts, lin.lora.b, o, False)
            y = self._add(y, u)
            saved["ts"] = ts
        return y, saved

    def _linear_bwd(self, lin: _Linear, saved, g, need_dx: bool):
        """Gradient of `project_2d`; returns dX (or None). Adapter gradients accumulate on the adapter."""
        i, o = lin.dims
        dx = None
        if lin.lora:
            lo = lin.lora
            # AddNode hands g to both summands. u = ts @ B: d_ts = g @ B^T, dB = ts^T @ g
            d_ts = self._matmul_bt(g, lo.b, lo.rank, False)
            gb = self._empty(lo.rank, o)
            self._e().matmul_at(self.m.ctx, saved["ts"], g, gb)
            lo.gb = self._accum(lo.gb, gb)
            d_t = self._scaled_copy(d_ts, lo.scale)
            # t = x @ A: dA = x^T @ d_t; dX only when x needs a gradient
            ga = self._empty(i, lo.rank)
            self._e().matmul_at(self.m.ctx, saved["x"], d_t, ga)
            lo.ga = self._accum(lo.ga, ga)
            if need_dx:
                dx = self._matmul_bt(d_t, lo.a, i, False)
        if need_dx:
            dx = self._accum(dx, self._matmul_bt(g, lin.w, i, lin.f16))
        return dx

    def train_chunk(self, rows, targets, masks):
        """Forward, loss, backward, gradient norm, clip, AdamW for B equally long rows. Returns
        (loss, grad_norm, clip_scale or None)."""
        m, cfg, ctx = self.m, self.m.cfg, self.m.ctx
        self.calls = 0
        rows = np.ascontiguousarray(rows, np.uint32)
        B, S = rows.shape
        T, H = B * S, cfg.hidden_size
        heads, kv = cfg.num_attention_heads, cfg.num_key_value_heads
        D = H // heads
        opts = AttentionOptions(causal=True)
        for lo in m.loras():
            lo.ga = lo.gb = None

        # ---- forward ----
        ids = UnifiedTensor.from_bytes(ctx, rows.tobytes(), [T])
        x = self._empty(T, H)
        self._e().embedding(ctx, m.embed, ids, x)       # the reference gathers on the host and uploads
        tape = []
        for layer in m.layers:
            rec = {"x": x}
            n1 = self._empty(T, H)
            self._e().rms_norm_eps(ctx, x, layer["norm1"], n1, cfg.rms_norm_eps)
            q, rec["q_lin"] = self._linear_fwd(layer["q_proj"], n1)
            k, rec["k_lin"] = self._linear_fwd(layer["k_proj"], n1)
            v, rec["v_lin"] = self._linear_fwd(layer["v_proj"], n1)
            qr, kr = self._empty(B, S, heads * D), self._empty(B, S, kv * D)
            self._e().copy_tensor(ctx, q, qr)            # RoPE: copy, then rotate in place
            self._e().rope_theta(ctx, qr, D, 0, cfg.rope_theta)
            self._e().copy_tensor(ctx, k, kr)
            self._e().rope_theta(ctx, kr, D, 0, cfg.rope_theta)
            q4, k4, v4 = qr.reshaped([B, S, heads, D]), kr.reshaped([B, S, kv, D]), v.reshaped([B, S, kv, D])
            att, stats = self._empty(B, S, heads, D), self._empty(B, heads, S, 2)
            self._e().flash_attention_v2_with_stats(ctx, q4, k4, v4, att, stats, opts)
            o, rec["o_lin"] = self._linear_fwd(layer["o_proj"], att.reshaped([T, heads * D]))
            h = self._add(x, o)
            n2 = self._empty(T, H)
            self._e().rms_norm_eps(ctx, h, layer["norm2"], n2, cfg.rms_norm_eps)
            up, rec["up_lin"] = self._linear_fwd(layer["up_proj"], n2)
            gate, rec["gate_lin"] = self._linear_fwd(layer["gate_proj"], n2)
            act = self._empty(T, cfg.intermediate_size)
            self._e().silu_gate_fused(ctx, gate, up, act)       # silu(first) * second
            down, rec["down_lin"] = self._linear_fwd(layer["down_proj"], act)
            rec.update(q4=q4, k4=k4, v4=v4, att=att, stats=stats, h=h, up=up, gate=gate)
            x = self._add(h, down)
            tape.append(rec)
        nf = self._empty(T, H)
        self._e().rms_norm_eps(ctx, x, m.norm_f, nf, cfg.rms_norm_eps)
        logits = self._matmul(nf, m.head.w, cfg.vocab_size, m.head.f16)

        # ---- loss: host builds targets and per-row weights, device does the rest ----
        tg = np.where((np.asarray(masks) != 0) & (np.asarray(targets) < cfg.vocab_size), targets, SKIP).astype(np.uint32)
        counts = (tg != SKIP).sum(axis=1)
        weights = np.where(tg != SKIP, 1.0 / np.maximum(counts, 1)[:, None], 0.0).astype(np.float32)
        t_dev = UnifiedTensor.from_bytes(ctx, tg.tobytes(), [T])
        w_dev = UnifiedTensor.new(ctx, weights.reshape(-1), [T])
        grad_logits, row_loss = self._empty(T, cfg.vocab_size), self._empty(T)
        self._e().masked_cross_entropy_weighted(ctx, logits, t_dev, w_dev, grad_logits, row_loss)
        per_row = row_loss.to_numpy().astype(np.float64).reshape(B, S)       # readback, as the reference does
        loss = float(sum(per_row[b].sum() / max(int(counts[b]), 1) for b in range(B)))

        # ---- backward (seed 1/B: the chunk is the accumulation window) ----
        g = self._empty(T, cfg.vocab_size)
        self._e().copy_tensor(ctx, grad_logits, g)
        if B != 1:
            self._e().gradient_scale(ctx, g, 1.0 / B)
        g = self._matmul_bt(g, m.head.w, H, m.head.f16)
        gx, gw = self._empty(T, H), self._empty(H)
        self._e().rms_norm_backward(ctx, x, m.norm_f, g, gx, gw, cfg.rms_norm_eps)
        g = gx
        for li in range(len(m.layers) - 1, -1, -1):
            layer, rec = m.layers[li], tape[li]
            need_in = li > 0                      # the embedding output needs no gradient
            d_act = self._linear_bwd(layer["down_proj"], rec["down_lin"], g, True)
            d_up, d_gate = self._empty(T, cfg.intermediate_size), self._empty(T, cfg.intermediate_size)
            self._e().silu_gate_backward(ctx, rec["gate"], rec["up"], d_act, d_gate, d_up)
            d_n2 = self._linear_bwd(layer["gate_proj"], rec["gate_lin"], d_gate, True)
            d_n2 = self._accum(d_n2, self._linear_bwd(layer["up_proj"], rec["up_lin"], d_up, True))
            gh, gw = self._empty(T, H), self._empty(H)
            self._e().rms_norm_backward(ctx, rec["h"], layer["norm2"], d_n2, gh, gw, cfg.rms_norm_eps)
            g_h = self._add(g, gh)
            d_att = self._linear_bwd(layer["o_proj"], rec["o_lin"], g_h, True)
            dq, dk, dv = self._empty(B, S, heads, D), self._empty(B, S, kv, D), self._empty(B, S, kv, D)
            self._e().flash_attention_v2_backward_with_stats(ctx, rec["q4"], rec["k4"], rec["v4"], rec["att"],
                                                           d_att.reshaped([B, S, heads, D]), dq, dk, dv, rec["stats"], opts)
            dq_r, dk_r = self._empty(B, S, heads * D), self._empty(B, S, kv * D)
            self._e().copy_tensor(ctx, dq.reshaped([B, S, heads * D]), dq_r)  # RoPENode: copy, inverse rotation
            self._e().rope_theta_inverse(ctx, dq_r, D, 0, cfg.rope_theta)
            self._e().copy_tensor(ctx, dk.reshaped([B, S, kv * D]), dk_r)
            self._e().rope_theta_inverse(ctx, dk_r, D, 0, cfg.rope_theta)
            d_n1 = self._linear_bwd(layer["v_proj"], rec["v_lin"], dv.reshaped([T, kv * D]), need_in)
            d_k = self._linear_bwd(layer["k_proj"], rec["k_lin"], dk_r.reshaped([T, kv * D]), need_in)
            d_q = self._linear_bwd(layer["q_proj"], rec["q_lin"], dq_r.reshaped([T, heads * D]), need_in)
            if need_in:
                d_n1 = self._accum(self._accum(d_n1, d_k), d_q)
                gx, gw = self._empty(T, H), self._empty(H)
                self._e().rms_norm_backward(ctx, rec["x"], layer["norm1"], d_n1, gx, gw, cfg.rms_norm_eps)
                g = self._add(g_h, gx)

        # ---- global norm, clip, AdamW: one call per tensor each ----
        params = [(lo.a, lo.ga) for lo in m.loras()] + [(lo.b, lo.gb) for lo in m.loras()]
        chunks = sum((p.numel() + 4095) // 4096 for p, _ in params)
        partial = self._empty(chunks)
        off = 0
        for _, gr in params:
            off += self._e().sum_squares_partial(ctx, gr, partial, off)
        norm = math.sqrt(float(partial.to_numpy().astype(np.float64).sum()))
        clip_scale = None
        if not math.isfinite(norm):
            return loss, norm, clip_scale
        if self.clip and norm > self.clip:
            clip_scale = self.clip / (norm + 1e-6)
            for _, gr in params:
                self._e().clip_grad_by_norm(ctx, gr, clip_scale)
        self.t += 1
        adam = AdamParams(t=float(self.t), **self.hyper)
        for i, (p, gr) in enumerate(params):
            if i not in self.moments:
                self.moments[i] = (UnifiedTensor.zeros(ctx, list(p.shape)), UnifiedTensor.zeros(ctx, list(p.shape)))
            mm, vv = self.moments[i]
            self._e().adamw_update(ctx, p, gr, mm, vv, adam)
        return loss, norm, clip_scale
