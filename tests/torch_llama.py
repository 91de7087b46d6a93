"""A Llama-style decoder written with torch autograd in float64, independent of the oracle's code.

It is first checked against the reference's own PyTorch fixture (logits, loss and every gradient of
ferrotensor-graph/tests/fixtures/gradient_parity), and then used to pin what that fixture leaves
open: projections with a `<prefix>.bias` tensor (Qwen2), `Linear::project_2d`
(ferrotensor-graph/src/lib.rs:112-141).
"""
import torch
import torch.nn.functional as F


def _rope(x, theta):
    # x [B, S, heads, D]: halves (i, i + D/2) rotated by pos * theta^(-2i/D)
    B, S, _, D = x.shape
    i = torch.arange(D // 2, dtype=torch.float64)
    ang = torch.arange(S, dtype=torch.float64)[:, None] * theta ** (-2.0 * i / D)[None, :]
    c, s = torch.cos(ang)[None, :, None, :], torch.sin(ang)[None, :, None, :]
    a, b = x[..., :D // 2], x[..., D // 2:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def _norm(x, w, eps):
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w


class TorchLlama:
    """Leaves (float64, requires_grad) keyed by the Hugging Face names: `<linear>.weight` [out, in],
    `<linear>.bias` [out], norm scales, and `<linear>.lora_a` [in, r] / `<linear>.lora_b` [r, out]."""

    def __init__(self, config, tensors, adapters=None, lora_alpha=0.0):
        self.c = config
        self.alpha = float(lora_alpha)
        self.p = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in tensors.items()}
        for k, v in (adapters or {}).items():
            self.p[k] = torch.tensor(v, dtype=torch.float64, requires_grad=True)

    def linear(self, prefix, x):
        p = self.p
        y = x @ p[prefix + ".weight"].T
        if prefix + ".lora_a" in p:
            a, b = p[prefix + ".lora_a"], p[prefix + ".lora_b"]
            y = y + (x @ a) @ b * (self.alpha / a.shape[1])
        if prefix + ".bias" in p:
            y = y + p[prefix + ".bias"]
        return y

    def logits(self, rows):
        c, p = self.c, self.p
        B, S = rows.shape
        nh, nkv = c.num_attention_heads, c.num_key_value_heads
        D = c.hidden_size // nh
        x = p["model.embed_tokens.weight"][torch.as_tensor(rows.astype("int64"))]
        mask = torch.full((S, S), float("-inf"), dtype=torch.float64).triu(1)
        for l in range(c.num_hidden_layers):
            pre = f"model.layers.{l}"
            h = _norm(x, p[pre + ".input_layernorm.weight"], c.rms_norm_eps)
            q = _rope(self.linear(pre + ".self_attn.q_proj", h).view(B, S, nh, D), c.rope_theta)
            k = _rope(self.linear(pre + ".self_attn.k_proj", h).view(B, S, nkv, D), c.rope_theta)
            v = self.linear(pre + ".self_attn.v_proj", h).view(B, S, nkv, D)
            k = k.repeat_interleave(nh // nkv, dim=2)
            v = v.repeat_interleave(nh // nkv, dim=2)
            s = torch.einsum("bqhd,bkhd->bhqk", q, k) / D ** 0.5 + mask
            o = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, -1), v).reshape(B, S, nh * D)
            x = x + self.linear(pre + ".self_attn.o_proj", o)
            h = _norm(x, p[pre + ".post_attention_layernorm.weight"], c.rms_norm_eps)
            act = F.silu(self.linear(pre + ".mlp.gate_proj", h)) * self.linear(pre + ".mlp.up_proj", h)
            x = x + self.linear(pre + ".mlp.down_proj", act)
        x = _norm(x, p["model.norm.weight"], c.rms_norm_eps)
        if "lm_head.weight" in p:
            return self.linear("lm_head", x)
        return x @ p["model.embed_tokens.weight"].T

    def loss_and_grads(self, rows, targets, masks):
        """The sum over sequences of each sequence's mean cross-entropy over its supervised tokens
        (`masked_cross_entropy_batch`, ferrotensor-trainer/src/lib.rs:296-360), and d loss / d leaf."""
        for t in self.p.values():
            t.grad = None
        logits = self.logits(rows)
        B, S, V = logits.shape
        sup = torch.as_tensor((masks != 0) & (targets < V))
        ce = F.cross_entropy(logits.reshape(B * S, V), torch.as_tensor(targets.astype("int64") % V).reshape(-1),
                             reduction="none").view(B, S)
        per_seq = (ce * sup).sum(1) / sup.sum(1).clamp(min=1)
        loss = per_seq.sum()
        loss.backward()
        grads = {k: t.grad.numpy() for k, t in self.p.items() if t.grad is not None}
        return logits.detach().numpy(), float(loss.detach()), grads
