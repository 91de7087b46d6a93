"""Readers for the reference's gradient-parity fixture (data copied from
ferrotensor-graph/tests/fixtures/gradient_parity of the reference)."""
import json
import os

import numpy as np
from safetensors.numpy import load_file

from oracle import reference_step as rs

ATOL = 1e-4   # ferrotensor-trainer/tests/gradient_parity.rs:48
RTOL = 1e-3   # ferrotensor-trainer/tests/gradient_parity.rs:49

LORA_EVERYWHERE = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj", "lm_head"]


class GradientParityFixture:
    def __init__(self, golden_dir):
        d = os.path.join(golden_dir, "gradient_parity")
        self.dir = d
        with open(os.path.join(d, "config.json")) as f:
            self.config_json = json.load(f)
        with open(os.path.join(d, "cases.json")) as f:
            self.meta = json.load(f)
        self.model = load_file(os.path.join(d, "model.safetensors"))
        self.adapters = load_file(os.path.join(d, "adapters.safetensors"))
        self.expected = load_file(os.path.join(d, "expected.safetensors"))

    @property
    def config(self):
        c = self.config_json
        return rs.ModelConfig(
            vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
            intermediate_size=c["intermediate_size"], num_hidden_layers=c["num_hidden_layers"],
            num_attention_heads=c["num_attention_heads"], num_key_value_heads=c["num_key_value_heads"],
            rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"],
            tie_word_embeddings=c["tie_word_embeddings"])

    def oracle_model(self):
        m = rs.Model.from_hf_tensors(self.config, self.model)
        for name, _ in m.named_linears():
            m.set_lora(name, self.adapters[name + ".lora_a"], self.adapters[name + ".lora_b"],
                       self.meta["lora_alpha"])
        return m

    def case(self, name):
        c = self.meta["cases"][name]
        return (np.array(c["rows"], np.uint32), np.array(c["targets"], np.uint32),
                np.array(c["masks"], np.uint8), bool(c["trainable_base"]), np.float32(c["loss"]))

    def expected_grads(self, case):
        pre = f"grad.{case}."
        return {k[len(pre):]: v for k, v in self.expected.items() if k.startswith(pre)}


def worst_ratio(actual, expected, atol=ATOL, rtol=RTOL):
    """max |a-e| / (atol + rtol*|e|): passes at <= 1 (the torch.allclose rule
    of gradient_parity.rs:36-49)."""
    a = np.asarray(actual, np.float64).reshape(-1)
    e = np.asarray(expected, np.float64).reshape(-1)
    assert a.shape == e.shape, (a.shape, e.shape)
    err = np.abs(a - e)
    if not np.all(np.isfinite(err)):
        return float("inf")
    return float(np.max(err / (atol + rtol * np.abs(e)))) if a.size else 0.0
