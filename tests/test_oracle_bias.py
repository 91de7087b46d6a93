"""Projection biases (`<prefix>.bias`, Qwen2) in the CPU oracle, pinned by torch autograd.

The reference holds no fixture with a bias, so the check is an independent torch model
(tests/torch_llama.py): it must first reproduce the reference's own gradient-parity fixture, and
then agree with the oracle on a model whose projections carry biases.
"""
import numpy as np
import pytest

from oracle import reference_step as rs
from tests.fixture_io import GradientParityFixture, worst_ratio
from tests.torch_llama import TorchLlama


@pytest.fixture(scope="module")
def fx(golden_dir):
    return GradientParityFixture(golden_dir)


def _torch_grads_in_oracle_layout(grads):
    """torch keeps `<linear>.weight` as [out, in]; the oracle (and the fixture) as [in, out]."""
    return {k: (g.T if k.endswith("_proj.weight") or k == "lm_head.weight" else g) for k, g in grads.items()}


@pytest.mark.parametrize("case", ["single", "masked", "full"])
def test_torch_model_reproduces_the_reference_fixture(fx, case):
    rows, targets, masks, trainable_base, want_loss = fx.case(case)
    tm = TorchLlama(fx.config, fx.model, fx.adapters, fx.meta["lora_alpha"])
    logits, loss, grads = tm.loss_and_grads(rows, targets, masks)
    grads = _torch_grads_in_oracle_layout(grads)
    assert worst_ratio(logits, fx.expected[f"logits.{case}"]) <= 1.0
    assert worst_ratio([loss], [want_loss]) <= 1.0
    want = fx.expected_grads(case)
    assert len(want) == (50 if trainable_base else 30)
    for n in want:
        assert worst_ratio(grads[n], want[n]) <= 1.0, n


def biased_tensors(fx, seed, which):
    rng = np.random.default_rng(seed)
    tensors = dict(fx.model)
    for name, w in fx.model.items():
        if name.endswith(".weight") and any(name.endswith(m + ".weight") for m in which):
            tensors[name[:-len(".weight")] + ".bias"] = (rng.standard_normal(w.shape[0]) * 0.1).astype(np.float32)
    return tensors


QKV = ("q_proj", "k_proj", "v_proj")
EVERY = QKV + ("o_proj", "gate_proj", "up_proj", "down_proj", "lm_head")


@pytest.mark.parametrize("which", [QKV, EVERY], ids=["qkv", "every-linear"])
@pytest.mark.parametrize("trainable_base", [False, True])
def test_biased_projections_against_torch_autograd(fx, which, trainable_base):
    rows, targets, masks, _, _ = fx.case("full")
    tensors = biased_tensors(fx, 3, which)
    assert sum(k.endswith(".bias") for k in tensors) == (6 if which is QKV else 15)
    tm = TorchLlama(fx.config, tensors, fx.adapters, fx.meta["lora_alpha"])
    want_logits, want_loss, want = tm.loss_and_grads(rows, targets, masks)
    want = _torch_grads_in_oracle_layout(want)

    model = rs.Model.from_hf_tensors(fx.config, tensors)
    for name, _ in model.named_linears():
        model.set_lora(name, fx.adapters[name + ".lora_a"], fx.adapters[name + ".lora_b"], fx.meta["lora_alpha"])
    logits, cache = model.forward(rows, trainable_base=trainable_base)
    loss, _, grad_logits = rs.masked_cross_entropy_batch(logits, targets, masks, rows.shape[0])
    grads = model.backward(grad_logits, cache)

    # the biases change the outputs: the unbiased fixture logits must NOT match any more
    assert worst_ratio(logits, fx.expected["logits.full"]) > 10.0
    assert worst_ratio(logits, want_logits) <= 1.0
    assert worst_ratio([loss], [want_loss]) <= 1.0
    n_bias = 6 if which is QKV else 15
    assert len(grads) == (50 + n_bias if trainable_base else 30)
    assert ("model.layers.1.self_attn.k_proj.bias" in grads) == trainable_base
    for n in grads:
        assert worst_ratio(grads[n], want[n]) <= 1.0, n
