"""The CPU oracle against the reference's own PyTorch-autograd fixture.

Mirrors ferrotensor-trainer/tests/gradient_parity.rs (check_case :325-395):
loss, logits and every expected gradient of the four cases within
|a-e| <= 1e-4 + 1e-3*|e|; and the logits.base check of
ferrotensor-graph/tests/model_correctness.rs:470-568.
"""
import numpy as np
import pytest

from oracle import reference_step as rs
from tests.fixture_io import GradientParityFixture, worst_ratio


@pytest.fixture(scope="module")
def fx(golden_dir):
    return GradientParityFixture(golden_dir)


@pytest.mark.parametrize("case", ["single", "batch", "masked", "full"])
def test_oracle_matches_pytorch_fixture(fx, case):
    rows, targets, masks, trainable_base, want_loss = fx.case(case)
    model = fx.oracle_model()
    logits, cache = model.forward(rows, trainable_base=trainable_base)
    res = rs.masked_cross_entropy_batch(logits, targets, masks, rows.shape[0])
    assert res is not None
    loss, per_seq, grad_logits = res
    grads = model.backward(grad_logits, cache)

    assert worst_ratio([loss], [want_loss]) <= 1.0, (loss, want_loss)
    assert worst_ratio(logits, fx.expected[f"logits.{case}"]) <= 1.0
    want = fx.expected_grads(case)
    assert len(want) == (50 if trainable_base else 30)
    assert set(grads) == set(want), set(grads) ^ set(want)
    bad = {n: worst_ratio(grads[n], want[n]) for n in want if worst_ratio(grads[n], want[n]) > 1.0}
    assert not bad, bad


def test_base_logits_without_adapters(fx):
    """logits.base: the frozen model with no adapter, first row."""
    model = rs.Model.from_hf_tensors(fx.config, fx.model)
    rows, *_ = fx.case("single")
    logits, _ = model.forward(rows)
    assert worst_ratio(logits, fx.expected["logits.base"], atol=1e-4, rtol=0.0) <= 1.0


def test_padding_to_bucket_leaves_loss_and_grads_unchanged(fx):
    """Trainer pads rows to a multiple of 32 with the last token and mask 0
    (trainer/src/lib.rs:431-450); causal attention hides the padding."""
    rows, targets, masks, _, want_loss = fx.case("masked")
    seqs = [(list(r), list(t), list(m)) for r, t, m in zip(rows, targets, masks)]
    prow, ptgt, pmask = rs.pad_chunk(seqs, 32)
    assert prow.shape == (2, 32) and (prow[:, 8:] == prow[:, 7:8]).all() and not pmask[:, 8:].any()
    model = fx.oracle_model()
    logits, cache = model.forward(prow)
    loss, _, gl = rs.masked_cross_entropy_batch(logits, ptgt, pmask, 2)
    grads = model.backward(gl, cache)
    assert worst_ratio([loss], [want_loss]) <= 1.0
    want = fx.expected_grads("masked")
    assert max(worst_ratio(grads[n], want[n]) for n in want) <= 1.0
