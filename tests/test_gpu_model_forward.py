"""The HIP model's forward pass against properties that do not need the step: the model-level tests of
ferrotensor-graph/tests/model_correctness.rs on the reference's tiny Llama fixture (2 layers, hidden 32,
vocabulary 32), with the CPU oracle as the independent decoder.

  * earlier_logits_do_not_depend_on_later_tokens (:279-300): bit-identical rows before a changed token
  * batched_forward_matches_each_sequence_alone (:302-317): 1e-4
  * fresh_lora_adapters_do_not_change_the_output (:357-380): bit-identical
  * trained_like_lora_delta_matches_the_merged_weight (:382-429): LoRA logits == logits of W + (alpha/r) A B, 1e-3,
    and the adapters move the logits by more than 0.1
  * f16_base_weights_stay_close_to_f32 (:572-584): 1e-2
"""
import numpy as np
import pytest

from oracle import reference_step as rs
from tests.fixture_io import LORA_EVERYWHERE, GradientParityFixture

pytestmark = pytest.mark.gpu

IDS = np.array([[3, 17, 5, 29, 0, 11, 23, 8]], np.uint32)        # model_correctness.rs:27
SECOND = np.array([[30, 2, 19, 7, 7, 26, 1, 14]], np.uint32)     # :307


@pytest.fixture(scope="module")
def ctx():
    from ferrotensor_amd import HipContext
    c = HipContext(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def fx(golden_dir):
    return GradientParityFixture(golden_dir)


def hip_model(ctx, fx, tensors=None, f16=False):
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig
    c = fx.config
    m = Lfm2Model(ctx, ModelConfig(c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers,
                                   c.num_attention_heads, c.num_key_value_heads, c.rms_norm_eps, c.rope_theta,
                                   c.tie_word_embeddings, f16))
    m.load_tensors(fx.model if tensors is None else tensors)
    return m


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def test_earlier_logits_do_not_depend_on_later_tokens(ctx, fx):
    model = hip_model(ctx, fx)
    changed = IDS.copy()
    changed[0, -1] = (IDS[0, -1] + 1) % fx.config.vocab_size
    a, b = model.forward_batch(IDS), model.forward_batch(changed)
    # causal attention, every other op per token: the rows before the changed token run the same arithmetic
    assert np.array_equal(bits(a[0, :-1]), bits(b[0, :-1]))
    assert np.abs(a[0, -1] - b[0, -1]).max() > 1e-3


def test_batched_forward_matches_each_sequence_alone(ctx, fx):
    model = hip_model(ctx, fx)
    both = model.forward_batch(np.concatenate([IDS, SECOND]))
    assert both.shape == (2, IDS.shape[1], fx.config.vocab_size)
    assert np.abs(both[0] - model.forward_batch(IDS)[0]).max() <= 1e-4
    assert np.abs(both[1] - model.forward_batch(SECOND)[0]).max() <= 1e-4


def test_fresh_lora_adapters_do_not_change_the_output(ctx, fx):
    base = hip_model(ctx, fx)
    with_lora = hip_model(ctx, fx)
    names = with_lora.linear_prefixes(LORA_EVERYWHERE)
    assert len(names) == fx.config.num_hidden_layers * 7 + 1
    for name in names:
        with_lora.add_lora(name, fx.meta["lora_rank"], fx.meta["lora_alpha"])   # A seeded, B = 0
    assert len(with_lora.params()) == 2 * len(names)
    assert np.array_equal(bits(with_lora.forward_batch(IDS)), bits(base.forward_batch(IDS)))


def test_lora_delta_matches_the_merged_weight(ctx, fx):
    rng = np.random.default_rng(1000)
    rank, alpha = fx.meta["lora_rank"], fx.meta["lora_alpha"]
    model = hip_model(ctx, fx)
    merged = {k: np.array(v, np.float32) for k, v in fx.model.items()}
    if "lm_head.weight" not in merged:           # tied head: the adapter only moves the head, not the embedding
        merged["lm_head.weight"] = merged["model.embed_tokens.weight"].copy()
    for name in model.linear_prefixes(LORA_EVERYWHERE):
        w = merged[name + ".weight"]              # HF layout [out, in]
        a = rng.uniform(-0.3, 0.3, (w.shape[1], rank)).astype(np.float32)
        b = rng.uniform(-0.3, 0.3, (rank, w.shape[0])).astype(np.float32)
        model.set_lora(name, a, b, alpha)
        merged[name + ".weight"] = (w.astype(np.float64) + (alpha / rank) * (a.astype(np.float64) @ b).T).astype(np.float32)
    untied = rs.ModelConfig(**{**fx.config.__dict__, "tie_word_embeddings": False})
    want, _ = rs.Model.from_hf_tensors(untied, merged).forward(IDS)
    got = model.forward_batch(IDS)
    assert np.abs(got - want).max() <= 1e-3
    base, _ = rs.Model.from_hf_tensors(fx.config, fx.model).forward(IDS)
    assert np.abs(want - base).max() > 0.1        # the adapters matter, or the comparison proves nothing


def test_f16_base_weights_stay_close_to_f32(ctx, fx):
    model = hip_model(ctx, fx, f16=True)
    want, _ = rs.Model.from_hf_tensors(fx.config, fx.model).forward(IDS)
    got = model.forward_batch(IDS)
    assert np.abs(got - want).max() <= 1e-2
    # and to the bit-level rounding rule: the oracle with the same f16-rounded weights agrees to 1e-4
    want16, _ = rs.Model.from_hf_tensors(fx.config, fx.model, f16_linears=True).forward(IDS)
    assert np.abs(got - want16).max() <= 1e-4
