"""The HIP LoRA step against the reference's PyTorch-autograd fixture and the CPU oracle.

Mirrors ferrotensor-trainer/tests/gradient_parity.rs (loss, logits, every LoRA
gradient within |a-e| <= 1e-4 + 1e-3*|e|) and BASELINE config 1 (tiny Llama,
one fwd+bwd+AdamW step compared element-wise with the oracle).
"""
import numpy as np
import pytest

from oracle import reference_step as rs
from tests.fixture_io import GradientParityFixture, worst_ratio
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from ferrotensor_amd import HipContext
    c = HipContext(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def fx(golden_dir):
    return GradientParityFixture(golden_dir)


def hip_model_from_fixture(ctx, fx, trainable_base=False):
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig
    c = fx.config
    cfg = ModelConfig(c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers,
                      c.num_attention_heads, c.num_key_value_heads, c.rms_norm_eps, c.rope_theta,
                      c.tie_word_embeddings, False, trainable_base=trainable_base)
    m = Lfm2Model(ctx, cfg)
    m.load_tensors(fx.model)
    for name in m.linear_prefixes(["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj",
                                   "lm_head"]):
        m.set_lora(name, fx.adapters[name + ".lora_a"], fx.adapters[name + ".lora_b"], fx.meta["lora_alpha"])
    return m


@pytest.mark.parametrize("case", ["single", "batch", "masked", "full"])
def test_lora_gradients_match_pytorch_fixture(ctx, fx, case):
    """The four cases of gradient_parity.rs:416-444; `full` trains the base as well: the gradients of every
    linear weight (in the stored [in, out] layout) and norm scale next to the 30 adapter gradients."""
    from ferrotensor_amd.trainer import Trainer
    rows, targets, masks, trainable_base, want_loss = fx.case(case)
    model = hip_model_from_fixture(ctx, fx, trainable_base)
    logits = model.forward_batch(rows)
    assert worst_ratio(logits, fx.expected[f"logits.{case}"]) <= 1.0
    # grad_accum_steps = 1 gives the backward seed 1 the fixture uses
    tr = Trainer(model, lr=1e-3, grad_accum_steps=1)
    st = tr.train_chunk(rows, targets, masks, apply=False)
    assert worst_ratio([st.loss], [want_loss]) <= 1.0, (st.loss, want_loss)
    want = fx.expected_grads(case)
    grads = model.grads()
    assert set(grads) == set(want) and len(want) == (50 if trainable_base else 30)
    bad = {n: worst_ratio(grads[n], want[n]) for n in want if worst_ratio(grads[n], want[n]) > 1.0}
    assert not bad, bad
    assert not st.optimizer_step


def test_trainable_base_accumulates_and_trains(ctx, fx):
    """With a trainable base the weight and norm-scale gradients accumulate over micro-batches like the adapter
    gradients (two one-sequence chunks == the two-sequence chunk), f16 storage is overridden by f32
    (model_builder.rs:325-340), and an optimizer step moves base weights and norm scales."""
    import dataclasses
    from ferrotensor_amd.trainer import Lfm2Model, Trainer
    rows, targets, masks, _, _ = fx.case("full")
    model = hip_model_from_fixture(ctx, fx, True)
    tr = Trainer(model, lr=1e-3, weight_decay=0.0, grad_accum_steps=2)
    tr.train_chunk(rows, targets, masks, apply=False)
    whole = model.grads()
    model2 = hip_model_from_fixture(ctx, fx, True)
    tr2 = Trainer(model2, lr=1e-3, weight_decay=0.0, grad_accum_steps=2)
    assert not tr2.train_chunk(rows[:1], targets[:1], masks[:1]).optimizer_step
    tr2.train_chunk(rows[1:], targets[1:], masks[1:], apply=False)
    parts = model2.grads()
    assert len(whole) == 50
    for n in whole:
        assert worst_ratio(parts[n], whole[n]) <= 1.0, n
    before = model.params()
    assert tr.train_chunk(rows, targets, masks).optimizer_step
    after = model.params()
    moved = [n for n in before if not np.array_equal(before[n], after[n])]
    assert "model.layers.0.mlp.down_proj.weight" in moved and "model.norm.weight" in moved and len(moved) == 50
    # f16 storage asked for, trainable base wins: the linears stay f32 and keep the fixture's logits
    cfg16 = dataclasses.replace(model.config, f16_linears=True)
    m16 = Lfm2Model(ctx, cfg16)
    m16.load_tensors(fx.model)
    assert worst_ratio(m16.forward_batch(fx.case("single")[0]), fx.expected["logits.base"], atol=1e-5, rtol=0.0) <= 1.0


def test_base_logits_without_adapters(ctx, fx):
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig
    c = fx.config
    m = Lfm2Model(ctx, ModelConfig(c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers,
                                   c.num_attention_heads, c.num_key_value_heads, c.rms_norm_eps, c.rope_theta))
    m.load_tensors(fx.model)
    rows, *_ = fx.case("single")
    assert worst_ratio(m.forward_batch(rows), fx.expected["logits.base"], atol=1e-4, rtol=0.0) <= 1.0


def test_model_directory_loader_and_adapter_file_reproduce_the_fixture(ctx, fx, golden_dir, tmp_path):
    """The reference's fixture directory through the file path a user takes: `load_model` (config.json +
    model.safetensors, f32 linears as the fixture was made), adapters converted to an adapter file and
    applied with `apply_lora_checkpoint` -> the PyTorch golden logits and gradients."""
    import os
    from ferrotensor_amd import checkpoint as ck
    from ferrotensor_amd import loader
    from ferrotensor_amd.trainer import Trainer
    model = loader.load_model(ctx, os.path.join(golden_dir, "gradient_parity"), f16_linears=False)
    rows, targets, masks, _, want_loss = fx.case("batch")
    assert worst_ratio(model.forward_batch(fx.case("single")[0]), fx.expected["logits.base"], atol=1e-4,
                       rtol=0.0) <= 1.0
    # the fixture names its adapters <prefix>.lora_a / .lora_b; the adapter file uses lora_A.weight / lora_B.weight
    tensors = {ck.file_name(n): v for n, v in fx.adapters.items()}
    path = str(tmp_path / "fixture_adapter.safetensors")
    ck.write_safetensors(path, tensors, ck.LoraMetadata(4, fx.meta["lora_alpha"], ["all"]).to_map())
    assert ck.apply_lora_checkpoint(model, ck.load_lora_checkpoint(path)) == 15
    assert worst_ratio(model.forward_batch(rows), fx.expected["logits.batch"]) <= 1.0
    st = Trainer(model, lr=1e-3, grad_accum_steps=1).train_chunk(rows, targets, masks, apply=False)
    assert worst_ratio([st.loss], [want_loss]) <= 1.0
    want = fx.expected_grads("batch")
    grads = model.grads()
    assert max(worst_ratio(grads[n], want[n]) for n in want) <= 1.0


def test_padding_to_bucket_changes_nothing(ctx, fx):
    """Rows padded to 32 with their last token and mask 0 (trainer/src/lib.rs:431-450)."""
    from ferrotensor_amd.trainer import Trainer, pad_chunk
    rows, targets, masks, _, want_loss = fx.case("masked")
    model = hip_model_from_fixture(ctx, fx)
    tr = Trainer(model, lr=1e-3, grad_accum_steps=1)
    seqs = [(list(r), list(t), list(m)) for r, t, m in zip(rows, targets, masks)]
    prow, ptgt, pmask = pad_chunk(seqs, 32)
    assert prow.shape == (len(seqs), 32)
    st = tr.train_chunk(prow, ptgt, pmask, apply=False)
    assert worst_ratio([st.loss], [want_loss]) <= 1.0
    want = fx.expected_grads("masked")
    grads = model.grads()
    assert max(worst_ratio(grads[n], want[n]) for n in want) <= 1.0


def test_train_batch_steps_after_the_same_sequences_as_one_at_a_time(ctx, fx):
    """`train_batch` drops unsupervised sequences and cuts its chunks at the accumulation
    boundary (trainer/src/lib.rs:385-423; the reference's gpu_training.rs:127-186 checks the
    same equivalence): three kept sequences with grad_accum_steps 2 step after the second one
    and leave the third in an open window, batched or one at a time."""
    from ferrotensor_amd.trainer import Trainer
    rows, targets, masks, _, _ = fx.case("masked")
    seqs = [(list(r), list(t), list(m)) for r, t, m in zip(rows, targets, masks)]
    third = (seqs[0][0][::-1], seqs[0][1][::-1], seqs[0][2])
    batch = [seqs[0], (seqs[1][0], seqs[1][1], [0] * len(seqs[1][2])), (seqs[0][0][:1], seqs[0][1][:1], [1]),
             seqs[1], third]

    def run(one_at_a_time):
        model = hip_model_from_fixture(ctx, fx)
        tr = Trainer(model, lr=1e-2, weight_decay=0.0, grad_accum_steps=2, clip_grad_norm=1.0)
        if one_at_a_time:
            stats = [s for q in batch for s in tr.train_batch([q])]
        else:
            stats = tr.train_batch(batch)
        out = (stats, tr.optimizer_steps, tr.step_in_accum, model.params(), model.grads())
        tr.close()
        model.close()
        return out

    stats_b, steps_b, open_b, params_b, grads_b = run(False)
    stats_s, steps_s, open_s, params_s, grads_s = run(True)
    assert [len(s.per_sequence) for s in stats_b] == [2, 1] and len(stats_s) == 3
    assert [s.optimizer_step for s in stats_b] == [True, False]
    assert [s.optimizer_step for s in stats_s] == [False, True, False]
    assert (steps_b, open_b) == (1, 1) and (steps_s, open_s) == (1, 1)
    assert worst_ratio([stats_b[0].loss], [stats_s[0].loss + stats_s[1].loss]) <= 1.0
    assert worst_ratio([stats_b[0].grad_norm], [stats_s[1].grad_norm]) <= 1.0
    for n in params_b:
        assert worst_ratio(params_b[n], params_s[n]) <= 1.0, n
        assert worst_ratio(grads_b[n], grads_s[n]) <= 1.0, n   # the open window: the third sequence alone
    assert Trainer(hip_model_from_fixture(ctx, fx), lr=1e-2).train_batch([batch[1], batch[2]]) == []


def test_a_window_without_supervised_tokens_takes_no_step(ctx, fx):
    """No supervised token: no backward; a window of such chunks has no gradients and
    apply_gradients returns before the norm and the optimizer (trainer/src/lib.rs:301-307).
    The stale gradients of the previous window must neither be applied nor added to."""
    from ferrotensor_amd.trainer import Trainer
    rows, targets, masks, _, _ = fx.case("masked")
    model = hip_model_from_fixture(ctx, fx)
    tr = Trainer(model, lr=1e-2, weight_decay=0.0, grad_accum_steps=2)
    first = tr.train_chunk(rows, targets, masks)
    assert first.optimizer_step and tr.optimizer_steps == 1
    before = model.params()
    blank = tr.train_chunk(rows, targets, np.zeros_like(masks))
    assert not blank.optimizer_step and blank.tokens == 0 and blank.loss == 0.0 and blank.grad_norm == 0.0
    assert tr.optimizer_steps == 1 and tr.step_in_accum == 0
    after = model.params()
    for n in before:
        assert np.array_equal(before[n], after[n]), n
    # an empty chunk that opens a window, then a supervised one that closes it: its gradient alone
    tr.train_chunk(rows[:1], targets[:1], np.zeros_like(masks[:1]))
    assert tr.step_in_accum == 1
    tr.train_chunk(rows[:1], targets[:1], masks[:1], apply=False)
    got = model.grads()
    ref_model = hip_model_from_fixture(ctx, fx)
    ref_tr = Trainer(ref_model, lr=1e-2, weight_decay=0.0, grad_accum_steps=2)
    ref_tr.train_chunk(rows, targets, masks)          # the same first step: same adapters as `model`
    ref_tr.train_chunk(rows[:1], targets[:1], masks[:1], apply=False)
    want = ref_model.grads()                           # one sequence in a window of two: never closed, seed 1/2
    for n in want:
        assert worst_ratio(got[n], want[n]) <= 1.0, n


# ---- BASELINE config 1: tiny Llama, one full step vs the oracle ----------------

def tiny_config(f16=False, tied=False):
    from ferrotensor_amd.trainer import ModelConfig
    return ModelConfig(vocab_size=256, hidden_size=32, intermediate_size=64, num_hidden_layers=2,
                       num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, rope_theta=10000.0,
                       tie_word_embeddings=tied, f16_linears=f16)


def random_model_tensors(cfg, seed):
    rng = np.random.default_rng(seed)
    n = lambda *s: (rng.standard_normal(s) * 0.02).astype(np.float32)
    H, F, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    D = H // cfg.num_attention_heads
    t = {"model.embed_tokens.weight": n(V, H), "model.norm.weight": np.ones(H, np.float32)}
    if not cfg.tie_word_embeddings:
        t["lm_head.weight"] = n(V, H)
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}"
        t[f"{p}.input_layernorm.weight"] = np.ones(H, np.float32)
        t[f"{p}.post_attention_layernorm.weight"] = np.ones(H, np.float32)
        t[f"{p}.self_attn.q_proj.weight"] = n(cfg.num_attention_heads * D, H)
        t[f"{p}.self_attn.k_proj.weight"] = n(cfg.num_key_value_heads * D, H)
        t[f"{p}.self_attn.v_proj.weight"] = n(cfg.num_key_value_heads * D, H)
        t[f"{p}.self_attn.o_proj.weight"] = n(H, cfg.num_attention_heads * D)
        t[f"{p}.mlp.gate_proj.weight"] = n(F, H)
        t[f"{p}.mlp.up_proj.weight"] = n(F, H)
        t[f"{p}.mlp.down_proj.weight"] = n(H, F)
    return t


def build_pair(ctx, cfg, targets_mods, rank, alpha, seed):
    """The same seeded model in the HIP library and in the oracle."""
    from ferrotensor_amd.trainer import Lfm2Model
    tensors = random_model_tensors(cfg, seed)
    hip = Lfm2Model(ctx, cfg)
    hip.load_tensors(tensors)
    ocfg = rs.ModelConfig(cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers,
                          cfg.num_attention_heads, cfg.num_key_value_heads, cfg.rms_norm_eps, cfg.rope_theta,
                          cfg.tie_word_embeddings)
    orc = rs.Model.from_hf_tensors(ocfg, tensors, f16_linears=cfg.f16_linears)
    rng = np.random.default_rng(seed + 1)
    for name in hip.linear_prefixes(targets_mods):
        i, o = hip.linear_dims(name)
        a = (rng.standard_normal((i, rank)) * 0.02).astype(np.float32)
        b = (rng.standard_normal((rank, o)) * 0.02).astype(np.float32)
        hip.set_lora(name, a, b, alpha)
        orc.set_lora(name, a, b, alpha)
    return hip, orc


@pytest.mark.parametrize("f16,tied", [(False, False), (True, True)])
def test_tiny_llama_full_step_matches_oracle(ctx, f16, tied):
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config(f16, tied)
    mods = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    hip, orc = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=11)
    rng = np.random.default_rng(5)
    B, S = 2, 16
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rng.integers(0, 256, (B, 1)).astype(np.uint32)], axis=1)
    masks = np.ones((B, S), np.uint8)
    masks[:, :4] = 0

    logits = hip.forward_batch(rows)
    want_logits, _ = orc.forward(rows)
    assert_close("logits", logits, want_logits)

    tr = Trainer(hip, lr=1e-3, weight_decay=0.01, clip_grad_norm=1.0)   # grad_accum = B (CLI: batch * accum)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.01)
    for step in range(3):
        # gradients of this step (no update), then the same step applied
        st0 = tr.train_chunk(rows, targets, masks, apply=False)
        grads = hip.grads()
        want_stats, _, want_grads = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0,
                                                   return_grads=True)
        # the oracle applied its update; grads it returns are clipped -> undo for comparison
        cs = want_stats.clip_scale or 1.0
        for n in grads:
            assert_close(f"step {step} grad {n}", grads[n], want_grads[n] / np.float32(cs))
        st = tr.train_chunk(rows, targets, masks, apply=True)
        assert st.optimizer_step and want_stats.optimizer_step
        assert_close("loss", [st.loss], [want_stats.loss])
        assert_close("grad_norm", [st.grad_norm], [want_stats.grad_norm])
        assert_close("clip_scale", [st.clip_scale], [cs], atol=1e-6)
        assert st.tokens == sum(t for _, t in want_stats.per_sequence)
        assert_close("per-sequence", st.per_sequence, [l for l, _ in want_stats.per_sequence])
        params = hip.params()
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)


def _moments(tr):
    """{param name: (m, v)} of the trainer's AdamW state, keyed like `Lfm2Model.params()`."""
    import ctypes as C
    out = {}
    for i, (name, numel) in enumerate(tr.model.named_params()):
        m, v = np.empty(numel, np.float32), np.empty(numel, np.float32)
        from ferrotensor_amd._lib import check
        check(tr._lib.ft_trainer_read_moments(tr.handle, i, m.ctypes.data_as(C.c_void_p),
                                              v.ctypes.data_as(C.c_void_p)))
        out[name] = (m, v)
    return out


def _adam_t(tr):
    import ctypes as C
    t = C.c_float()
    tr._lib.ft_trainer_get_adam_t(tr.handle, C.byref(t))
    return t.value


def _clip_case(ctx, seed=11):
    cfg = tiny_config(True, True)
    mods = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    hip, orc = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=seed)
    rng = np.random.default_rng(5)
    B, S = 2, 16
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rng.integers(0, 256, (B, 1)).astype(np.uint32)], axis=1)
    masks = np.ones((B, S), np.uint8)
    masks[:, :4] = 0
    return hip, orc, rows, targets, masks, rng


def test_gradient_clip_fires_against_oracle(ctx):
    """`apply_gradients` with the clip active (trainer/src/lib.rs:336-343): the tiny config's gradient norm is
    0.07-0.08, so a clip at 0.01 scales every gradient in every step. Norm, clip scale, the updated weights
    and both AdamW moments against the oracle over three steps."""
    from ferrotensor_amd.trainer import Trainer
    hip, orc, rows, targets, masks, _ = _clip_case(ctx)
    tr = Trainer(hip, lr=1e-3, weight_decay=0.01, clip_grad_norm=0.01)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.01)
    for step in range(3):
        want = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=0.01)
        st = tr.train_chunk(rows, targets, masks)
        assert st.optimizer_step and want.optimizer_step
        assert want.clip_scale is not None and want.clip_scale < 0.5, want
        assert_close("loss", [st.loss], [want.loss])
        assert_close("grad_norm", [st.grad_norm], [want.grad_norm])
        assert_close("clip_scale", [st.clip_scale], [want.clip_scale], atol=1e-7, rtol=1e-3)
        params, mom = hip.params(), _moments(tr)
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)
            # the moments of clipped gradients are tiny (m ~1e-5, v ~1e-11): bars relative to their scale
            m_bar, v_bar = 1e-3 * np.abs(opt.m[n]).max(), 2e-3 * np.abs(opt.v[n]).max()
            assert_close(f"step {step} m {n}", mom[n][0], opt.m[n], atol=m_bar, rtol=1e-3)
            assert_close(f"step {step} v {n}", mom[n][1], opt.v[n], atol=v_bar, rtol=2e-3)
        assert _adam_t(tr) == opt.t == step + 1


def test_gradient_clip_over_an_accumulation_window(ctx):
    """A window of 4 sequences fed as two chunks of 2 (seed 1/4 each): the norm and the clip see the summed
    gradients, once, when the window closes."""
    from ferrotensor_amd.trainer import Trainer
    hip, orc, rows, targets, masks, rng = _clip_case(ctx, seed=13)
    B = rows.shape[0]
    tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=0.03, grad_accum_steps=4)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.0)
    rows2 = rng.integers(0, 256, rows.shape).astype(np.uint32)
    targets2 = np.concatenate([rows2[:, 1:], rows2[:, :1]], axis=1)
    first = tr.train_chunk(rows, targets, masks)
    assert not first.optimizer_step and first.clip_scale == 1.0
    st = tr.train_chunk(rows2, targets2, masks)
    assert st.optimizer_step
    params_o = orc.lora_params()
    total = {}
    for r_, t_ in ((rows, targets), (rows2, targets2)):
        logits, cache = orc.forward(r_)
        _, _, gl = rs.masked_cross_entropy_batch(logits, t_, masks, B)
        for n, gval in orc.backward(rs.cpu.scale(gl, 0.25), cache).items():
            total[n] = gval if n not in total else rs.cpu.add(total[n], gval)
    stats = rs.StepStats(0.0, [], None, False)
    rs.apply_gradients(params_o, total, opt, stats, clip_grad_norm=0.03)
    assert stats.clip_scale is not None and stats.clip_scale < 0.95, stats
    assert_close("grad_norm", [st.grad_norm], [stats.grad_norm])
    assert_close("clip_scale", [st.clip_scale], [stats.clip_scale], atol=1e-7, rtol=1e-3)
    params = hip.params()
    for n, w in params_o:
        assert_close(f"weight {n}", params[n], w, atol=1e-6, rtol=1e-4)


def test_fixture_model_step_with_the_clip_at_one(ctx, fx):
    """The reference fixture's model has a gradient norm of about 4.4 on its `batch` case: with the CLI's
    `clip_grad_norm = 1.0` the clip scale is about 0.22. Two optimizer steps against the oracle."""
    from ferrotensor_amd.trainer import Trainer
    rows, targets, masks, _, _ = fx.case("batch")
    model = hip_model_from_fixture(ctx, fx)
    orc = fx.oracle_model()
    tr = Trainer(model, lr=1e-2, weight_decay=0.0, clip_grad_norm=1.0)
    opt = rs.AdamW(lr=1e-2, weight_decay=0.0)
    for step in range(2):
        want = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0)
        st = tr.train_chunk(rows, targets, masks)
        assert want.clip_scale is not None and want.grad_norm > 1.0
        assert_close("loss", [st.loss], [want.loss])
        assert_close("grad_norm", [st.grad_norm], [want.grad_norm])
        assert_close("clip_scale", [st.clip_scale], [want.clip_scale], atol=1e-7, rtol=1e-3)
        params = model.params()
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)


@pytest.mark.parametrize("bad", [np.nan, np.inf])
def test_non_finite_gradient_norm_skips_the_step(ctx, bad):
    """trainer/src/lib.rs:330-335: a NaN / Inf gradient norm skips the optimizer step. Weights, moments, AdamW's
    t, the step counter and the LR schedule stay where they were, the window is closed (zero_grad), and the
    next clean window overwrites the poisoned gradients and steps as if nothing had happened."""
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config(True, True)
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    hip, orc = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=29)
    rng = np.random.default_rng(15)
    rows = rng.integers(0, 256, (2, 16)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((2, 16), np.uint8)
    kw = dict(lr=2e-3, weight_decay=0.01, clip_grad_norm=1.0, lr_schedule="warmup_cosine", warmup_steps=2,
              total_steps=6, min_lr=2e-4)
    tr = Trainer(hip, **kw)
    opt = rs.AdamW(lr=2e-3, weight_decay=0.01)
    sched = rs.WarmupCosineScheduler(2e-3, 2e-4, 2, 6)
    want = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0, scheduler=sched)
    st = tr.train_chunk(rows, targets, masks)
    assert st.optimizer_step and tr.optimizer_steps == 1 and _adam_t(tr) == 1.0

    # poison one element of one B factor (both models)
    name = "model.layers.1.self_attn.v_proj"
    clean = hip.params()
    a = clean[name + ".lora_a"].reshape(cfg.hidden_size, 4)
    b = clean[name + ".lora_b"].reshape(4, -1).copy()
    b_bad = b.copy()
    b_bad[2, 5] = bad
    hip.set_lora(name, a, b_bad, 8.0)
    before, mom_before = hip.params(), _moments(tr)
    skipped = tr.train_chunk(rows, targets, masks)
    assert not skipped.optimizer_step and skipped.lr is None
    assert not np.isfinite(skipped.grad_norm)
    assert tr.optimizer_steps == 1 and _adam_t(tr) == 1.0 and tr.step_in_accum == 0
    after, mom_after = hip.params(), _moments(tr)
    for n in before:
        assert np.array_equal(before[n].view(np.uint32), after[n].view(np.uint32)), n
        assert np.array_equal(mom_before[n][0], mom_after[n][0]) and np.array_equal(mom_before[n][1], mom_after[n][1]), n
    # the oracle follows the same rule on the same poisoned factor
    orc_lin = dict(orc.named_linears())[name]
    orc_b_clean = orc_lin.lora_b.copy()
    orc_lin.lora_b[2, 5] = bad
    want_skip = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0, scheduler=sched)
    assert not want_skip.optimizer_step and opt.t == 1.0 and sched.current == 1
    orc_lin.lora_b[...] = orc_b_clean

    # repaired: the next window steps with t = 2 and the schedule's second value
    hip.set_lora(name, a, b, 8.0)
    want2 = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0, scheduler=sched)
    st2 = tr.train_chunk(rows, targets, masks)
    assert st2.optimizer_step and tr.optimizer_steps == 2 and _adam_t(tr) == 2.0
    assert abs(st2.lr - want2.lr) <= 2e-7 * 2e-3
    assert_close("loss", [st2.loss], [want2.loss])
    assert_close("grad_norm", [st2.grad_norm], [want2.grad_norm])
    params = hip.params()
    for n, w in orc.lora_params():
        assert_close(f"weight {n}", params[n], w, atol=1e-6, rtol=1e-4)


def test_a_trainer_is_refused_after_the_adapters_change(ctx):
    """A trainer sizes its moments from, and points into, the adapters it was created over. Changing a rank or
    adding an adapter afterwards reallocates them: the old trainer must report an error, not run through
    freed buffers; a new trainer works, and re-setting an adapter at the same rank keeps the old one valid."""
    from ferrotensor_amd import FtError
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config()
    hip, _ = build_pair(ctx, cfg, ["q_proj", "v_proj"], rank=4, alpha=8.0, seed=33)
    rng = np.random.default_rng(1)
    rows = rng.integers(0, 256, (2, 16)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((2, 16), np.uint8)
    tr = Trainer(hip, lr=1e-3)
    assert tr.train_chunk(rows, targets, masks).optimizer_step
    name = "model.layers.0.self_attn.q_proj"
    i, o = hip.linear_dims(name)
    same = hip.params()
    hip.set_lora(name, same[name + ".lora_a"].reshape(i, 4), same[name + ".lora_b"].reshape(4, o), 8.0)
    assert tr.train_chunk(rows, targets, masks).optimizer_step          # same rank: nothing was reallocated
    hip.set_lora(name, np.zeros((i, 8), np.float32), np.zeros((8, o), np.float32), 16.0)
    with pytest.raises(FtError, match="create a new trainer"):
        tr.train_chunk(rows, targets, masks)
    with pytest.raises(FtError, match="create a new trainer"):
        _moments(tr)
    assert tr.optimizer_steps == 2
    tr2 = Trainer(hip, lr=1e-3)
    assert tr2.train_chunk(rows, targets, masks).optimizer_step
    hip.add_lora("model.layers.1.mlp.down_proj", 4, 8.0)                  # a new adapter: same rule
    with pytest.raises(FtError, match="create a new trainer"):
        tr2.train_chunk(rows, targets, masks)
    assert Trainer(hip, lr=1e-3).train_chunk(rows, targets, masks).optimizer_step


@pytest.mark.parametrize("rank", [2, 32])
def test_other_ranks_step_with_accumulation_matches_oracle(ctx, rank):
    """Ranks outside {4, 8, 16} take the general kernels for x@A, dT, dA, dB and the rank-r terms, and with
    two micro-batches per window the accumulate branch of the factor gradients (temporary + add). Two
    optimizer steps of a window of 4 sequences fed 2 + 2, against the oracle's summed gradients."""
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config(True, True)
    mods = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    hip, orc = build_pair(ctx, cfg, mods, rank=rank, alpha=2.0 * rank, seed=37)
    rng = np.random.default_rng(7)
    B, S = 4, 16
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = (rng.random((B, S)) > 0.2).astype(np.uint8)
    tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0, grad_accum_steps=B)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.0)
    for step in range(2):
        first = tr.train_chunk(rows[:2], targets[:2], masks[:2])
        assert not first.optimizer_step
        st = tr.train_chunk(rows[2:], targets[2:], masks[2:])
        assert st.optimizer_step
        # the oracle on all four sequences at once: the same window
        want = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0)
        assert_close("loss", [first.loss + st.loss], [want.loss])
        assert_close("grad_norm", [st.grad_norm], [want.grad_norm])
        params = hip.params()
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)
    # and the gradients themselves, element by element, on one more window
    tr.train_chunk(rows[:2], targets[:2], masks[:2], apply=False)
    tr.train_chunk(rows[2:], targets[2:], masks[2:], apply=False)
    grads = hip.grads()
    want, _, want_grads = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=None, return_grads=True)
    for n in grads:
        assert_close(f"grad {n}", grads[n], want_grads[n])


def test_warmup_cosine_schedule_drives_the_step(ctx):
    """Optimizer step k uses the schedule's value at k (trainer/src/lib.rs:345-352); a resumed
    trainer continues the curve where the counter says."""
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config()
    hip, orc = build_pair(ctx, cfg, ["q_proj", "k_proj", "v_proj", "o_proj"], rank=4, alpha=8.0, seed=21)
    rng = np.random.default_rng(6)
    rows = rng.integers(0, 256, (2, 16)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((2, 16), np.uint8)
    peak, low, warm, total = 2e-3, 2e-4, 2, 6
    tr = Trainer(hip, lr=peak, weight_decay=0.0, lr_schedule="warmup_cosine", warmup_steps=warm, total_steps=total,
                 min_lr=low)
    opt = rs.AdamW(lr=peak, weight_decay=0.0)
    sched = rs.WarmupCosineScheduler(peak, low, warm, total)
    for step in range(4):
        want = rs.train_chunk(orc, opt, rows, targets, masks, scheduler=sched)
        st = tr.train_chunk(rows, targets, masks)
        assert st.optimizer_step and tr.optimizer_steps == step + 1
        assert abs(st.lr - want.lr) <= 2e-7 * peak, (step, st.lr, want.lr)
        assert_close("loss", [st.loss], [want.loss])
        params = hip.params()
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)
    # resume at step 5 of 6: the next step is the last of the curve and lands on min_lr
    tr.set_optimizer_steps(5)
    st = tr.train_chunk(rows, targets, masks)
    assert st.lr == np.float32(low) and tr.optimizer_steps == 6


def test_fresh_adapters_are_seeded_like_the_builder(ctx):
    """`maybe_add_lora`: A from xorshift64* seeded by (layer index + 1, module name), B zero, so the
    model starts at the base logits; one training step then moves B away from zero."""
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config()
    hip, orc = build_pair(ctx, cfg, [], rank=4, alpha=8.0, seed=13)
    rows = np.random.default_rng(2).integers(0, 256, (2, 16)).astype(np.uint32)
    base = hip.forward_batch(rows)
    for prefix in hip.linear_prefixes(["q_proj", "v_proj", "down_proj"]):
        hip.add_lora(prefix, 4, 8.0)
    params = hip.params()
    for layer in range(cfg.num_hidden_layers):
        for mod, sub in (("q_proj", "self_attn"), ("v_proj", "self_attn"), ("down_proj", "mlp")):
            prefix = f"model.layers.{layer}.{sub}.{mod}"
            i, o = hip.linear_dims(prefix)
            want = rs.lora_init_a(i, o, 4, rs.lora_seed(layer + 1, mod))
            np.testing.assert_array_equal(params[prefix + ".lora_a"].reshape(want.shape), want)
            assert not params[prefix + ".lora_b"].any()
    np.testing.assert_array_equal(hip.forward_batch(rows), base)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    st = Trainer(hip, lr=1e-2, weight_decay=0.0).train_chunk(rows, targets, np.ones((2, 16), np.uint8))
    assert st.optimizer_step
    after = hip.params()
    assert all(after[n].any() for n in after if n.endswith(".lora_b"))


def test_block_checkpointing_changes_no_bit(ctx):
    """Recomputing a block in backward runs the same kernels on the same inputs: loss, gradients and
    updated weights are identical to the plain step (ferrotensor-graph/tests/block_checkpointing.rs)."""
    import dataclasses
    from ferrotensor_amd.trainer import Trainer
    mods = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    rng = np.random.default_rng(8)
    rows = rng.integers(0, 256, (2, 32)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = (rng.random((2, 32)) > 0.3).astype(np.uint8)
    results = []
    for ckpt in (False, True):
        cfg = dataclasses.replace(tiny_config(True, True), checkpoint_blocks=ckpt, num_hidden_layers=3)
        hip, _ = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=17)
        tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0)
        losses = []
        for _ in range(2):
            st0 = tr.train_chunk(rows, targets, masks, apply=False)
            grads = hip.grads()
            st = tr.train_chunk(rows, targets, masks)
            losses.append((st0.loss, st.loss, st.grad_norm))
        results.append((losses, grads, hip.params()))
        tr.close()
        hip.close()
    (l0, g0, p0), (l1, g1, p1) = results
    assert l0 == l1
    for n in g0:
        np.testing.assert_array_equal(g0[n], g1[n])
    for n in p0:
        np.testing.assert_array_equal(p0[n], p1[n])


def test_resume_from_adapter_and_state_files_is_bit_identical(ctx, tmp_path):
    """3 steps straight through == 2 steps, save (adapter file + training checkpoint), fresh model and
    trainer, load, 1 step: weights, moments and the schedule all continue where they stopped."""
    from ferrotensor_amd import checkpoint as ck
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config(True, True)
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    rng = np.random.default_rng(12)
    rows = rng.integers(0, 256, (2, 16)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((2, 16), np.uint8)
    kw = dict(lr=1e-3, weight_decay=0.01, clip_grad_norm=1.0, lr_schedule="warmup_cosine", warmup_steps=2,
              total_steps=5, min_lr=1e-4)

    hip, _ = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=19)
    tr = Trainer(hip, **kw)
    straight = [tr.train_chunk(rows, targets, masks) for _ in range(3)]
    want = hip.params()

    hip2, _ = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=19)
    tr2 = Trainer(hip2, **kw)
    for _ in range(2):
        tr2.train_chunk(rows, targets, masks)
    adapter, state_path = str(tmp_path / "adapter.safetensors"), str(tmp_path / "run.state.json")
    ck.save_lora_checkpoint(hip2, adapter, ck.LoraMetadata(4, 8.0, mods))
    ck.save_training_checkpoint(state_path, ck.TrainingState(step=tr2.optimizer_steps, total_steps=5, lr=1e-3),
                                ck.optimizer_state(tr2))
    tr2.close()
    hip2.close()

    hip3, _ = build_pair(ctx, cfg, [], rank=4, alpha=8.0, seed=19)        # base weights only
    loaded = ck.load_lora_checkpoint(adapter)
    assert loaded.metadata == ck.LoraMetadata(4, 8.0, mods) and len(loaded.tensors) == 2 * 4 * cfg.num_hidden_layers
    assert "model.layers.1.self_attn.o_proj.lora_B.weight" in loaded.tensors
    assert ck.apply_lora_checkpoint(hip3, loaded) == 4 * cfg.num_hidden_layers
    tr3 = Trainer(hip3, **kw)
    state, adam = ck.load_training_checkpoint(state_path)
    assert state.step == 2 and adam.t == 2.0
    assert ck.restore_optimizer(tr3, adam, state.step) == ck.OptimizerLoad(2 * 4 * cfg.num_hidden_layers, 0, 0)
    st = tr3.train_chunk(rows, targets, masks)
    assert (st.loss, st.grad_norm, st.lr) == (straight[2].loss, straight[2].grad_norm, straight[2].lr)
    got = hip3.params()
    for n in want:
        np.testing.assert_array_equal(got[n], want[n])


def test_optimizer_state_load_reports_what_it_matched(ctx):
    """`optimizer_state_load_reports_what_it_matched` (ferrotensor-trainer/tests/gpu_training.rs:338-402): the same
    parameters all take their moments back (and `t`, and the saved hyperparameters); disjoint names match
    nothing, say so and leave the optimizer as it was; a moment of the wrong shape is an error that names the
    parameter, and nothing is applied."""
    import dataclasses
    from ferrotensor_amd import checkpoint as ck
    from ferrotensor_amd.trainer import Trainer
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    seq = np.array([(i * 7 + 3) % 64 for i in range(24)], np.uint32)
    rows, targets, masks = seq[None, :-1], seq[None, 1:], np.ones((1, 23), np.uint8)
    hip, _ = build_pair(ctx, tiny_config(), mods, rank=4, alpha=8.0, seed=31)
    trained = Trainer(hip, lr=1e-2, beta1=0.8, weight_decay=0.05, grad_accum_steps=1)
    for _ in range(2):
        trained.train_chunk(rows, targets, masks)
    state = ck.optimizer_state(trained)
    n = len(hip.named_params())
    assert n == 2 * 4 * 2 and state.t == 2.0

    def moments(tr):
        return ck.optimizer_state(tr)

    same = Trainer(hip, lr=1e-3, grad_accum_steps=1)
    assert ck.restore_optimizer(same, state) == ck.OptimizerLoad(n, 0, 0)
    back = moments(same)
    assert back.t == 2.0 and (back.lr, back.beta1, back.weight_decay) == (1e-2, 0.8, 0.05)
    for k in state.m_states:
        assert np.array_equal(back.m_states[k], state.m_states[k]) and np.array_equal(back.v_states[k], state.v_states[k])
    # the restored optimizer continues exactly like the one that was saved: same adapters, same third step
    before = hip.params()
    third = trained.train_chunk(rows, targets, masks)
    want = hip.params()
    for i, (name, _) in enumerate(hip.named_params()):
        hip.write_param(i, before[name])
    again = same.train_chunk(rows, targets, masks)
    assert (again.loss, again.grad_norm) == (third.loss, third.grad_norm)
    got = hip.params()
    for name in want:
        assert np.array_equal(got[name].view(np.uint32), want[name].view(np.uint32)), name
    same.close()

    renamed = dataclasses.replace(state, m_states={"other." + k: v for k, v in state.m_states.items()},
                                  v_states={"other." + k: v for k, v in state.v_states.items()})
    other = Trainer(hip, lr=1e-3, grad_accum_steps=1)
    assert ck.restore_optimizer(other, renamed) == ck.OptimizerLoad(0, n, n)
    untouched = moments(other)
    assert untouched.t == 0.0 and untouched.lr == 1e-3 and all(not m.any() for m in untouched.m_states.values())
    other.close()

    victim = min(state.v_states)
    bad = dataclasses.replace(state, v_states={**state.v_states, victim: state.v_states[victim].reshape(-1)})
    wrong = Trainer(hip, lr=1e-3, grad_accum_steps=1)
    with pytest.raises(ValueError) as err:
        ck.restore_optimizer(wrong, bad)
    assert victim in str(err.value) and "shape" in str(err.value)
    untouched = moments(wrong)
    assert untouched.t == 0.0 and all(not m.any() for m in untouched.m_states.values())
    wrong.close()
    trained.close()
    hip.close()


def test_adapter_with_wrong_rank_is_rejected(ctx, tmp_path):
    """`adapter_with_wrong_rank_is_rejected` (gpu_training.rs:404-443): a model built with rank-2 adapters cannot
    take the rank-4 tensors of an adapter file saved without metadata; the error speaks of the shape."""
    from ferrotensor_amd import checkpoint as ck
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    hip, _ = build_pair(ctx, tiny_config(), mods, rank=4, alpha=8.0, seed=33)
    path = str(tmp_path / "a.safetensors")
    ck.save_lora_checkpoint(hip, path)
    hip.close()
    loaded = ck.load_lora_checkpoint(path)
    assert loaded.metadata is None
    other, _ = build_pair(ctx, tiny_config(), mods, rank=2, alpha=8.0, seed=33)
    with pytest.raises(ValueError) as err:
        ck.apply_checkpoint(loaded, other)
    assert "shape" in str(err.value)
    other.close()


def test_micro_batches_accumulate_to_the_batched_step(ctx):
    """`--batch 1 --accum 4` == `--batch 4` (ferrotensor-trainer/tests/gpu_training.rs:127-186): four
    one-sequence chunks accumulate into the gradients of the four-sequence chunk, and the optimizer
    steps once, after the last one."""
    from ferrotensor_amd.trainer import Trainer
    mods = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    rng = np.random.default_rng(14)
    rows = rng.integers(0, 256, (4, 32)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = (rng.random((4, 32)) > 0.25).astype(np.uint8)
    out = []
    for micro in (4, 1, 2):
        hip, _ = build_pair(ctx, tiny_config(True, True), mods, rank=4, alpha=8.0, seed=23)
        tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0, grad_accum_steps=4)
        steps, loss = [], 0.0
        for i in range(0, 4, micro):
            st = tr.train_chunk(rows[i:i + micro], targets[i:i + micro], masks[i:i + micro])
            steps.append(st.optimizer_step)
            loss += st.loss
        assert steps == [False] * (4 // micro - 1) + [True] and tr.optimizer_steps == 1
        out.append((loss, st.grad_norm, hip.grads(), hip.params()))
        tr.close()
        hip.close()
    (l0, n0, g0, p0) = out[0]
    for (l, n, g, p) in out[1:]:
        assert_close("loss", [l], [l0])
        assert_close("grad_norm", [n], [n0])
        for k in g0:
            assert_close("grad " + k, g[k], g0[k])
            assert_close("param " + k, p[k], p0[k], atol=1e-6, rtol=1e-4)


def test_training_on_one_batch_halves_the_loss(ctx):
    """`lora_training_reduces_loss_on_a_tiny_model` and `f16_base_weights_halve_memory_and_train_like_f32`
    (ferrotensor-trainer/tests/gpu_training.rs:24-54, 56-95): a tiny model with weights of the reference test's
    scale (embedding 0.5, linears 0.2, tests/common/mod.rs:102-118), freshly seeded rank-4 adapters on q/k/v/o,
    one memorisable sequence ((7i + 3) mod 64, common/mod.rs:370-372), AdamW at 1e-2: 40 optimizer steps at
    least halve the loss, with f32 and with f16 base weights, whose first loss is within 1 % of the f32 one."""
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig, Trainer
    seq = np.array([(i * 7 + 3) % 64 for i in range(24)], np.uint32)
    rows, targets = seq[None, :-1], seq[None, 1:]
    masks = np.ones_like(rows, dtype=np.uint8)
    runs = {}
    for f16 in (False, True):
        cfg = ModelConfig(vocab_size=64, hidden_size=32, intermediate_size=64, num_hidden_layers=2,
                          num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, rope_theta=10000.0,
                          tie_word_embeddings=False, f16_linears=f16)
        tensors = random_model_tensors(cfg, 3)
        rng = np.random.default_rng(17)
        for name, w in tensors.items():
            if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
                continue
            scale = 0.5 if "embed_tokens" in name else 0.2
            tensors[name] = rng.uniform(-scale, scale, w.shape).astype(np.float32)
        hip = Lfm2Model(ctx, cfg)
        hip.load_tensors(tensors)
        for prefix in hip.linear_prefixes(["q_proj", "k_proj", "v_proj", "o_proj"]):
            hip.add_lora(prefix, 4, 8.0)
        tr = Trainer(hip, lr=1e-2, grad_accum_steps=1)
        losses = []
        for _ in range(40):
            st = tr.train_chunk(rows, targets, masks)
            assert st.optimizer_step
            losses.append(st.loss)
        tr.close()
        hip.close()
        assert all(np.isfinite(losses))
        assert losses[-1] < 0.5 * losses[0], (f16, losses)
        runs[f16] = losses
    assert abs(runs[True][0] - runs[False][0]) <= 1e-2 * runs[False][0], (runs[True][0], runs[False][0])


def test_gradient_accumulation_defers_the_step_and_is_deterministic(ctx):
    """gpu_training.rs:224-253: with grad_accum = 2 the first sequence only accumulates and the second applies
    the update; repeating the run gives bit-identical adapters, stepping after every sequence different ones."""
    from ferrotensor_amd.trainer import Trainer
    seq = np.array([(i * 7 + 3) % 64 for i in range(24)], np.uint32)
    a = (seq[None, :12], seq[None, 1:13])
    b = (seq[None, 6:18], seq[None, 7:19])
    ones = np.ones((1, 12), np.uint8)

    def run(accum):
        hip, _ = build_pair(ctx, tiny_config(False, False), ["q_proj", "k_proj", "v_proj", "o_proj"], rank=4,
                            alpha=8.0, seed=29)
        tr = Trainer(hip, lr=1e-2, grad_accum_steps=accum)
        s1 = tr.train_chunk(a[0], a[1], ones)
        s2 = tr.train_chunk(b[0], b[1], ones)
        values = hip.params()
        tr.close()
        hip.close()
        return s1, s2, values

    s1, s2, accumulated = run(2)
    assert not s1.optimizer_step and s2.optimizer_step
    _, _, again = run(2)
    for k in accumulated:
        assert np.array_equal(accumulated[k].view(np.uint32), again[k].view(np.uint32)), k
    p1, p2, sequential = run(1)
    assert p1.optimizer_step and p2.optimizer_step
    assert any(not np.array_equal(accumulated[k], sequential[k]) for k in accumulated)

def test_the_step_is_deterministic_to_the_bit(ctx):
    """Two runs of the same three steps from the same state give the same bits in every gradient, weight and
    moment (gpu_training.rs:224-253): every reduction of the step has a fixed order, including the factor
    gradients computed on the second stream and the split-K partial sums."""
    from ferrotensor_amd.trainer import Trainer
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    rng = np.random.default_rng(6)
    rows = rng.integers(0, 256, (3, 64)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = (rng.random((3, 64)) > 0.3).astype(np.uint8)
    from ferrotensor_amd import checkpoint as ck
    from ferrotensor_amd.trainer import ModelConfig
    cfg = ModelConfig(vocab_size=256, hidden_size=192, intermediate_size=256, num_hidden_layers=2,
                      num_attention_heads=3, num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=100000.0,
                      tie_word_embeddings=True, f16_linears=True)
    runs = []
    for _ in range(2):
        hip, _ = build_pair(ctx, cfg, mods, rank=8, alpha=16.0, seed=41)
        tr = Trainer(hip, lr=1e-3, weight_decay=0.01, clip_grad_norm=1.0, grad_accum_steps=3)
        stats = [tr.train_chunk(rows, targets, masks) for _ in range(3)]
        adam = ck.optimizer_state(tr)
        runs.append(([(s.loss, s.grad_norm) for s in stats], hip.grads(), hip.params(), adam.m_states,
                     adam.v_states))
        tr.close()
        hip.close()
    a, b = runs
    assert a[0] == b[0]
    for x, y in zip(a[1:], b[1:]):
        assert x.keys() == y.keys()
        for k in x:
            assert np.array_equal(np.asarray(x[k]).view(np.uint32), np.asarray(y[k]).view(np.uint32)), k


def test_head_on_supervised_rows_changes_no_bit(ctx):
    """The step runs the final norm, the vocabulary head and the loss on the supervised positions only; with
    `head_all_rows` it runs them on every position as the reference does. Losses, gradients, weights after
    two steps and the evaluation loss agree to the bit, with ragged masks and a sequence without any target."""
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig, Trainer
    rng = np.random.default_rng(8)
    B, S = 4, 64
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = (rng.random((B, S)) > 0.4).astype(np.uint8)
    masks[1, :] = 0                      # a sequence with nothing to learn from
    masks[2, :40] = 0                    # a long prompt
    targets[3, 5] = 100000               # out of vocabulary: not supervised either
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    out = []
    for all_rows in (False, True):
        cfg = ModelConfig(vocab_size=256, hidden_size=192, intermediate_size=256, num_hidden_layers=2,
                          num_attention_heads=3, num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=100000.0,
                          tie_word_embeddings=True, f16_linears=True, head_all_rows=all_rows)
        hip, _ = build_pair(ctx, cfg, mods, rank=8, alpha=16.0, seed=52)
        tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0, grad_accum_steps=B)
        stats = [tr.train_chunk(rows, targets, masks) for _ in range(2)]
        seqs = [(list(r), list(t_), list(m)) for r, t_, m in zip(rows, targets, masks)]
        out.append(([(s.loss, s.grad_norm, s.tokens) for s in stats], hip.evaluate(seqs), hip.grads(),
                    hip.params()))
        tr.close()
        hip.close()
    a, b = out
    assert a[0] == b[0] and a[1] == b[1]
    for x, y in zip(a[2:], b[2:]):
        for k in x:
            assert np.array_equal(x[k].view(np.uint32), y[k].view(np.uint32)), k


def test_evaluate_is_the_token_weighted_forward_loss(ctx):
    """`evaluate` (ferrotensor-cli/src/main.rs:1110-1137): sum(loss_i * n_i) / sum(n_i) over ragged
    examples, forward only: parameters and gradients are untouched."""
    from ferrotensor_amd.data import TrainingExample
    cfg = tiny_config(True, True)
    hip, orc = build_pair(ctx, cfg, ["q_proj", "v_proj"], rank=4, alpha=8.0, seed=27)
    rng = np.random.default_rng(3)
    examples = [TrainingExample.from_sft_prompt_response(rng.integers(0, 256, p).tolist(),
                                                         rng.integers(0, 256, r).tolist())
                for p, r in [(5, 9), (12, 3), (1, 30), (20, 20), (7, 1)]]
    examples.append(TrainingExample([1, 2, 3], [2, 3, 4], [0, 0, 0]))       # nothing supervised
    before = hip.params()
    loss, tokens = hip.evaluate([e.as_tuple() for e in examples], batch=4)
    want_sum, want_tokens = 0.0, 0
    for e in examples:
        if not any(e.loss_mask):
            continue
        logits, _ = orc.forward(np.array([e.input_ids], np.uint32))
        res = rs.masked_cross_entropy_batch(logits, np.array([e.target_ids], np.uint32),
                                            np.array([e.loss_mask], np.uint8), 1)
        (mean, n), = res[1]
        want_sum += float(mean) * n
        want_tokens += n
    assert tokens == want_tokens == sum(sum(e.loss_mask) for e in examples)
    assert_close("eval loss", [loss], [want_sum / want_tokens])
    after = hip.params()
    for n in before:
        np.testing.assert_array_equal(before[n], after[n])
    assert hip.evaluate([examples[-1].as_tuple()])[1] == 0


@pytest.mark.parametrize("checkpoint", [False, True])
def test_head_dim_64_step_matches_oracle(ctx, checkpoint):
    """Head dim 64 takes the fused paths of the 360M shape (RoPE in the q/k projection epilogue, inverse
    RoPE in the attention backward kernels, LDS attention kernels, fused MLP halves): gradients and two
    optimizer steps against the oracle."""
    from ferrotensor_amd.trainer import ModelConfig, Trainer
    cfg = ModelConfig(vocab_size=256, hidden_size=192, intermediate_size=256, num_hidden_layers=2,
                      num_attention_heads=3, num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=100000.0,
                      tie_word_embeddings=True, f16_linears=True, checkpoint_blocks=checkpoint)
    hip, orc = build_pair(ctx, cfg, ["q_proj", "k_proj", "v_proj", "o_proj"], rank=8, alpha=16.0, seed=31)
    rng = np.random.default_rng(4)
    B, S = 2, 64
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((B, S), np.uint8)
    masks[:, :9] = 0
    want_logits, _ = orc.forward(rows)
    assert_close("logits", hip.forward_batch(rows), want_logits)
    tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.0)
    for step in range(2):
        tr.train_chunk(rows, targets, masks, apply=False)
        grads = hip.grads()
        want_stats, _, want_grads = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0,
                                                   return_grads=True)
        cs = want_stats.clip_scale or 1.0
        for n in grads:
            assert_close(f"step {step} grad {n}", grads[n], want_grads[n] / np.float32(cs))
        st = tr.train_chunk(rows, targets, masks)
        assert_close("loss", [st.loss], [want_stats.loss])
        assert_close("grad_norm", [st.grad_norm], [want_stats.grad_norm])
        params = hip.params()
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)


@pytest.mark.parametrize("checkpoint", [False, True])
def test_135m_width_step_matches_oracle(ctx, checkpoint):
    """Hidden 576 at 8 x 256 tokens: every 576-column product has 288 output tiles, a few more than the GPU has
    CUs, so its last tiles are shared out along K and their shares are added by the norm kernel that reads the
    product next (forward: o and down projections; backward: both grouped input gradients) or by the reduce
    kernel (o projection's input gradient). Logits, gradients and one optimizer step against the oracle, also
    with the blocks' forward recomputed in the backward pass."""
    from ferrotensor_amd.trainer import ModelConfig, Trainer
    cfg = ModelConfig(vocab_size=256, hidden_size=576, intermediate_size=1536, num_hidden_layers=2,
                      num_attention_heads=9, num_key_value_heads=3, rms_norm_eps=1e-5, rope_theta=100000.0,
                      tie_word_embeddings=True, f16_linears=True, checkpoint_blocks=checkpoint)
    hip, orc = build_pair(ctx, cfg, ["q_proj", "k_proj", "v_proj", "o_proj"], rank=8, alpha=16.0, seed=77)
    rng = np.random.default_rng(8)
    B, S = 8, 256
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((B, S), np.uint8)
    masks[:, :40] = 0
    want_logits, _ = orc.forward(rows)
    assert_close("logits", hip.forward_batch(rows), want_logits)
    tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.0)
    tr.train_chunk(rows, targets, masks, apply=False)
    grads = hip.grads()
    want_stats, _, want_grads = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0, return_grads=True)
    cs = want_stats.clip_scale or 1.0
    for n in grads:
        assert_close(f"grad {n}", grads[n], want_grads[n] / np.float32(cs))
    before = hip.params()
    st = tr.train_chunk(rows, targets, masks)
    assert_close("loss", [st.loss], [want_stats.loss])
    assert_close("grad_norm", [st.grad_norm], [want_stats.grad_norm])
    params = hip.params()
    # AdamW's first step moves a weight by lr * g / (|g| + 1e-8). Where the (clipped) gradient is above 3e-7 that
    # is +-lr to within 3 %, whatever the rounding of g: compared as tightly as in the other tests. Below it
    # (a handful of the 4608 elements of a factor) rounding noise of 1e-10 in g moves the step by up to
    # lr * 1e-10 / 1e-8, so only the size of the step is checked there.
    for n, w in orc.lora_params():
        firm = np.abs(want_grads[n]).reshape(-1) > 3e-7
        assert firm.mean() > 0.95, n
        assert_close(f"weight {n}", params[n].reshape(-1)[firm], w.reshape(-1)[firm], atol=1e-6, rtol=1e-4)
        assert np.all(np.abs(params[n] - before[n]).reshape(-1)[~firm] <= 1.001e-3), n


def _with_biases(tensors, which, seed):
    rng = np.random.default_rng(seed)
    out = dict(tensors)
    for name, w in tensors.items():
        if any(name.endswith(m + ".weight") for m in which):
            out[name[:-len(".weight")] + ".bias"] = (rng.standard_normal(w.shape[0]) * 0.1).astype(np.float32)
    return out


@pytest.mark.parametrize("head_dim_64", [False, True])
def test_biased_projections_step_matches_oracle(ctx, head_dim_64):
    """Qwen2-style `q/k/v_proj.bias` (Linear::project_2d, graph/src/lib.rs:128-139): logits, adapter gradients
    and two optimizer steps against the oracle. With head dim 64 the unbiased model rotates q and k in the
    GEMM epilogue; the biased one must add the bias first and rotate afterwards."""
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig, Trainer
    if head_dim_64:
        cfg = ModelConfig(vocab_size=256, hidden_size=192, intermediate_size=256, num_hidden_layers=2,
                          num_attention_heads=3, num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=100000.0,
                          tie_word_embeddings=True, f16_linears=True)
    else:
        cfg = tiny_config(False, False)
    tensors = _with_biases(random_model_tensors(cfg, 41), ("q_proj", "k_proj", "v_proj"), 42)
    assert sum(k.endswith(".bias") for k in tensors) == 3 * cfg.num_hidden_layers
    hip = Lfm2Model(ctx, cfg)
    hip.load_tensors(tensors)
    ocfg = rs.ModelConfig(cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers,
                          cfg.num_attention_heads, cfg.num_key_value_heads, cfg.rms_norm_eps, cfg.rope_theta,
                          cfg.tie_word_embeddings)
    orc = rs.Model.from_hf_tensors(ocfg, tensors, f16_linears=cfg.f16_linears)
    plain = rs.Model.from_hf_tensors(ocfg, {k: v for k, v in tensors.items() if not k.endswith(".bias")},
                                     f16_linears=cfg.f16_linears)
    rng = np.random.default_rng(43)
    for name in hip.linear_prefixes(["q_proj", "k_proj", "v_proj", "o_proj"]):
        i, o = hip.linear_dims(name)
        a = (rng.standard_normal((i, 8)) * 0.02).astype(np.float32)
        b = (rng.standard_normal((8, o)) * 0.02).astype(np.float32)
        hip.set_lora(name, a, b, 16.0)
        orc.set_lora(name, a, b, 16.0)
        plain.set_lora(name, a, b, 16.0)
    B, S = 2, 64
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rows[:, :1]], axis=1)
    masks = np.ones((B, S), np.uint8)
    masks[:, :5] = 0
    want_logits, _ = orc.forward(rows)
    got_logits = hip.forward_batch(rows)
    assert_close("logits", got_logits, want_logits)
    # the biases matter at this tolerance: the same model without them is far off
    assert np.abs(plain.forward(rows)[0] - want_logits).max() > 100 * 1e-4
    tr = Trainer(hip, lr=1e-3, weight_decay=0.0, clip_grad_norm=1.0)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.0)
    for step in range(2):
        tr.train_chunk(rows, targets, masks, apply=False)
        grads = hip.grads()
        assert not any(n.endswith(".bias") for n in grads)   # frozen with the base
        want_stats, _, want_grads = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=1.0,
                                                   return_grads=True)
        cs = want_stats.clip_scale or 1.0
        for n in grads:
            assert_close(f"step {step} grad {n}", grads[n], want_grads[n] / np.float32(cs))
        st = tr.train_chunk(rows, targets, masks)
        assert_close("loss", [st.loss], [want_stats.loss])
        assert_close("grad_norm", [st.grad_norm], [want_stats.grad_norm])
        params = hip.params()
        for n, w in orc.lora_params():
            assert_close(f"step {step} weight {n}", params[n], w, atol=1e-6, rtol=1e-4)


def test_model_directory_with_biases_loads_them(ctx, fx, golden_dir, tmp_path):
    """`load_model` on a directory whose q/k/v projections have `.bias` tensors (build_linear,
    model_builder.rs:454-469): the logits are the oracle's for the biased model; a bias of the wrong length
    is refused."""
    import os
    import shutil
    from ferrotensor_amd import checkpoint as ck
    from ferrotensor_amd import loader
    from ferrotensor_amd._lib import FtError
    tensors = _with_biases(fx.model, ("q_proj", "k_proj", "v_proj"), 9)
    d = tmp_path / "biased"
    d.mkdir()
    shutil.copy(os.path.join(golden_dir, "gradient_parity", "config.json"), d / "config.json")
    ck.write_safetensors(str(d / "model.safetensors"), tensors, {})
    model = loader.load_model(ctx, str(d), f16_linears=False)
    rows = fx.case("batch")[0]
    want, _ = rs.Model.from_hf_tensors(fx.config, tensors).forward(rows)
    assert worst_ratio(model.forward_batch(rows), want) <= 1.0
    plain, _ = rs.Model.from_hf_tensors(fx.config, fx.model).forward(rows)
    assert worst_ratio(plain, want) > 10.0
    bad = dict(tensors)
    bad["model.layers.0.self_attn.k_proj.bias"] = np.zeros(7, np.float32)
    d2 = tmp_path / "bad"
    d2.mkdir()
    shutil.copy(os.path.join(golden_dir, "gradient_parity", "config.json"), d2 / "config.json")
    ck.write_safetensors(str(d2 / "model.safetensors"), bad, {})
    with pytest.raises(FtError, match="k_proj.bias must be"):
        loader.load_model(ctx, str(d2), f16_linears=False)


def test_trainable_biases_on_every_linear_match_oracle(ctx, fx):
    """Every linear biased (lm_head too) and the base trainable: the bias gradients (ones^T @ dy) and all the
    others against the oracle, accumulated over two micro-batches, then one optimizer step moves the biases.
    Parameter order within a linear is weight, bias, adapter (Linear::params, graph/src/lib.rs:180-188)."""
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig, Trainer
    c = fx.config
    every = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj", "lm_head")
    tensors = _with_biases(fx.model, every, 3)
    cfg = ModelConfig(c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers,
                      c.num_attention_heads, c.num_key_value_heads, c.rms_norm_eps, c.rope_theta,
                      c.tie_word_embeddings, False, trainable_base=True)
    hip = Lfm2Model(ctx, cfg)
    hip.load_tensors(tensors)
    orc = rs.Model.from_hf_tensors(c, tensors)
    for name in hip.linear_prefixes(list(every)):
        hip.set_lora(name, fx.adapters[name + ".lora_a"], fx.adapters[name + ".lora_b"], fx.meta["lora_alpha"])
        orc.set_lora(name, fx.adapters[name + ".lora_a"], fx.adapters[name + ".lora_b"], fx.meta["lora_alpha"])
    rows, targets, masks, _, _ = fx.case("full")
    logits, cache = orc.forward(rows, trainable_base=True)
    loss, _, grad_logits = rs.masked_cross_entropy_batch(logits, targets, masks, rows.shape[0])
    want = orc.backward(grad_logits, cache)
    assert len(want) == 65
    tr = Trainer(hip, lr=1e-3, weight_decay=0.0, grad_accum_steps=1)
    st = tr.train_chunk(rows, targets, masks, apply=False)
    grads = hip.grads()
    assert set(grads) == set(want)
    names = list(grads)
    i = names.index("model.layers.0.self_attn.q_proj.weight")
    assert names[i + 1:i + 4] == ["model.layers.0.self_attn.q_proj.bias", "model.layers.0.self_attn.q_proj.lora_a",
                                  "model.layers.0.self_attn.q_proj.lora_b"]
    assert worst_ratio([st.loss], [loss]) <= 1.0
    for n in want:
        assert worst_ratio(grads[n], want[n]) <= 1.0, n
    # two one-sequence micro-batches accumulate to half the two-sequence gradients (seed 1/2 each)
    hip2 = Lfm2Model(ctx, cfg)
    hip2.load_tensors(tensors)
    for name in hip2.linear_prefixes(list(every)):
        hip2.set_lora(name, fx.adapters[name + ".lora_a"], fx.adapters[name + ".lora_b"], fx.meta["lora_alpha"])
    tr2 = Trainer(hip2, lr=1e-3, weight_decay=0.0, grad_accum_steps=2)
    assert not tr2.train_chunk(rows[:1], targets[:1], masks[:1]).optimizer_step
    tr2.train_chunk(rows[1:], targets[1:], masks[1:], apply=False)
    parts = hip2.grads()
    for n in want:
        if n.endswith(".bias"):
            assert worst_ratio(parts[n], want[n] * np.float32(0.5)) <= 1.0, n
    before = hip.params()
    assert tr.train_chunk(rows, targets, masks).optimizer_step
    after = hip.params()
    assert all(not np.array_equal(before[n], after[n]) for n in want if n.endswith(".bias"))


def test_targets_masking_is_bit_exact_against_oracle(ctx):
    """Skipped rows (mask 0 or target >= vocab) contribute exactly nothing:
    the loss equals the oracle's and flipping masked targets changes no bit."""
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config()
    hip, _ = build_pair(ctx, cfg, ["q_proj", "v_proj"], rank=4, alpha=8.0, seed=3)
    rng = np.random.default_rng(9)
    rows = rng.integers(0, 256, (2, 32)).astype(np.uint32)
    targets = rng.integers(0, 256, (2, 32)).astype(np.uint32)
    masks = (rng.random((2, 32)) > 0.5).astype(np.uint8)
    targets[0, 5] = 70000  # out of vocabulary: skipped even with mask 1
    masks[0, 5] = 1
    tr = Trainer(hip, lr=1e-3)
    a = tr.train_chunk(rows, targets, masks, apply=False)
    ga = hip.grads()
    t2 = targets.copy()
    t2[masks == 0] = (t2[masks == 0] + 17) % 256
    b = tr.train_chunk(rows, t2, masks, apply=False)
    gb = hip.grads()
    assert a.loss == b.loss and a.tokens == b.tokens == int(masks.sum()) - 1
    for n in ga:
        np.testing.assert_array_equal(ga[n], gb[n])


def test_out_of_range_token_embeds_as_zero_row(ctx):
    cfg = tiny_config()
    hip, orc = build_pair(ctx, cfg, ["q_proj"], rank=4, alpha=8.0, seed=4)
    rows = np.array([[1, 2, 999, 4, 5, 6, 7, 8]], np.uint32)
    want, _ = orc.forward(rows)
    assert_close("logits", hip.forward_batch(rows), want)


# ---- the step composed of the 1:1 ComputeEngine entry points, in the reference's op order ----

@pytest.mark.parametrize("f16", [False, True])
def test_engine_ops_step_matches_the_oracle_and_the_fused_driver(ctx, f16):
    """`ferrotensor_amd.engine_step`: the same step issued op by op as ferrotensor-autograd would (project_2d's
    six calls per linear, copy + scale, copy + rope, one sum_squares / clip / adamw call per tensor) gives the
    oracle's loss, gradient norm, clip and post-step weights, i.e. what the fused driver gives."""
    from ferrotensor_amd.engine_step import EngineOpsModel, EngineOpsTrainer
    from ferrotensor_amd.trainer import Trainer
    cfg = tiny_config(f16, tied=True)
    mods = ["q_proj", "k_proj", "v_proj", "o_proj"]
    hip, orc = build_pair(ctx, cfg, mods, rank=4, alpha=8.0, seed=21)
    eo = EngineOpsModel(ctx, cfg, random_model_tensors(cfg, 21))
    frng = np.random.default_rng(22)          # the factors build_pair drew (seed + 1, same order)
    prefixes = hip.linear_prefixes(mods)
    for name in prefixes:
        i, o = hip.linear_dims(name)
        a = (frng.standard_normal((i, 4)) * 0.02).astype(np.float32)
        b = (frng.standard_normal((4, o)) * 0.02).astype(np.float32)
        parts = name.split(".")      # model.layers.N.self_attn.q_proj
        eo.set_lora(int(parts[2]), parts[-1], a, b, 8.0)
    rng = np.random.default_rng(6)
    B, S = 2, 32
    rows = rng.integers(0, 256, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rng.integers(0, 256, (B, 1)).astype(np.uint32)], axis=1)
    masks = np.ones((B, S), np.uint8)
    masks[0, :5] = 0
    masks[1, :9] = 0
    tr = Trainer(hip, lr=1e-3, weight_decay=0.01, clip_grad_norm=0.01)
    et = EngineOpsTrainer(eo, lr=1e-3, weight_decay=0.01, clip_grad_norm=0.01)
    opt = rs.AdamW(lr=1e-3, weight_decay=0.01)
    for step in range(2):
        want = rs.train_chunk(orc, opt, rows, targets, masks, clip_grad_norm=0.01)
        st = tr.train_chunk(rows, targets, masks)
        loss, norm, clip = et.train_chunk(rows, targets, masks)
        assert want.clip_scale is not None and clip is not None
        assert_close("loss", [loss], [want.loss])
        assert_close("grad norm", [norm], [want.grad_norm])
        assert_close("clip scale", [clip], [want.clip_scale], atol=1e-6)
        assert_close("loss (fused)", [st.loss], [loss])
        for n, w in orc.lora_params():
            parts = n.split(".")     # model.layers.N.self_attn.q_proj.lora_a
            lo = eo.layers[int(parts[2])][parts[4]].lora
            got = (lo.a if parts[-1] == "lora_a" else lo.b).to_numpy()
            assert_close(f"step {step} weight {n}", got.reshape(-1), w.reshape(-1), atol=1e-6, rtol=1e-4)
    assert et.calls > 200     # op by op: hundreds of engine calls where the fused driver makes a few dozen launches

