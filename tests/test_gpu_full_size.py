"""The step at BASELINE.json's full sizes: the headline (SmolLM2-360M shape, 8 x 256, vocabulary 49152),
the 135M shape (576 hidden: the GEMM shapes that split K), and the 1.7B shape (2048 hidden, 32 heads
without grouping, rank 16 on all seven projections, block checkpointing, sequences of 1024 tokens) twice:
at its full depth of 24 layers and 8 x 1024 tokens, and cut to 4 layers and 2 x 1024 tokens.

The oracle finishes one sequence of the 360M / 135M models, and one 1024-token sequence of the 4-layer cut
of the 1.7B model, in seconds, so there one sequence is compared with it element by element (loss, gradient
norm, every LoRA gradient); every shape's full batch, the 24-layer 1.7B step included, is checked through
properties that do not depend on size: two runs agree to the bit, and one-sequence passes accumulate to
the batched step (loss, gradient norm and every gradient).
"""
import numpy as np
import pytest

import bench
from oracle import reference_step as rs
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu

SHAPES = {"360m": bench.WORKLOADS["360m"], "135m": bench.WORKLOADS["135m"],
          "1.7b-four-layers": dict(bench.WORKLOADS["1.7b"], layers=4, B=2),
          # 6.8 GB of f32 weights on the host: streamed to the device, not kept, and no oracle model
          "1.7b": dict(bench.WORKLOADS["1.7b"], oracle=False)}


ORACLE_SHAPES = [n for n, W in SHAPES.items() if W.get("oracle", True)]   # a prefix of SHAPES, in its order


@pytest.fixture(scope="module")
def world(request):
    from ferrotensor_amd import HipContext
    W = SHAPES[request.param]
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig
    ctx = HipContext(0)
    cfg = ModelConfig(vocab_size=W["vocab"], hidden_size=W["hidden"], intermediate_size=W["ffn"],
                      num_hidden_layers=W["layers"], num_attention_heads=W["heads"], num_key_value_heads=W["kv"],
                      rms_norm_eps=1e-5, rope_theta=100000.0, tie_word_embeddings=True, f16_linears=True,
                      checkpoint_blocks=bool(W.get("checkpoint", False)))
    model = Lfm2Model(ctx, cfg)
    if W.get("oracle", True):
        tensors = dict(bench.synthetic_tensors(W))
        model.load_tensors(tensors)
    else:
        tensors = None
        for name, value in bench.synthetic_tensors(W):
            model.set_tensor(name, value)
    factors = list(bench.lora_factors(model, W))
    yield ctx, model, tensors, factors, W
    model.close()
    ctx.close()


def reset_adapters(model, factors, W):
    for name, a, b in factors:
        model.set_lora(name, a, b, W["alpha"])


def run_step(model, factors, W, rows, targets, masks, micro):
    from ferrotensor_amd.trainer import Trainer
    reset_adapters(model, factors, W)
    tr = Trainer(model, lr=2e-4, weight_decay=0.0, clip_grad_norm=1.0, grad_accum_steps=len(rows))
    per_seq = []
    st = None
    for i in range(0, len(rows), micro):
        st = tr.train_chunk(rows[i:i + micro], targets[i:i + micro], masks[i:i + micro], apply=False)
        per_seq.append(st.loss)
    grads = model.grads()
    tr.close()
    return st, per_seq, grads


@pytest.mark.parametrize("world", list(SHAPES), indirect=True)
def test_full_size_batch_properties(world):
    ctx, model, _, factors, W = world
    rows, targets, masks = bench.synthetic_batch(W)
    st_a, _, g_a = run_step(model, factors, W, rows, targets, masks, micro=len(rows))
    st_b, _, g_b = run_step(model, factors, W, rows, targets, masks, micro=len(rows))
    assert np.isfinite(st_a.loss) and st_a.tokens == int(masks.sum())
    # determinism at the real shape: every reduction of the step has a fixed order
    assert (st_a.loss, st_a.grad_norm) == (st_b.loss, st_b.grad_norm)
    for k in g_a:
        assert np.array_equal(g_a[k].view(np.uint32), g_b[k].view(np.uint32)), k
    # eight one-sequence passes (split-K GEMMs, accumulated factor gradients) add up to the batched step
    st_c, per_seq, g_c = run_step(model, factors, W, rows, targets, masks, micro=1)
    assert_close("sum of the per-sequence losses", [sum(per_seq)], [st_a.loss])
    assert_close("grad norm", [st_c.grad_norm], [st_a.grad_norm])
    scale = max(float(np.abs(g).max()) for g in g_a.values())
    for k in g_a:
        # gradients of this model are ~1e-3 and smaller: the absolute term of the parity bar, scaled to them
        assert_close("accumulated " + k, g_c[k], g_a[k], atol=1e-4 * scale, rtol=1e-3)


@pytest.mark.parametrize("world", ORACLE_SHAPES, indirect=True)
def test_one_full_size_sequence_matches_the_oracle(world):
    ctx, model, tensors, factors, W = world
    cfg = rs.ModelConfig(W["vocab"], W["hidden"], W["ffn"], W["layers"], W["heads"], W["kv"], 1e-5, 100000.0, True)
    orc = rs.Model.from_hf_tensors(cfg, tensors, f16_linears=True)
    for name, a, b in factors:
        orc.set_lora(name, a, b, W["alpha"])
    rows, targets, masks = bench.synthetic_batch(W, B=1)
    st, _, grads = run_step(model, factors, W, rows, targets, masks, micro=1)
    want_stats, _, want_grads = rs.train_chunk(orc, rs.AdamW(lr=2e-4, weight_decay=0.0), rows, targets, masks,
                                               grad_accum_steps=1, clip_grad_norm=1.0, return_grads=True)
    clip = np.float32(want_stats.clip_scale or 1.0)   # the oracle hands back the clipped gradients
    assert_close("loss", [st.loss], [want_stats.loss])
    assert_close("grad norm", [st.grad_norm], [want_stats.grad_norm])
    scale = max(float(np.abs(g).max()) for g in want_grads.values()) / float(clip)
    for k in grads:
        # gradients of this model are ~1e-2 and smaller: the absolute term of the parity bar, scaled to them
        assert_close("grad " + k, grads[k], want_grads[k] / clip, atol=1e-4 * scale, rtol=1e-3)
