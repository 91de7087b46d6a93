"""Hugging Face directory loader: config rules pinned by the reference's own config vectors
(ferrotensor-graph/src/model_builder.rs:770-868), tensor access against the `safetensors` library."""
import copy
import json
import os

import numpy as np
import pytest

from ferrotensor_amd import loader

# The `config.json` of Qwen2.5-0.5B, as in the reference's tests (model_builder.rs:771-796).
QWEN = {"architectures": ["Qwen2ForCausalLM"], "attention_dropout": 0.0, "bos_token_id": 151643,
        "eos_token_id": 151643, "hidden_act": "silu", "hidden_size": 896, "initializer_range": 0.02,
        "intermediate_size": 4864, "max_position_embeddings": 32768, "max_window_layers": 24, "model_type": "qwen2",
        "num_attention_heads": 14, "num_hidden_layers": 24, "num_key_value_heads": 2, "rms_norm_eps": 1e-06,
        "rope_theta": 1000000.0, "sliding_window": 32768, "tie_word_embeddings": True, "torch_dtype": "bfloat16",
        "use_cache": True, "use_sliding_window": False, "vocab_size": 151936}


def with_changes(changes):
    c = copy.deepcopy(QWEN)
    c.update(changes)
    return c


@pytest.mark.parametrize("changes", [
    {},
    {"rope_theta": None, "rope_parameters": {"rope_type": "default", "rope_theta": 1000000.0}},
    {"use_sliding_window": None, "sliding_window": 4096},
    {"rope_scaling": {"rope_theta": 1000000.0}},
])
def test_supported_configs(changes):
    """`qwen2_5_config_is_supported` (model_builder.rs:808-831)."""
    loader.check_supported(with_changes(changes))
    cfg = loader.model_config(with_changes(changes), tied=True)
    assert (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (896, 14, 2)
    assert cfg.rope_theta == 1000000.0 and cfg.rms_norm_eps == pytest.approx(1e-6)


@pytest.mark.parametrize("changes,message", [
    ({"hidden_act": "gelu_pytorch_tanh"},
     'hidden_act "gelu_pytorch_tanh" is not supported: the MLP computes SiLU (silu) only'),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}},
     'rope_scaling type "llama3" is not supported: RoPE runs unscaled'),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}},
     'rope_scaling type "linear" is not supported: RoPE runs unscaled'),
    ({"rope_parameters": {"rope_type": "yarn", "rope_theta": 1e6}},
     'rope_parameters type "yarn" is not supported: RoPE runs unscaled'),
    ({"use_sliding_window": True},
     "sliding_window 32768 is not supported: attention always covers the whole sequence"),
    ({"rope_scaling": {"factor": 4.0}}, 'rope_scaling type "unnamed" is not supported: RoPE runs unscaled'),
])
def test_unsupported_config_features_are_named(changes, message):
    """`unsupported_config_features_are_named` (model_builder.rs:833-868): same messages."""
    with pytest.raises(loader.BuildError) as e:
        loader.check_supported(with_changes(changes))
    assert str(e.value) == message


def test_config_defaults_and_head_rules():
    base = {"hidden_size": 64, "intermediate_size": 128, "num_attention_heads": 4, "num_hidden_layers": 2,
            "vocab_size": 100}
    cfg = loader.model_config(base, tied=False)
    assert cfg.num_key_value_heads == 4 and cfg.rms_norm_eps == pytest.approx(1e-5) and cfg.rope_theta == 10000.0
    assert loader.model_config(dict(base, norm_eps=1e-6), tied=False).rms_norm_eps == pytest.approx(1e-6)
    with pytest.raises(loader.BuildError, match="positive multiple"):
        loader.model_config(dict(base, num_key_value_heads=3), tied=False)
    with pytest.raises(loader.BuildError, match="head_dim 256 is not supported"):
        loader.model_config(dict(base, hidden_size=1024), tied=False)
    with pytest.raises(loader.BuildError, match="LFM2"):
        loader.model_config(dict(base, model_type="lfm2"), tied=False)


def test_reads_the_reference_fixture_directory(golden_dir):
    """The reference's own tiny Llama checkpoint (config.json + model.safetensors, 21 f32 tensors)."""
    from safetensors.numpy import load_file
    d = os.path.join(golden_dir, "gradient_parity")
    want = load_file(os.path.join(d, "model.safetensors"))
    w = loader.WeightsContext(d)
    assert sorted(w.names()) == sorted(want) and len(want) == 21
    for n in want:
        np.testing.assert_array_equal(w.read(n), want[n])
    cfg = loader.model_config(loader.read_config(d), tied=not w.has("lm_head.weight"))
    assert not cfg.tie_word_embeddings and cfg.rope_theta == 500.0 and cfg.rms_norm_eps == pytest.approx(1e-6)
    assert sorted(loader.expected_tensors(cfg, False)) == sorted(want)


def test_sharded_half_precision_checkpoint(tmp_path):
    import torch
    from safetensors.torch import save_file
    a, b, c = torch.randn(6, 4), torch.randn(4, 6), torch.randn(4)
    save_file({"model.embed_tokens.weight": a.to(torch.bfloat16)}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({"model.norm.weight": c.to(torch.float16), "lm_head.weight": b},
              str(tmp_path / "model-00002-of-00002.safetensors"))
    json.dump({"weight_map": {"model.embed_tokens.weight": "model-00001-of-00002.safetensors",
                              "model.norm.weight": "model-00002-of-00002.safetensors",
                              "lm_head.weight": "model-00002-of-00002.safetensors"}},
              open(tmp_path / "model.safetensors.index.json", "w"))
    w = loader.WeightsContext(str(tmp_path))
    np.testing.assert_array_equal(w.read("model.embed_tokens.weight"), a.to(torch.bfloat16).float().numpy())
    np.testing.assert_array_equal(w.read("model.norm.weight"), c.to(torch.float16).float().numpy())
    np.testing.assert_array_equal(w.read("lm_head.weight"), b.numpy())
    assert w.has("lm_head.weight") and not w.has("model.layers.0.mlp.up_proj.weight")
    with pytest.raises(loader.BuildError, match="no tensor"):
        w.read("nope")
    with pytest.raises(loader.BuildError, match="neither"):
        loader.WeightsContext(str(tmp_path / "missing"))
