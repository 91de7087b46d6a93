"""Adapter / optimizer-state files: the container, the names and the metadata the reference reads
(ferrotensor-trainer/src/checkpoint.rs). CPU only; the `safetensors` package is used here as the
independent reader / writer the files must interoperate with."""
import json
import os

import numpy as np
import pytest

from ferrotensor_amd import checkpoint as ck


def test_reads_the_reference_adapter_fixture_like_the_safetensors_library(golden_dir):
    from safetensors.numpy import load_file
    path = os.path.join(golden_dir, "gradient_parity", "adapters.safetensors")
    want = load_file(path)
    got, meta = ck.read_safetensors(path)
    assert sorted(got) == sorted(want) and len(got) == 30
    for n in want:
        np.testing.assert_array_equal(got[n], want[n])
        assert got[n].dtype == np.float32


def test_written_files_load_with_the_safetensors_library(tmp_path):
    from safetensors import safe_open
    from safetensors.numpy import load_file
    rng = np.random.default_rng(0)
    tensors = {"model.layers.0.self_attn.q_proj.lora_A.weight": rng.standard_normal((960, 8), dtype=np.float32),
               "model.layers.0.self_attn.q_proj.lora_B.weight": rng.standard_normal((8, 960), dtype=np.float32),
               "lm_head.lora_A.weight": rng.standard_normal((3, 1), dtype=np.float32),
               "empty": np.zeros((0, 4), np.float32)}
    meta = ck.LoraMetadata(8, 16.0, ["q_proj", "k_proj", "v_proj", "o_proj"])
    path = str(tmp_path / "adapter.safetensors")
    ck.write_safetensors(path, tensors, meta.to_map())
    assert not os.path.exists(path + ".tmp")
    back = load_file(path)
    assert sorted(back) == sorted(tensors)
    for n in tensors:
        np.testing.assert_array_equal(back[n], tensors[n])
    with safe_open(path, framework="numpy") as f:
        assert f.metadata() == {"format": "ferrotensor-lora", "rank": "8", "alpha": "16",
                                "target_modules": "q_proj,k_proj,v_proj,o_proj"}
    # header: 8-byte length, JSON padded to a multiple of 8, data right behind it
    raw = open(path, "rb").read()
    n = int.from_bytes(raw[:8], "little")
    assert n % 8 == 0 and json.loads(raw[8:8 + n])["empty"]["shape"] == [0, 4]
    got, m = ck.read_safetensors(path)
    assert ck.LoraMetadata.from_map(m) == meta
    for name in tensors:
        np.testing.assert_array_equal(got[name], tensors[name])


def test_f16_and_bf16_tensors_are_widened_exactly(tmp_path):
    import torch
    from safetensors.torch import save_file
    x = torch.randn(7, 5)
    path = str(tmp_path / "half.safetensors")
    save_file({"h": x.to(torch.float16), "b": x.to(torch.bfloat16), "f": x}, path)
    got, _ = ck.read_safetensors(path)
    np.testing.assert_array_equal(got["h"], x.to(torch.float16).float().numpy())
    np.testing.assert_array_equal(got["b"], x.to(torch.bfloat16).float().numpy())
    np.testing.assert_array_equal(got["f"], x.numpy())


def test_numbers_are_printed_the_way_rust_prints_f32():
    # `f32::to_string()`: shortest round-trip decimal, positional, integers without a fraction
    for value, text in [(16.0, "16"), (0.5, "0.5"), (3.0, "3"), (0.1, "0.1"), (1e-8, "0.00000001"),
                        (32.0, "32"), (2.5, "2.5"), (0.0, "0")]:
        assert ck.format_f32(value) == text
        assert np.float32(float(text)) == np.float32(value)


def test_metadata_round_trip_and_missing_fields():
    m = ck.LoraMetadata(4, 8.0, ["q_proj", "down_proj"])
    assert ck.LoraMetadata.from_map(m.to_map()) == m
    assert ck.LoraMetadata.from_map({"rank": "4"}) is None
    w = ck.LoraMetadata(0, 0.0, [], trained_modules="attn")
    assert w.to_map()["format"] == "ferrotensor-weights" and ck.LoraMetadata.from_map(w.to_map()) == w


def test_training_checkpoint_round_trip_and_step_mismatch(tmp_path):
    rng = np.random.default_rng(1)
    names = ["model.layers.0.self_attn.q_proj.lora_A.weight", "model.layers.0.self_attn.q_proj.lora_B.weight"]
    shapes = [(32, 4), (4, 32)]
    adam = ck.AdamWState(2e-4, 0.9, 0.999, 1e-8, 0.0, 7.0,
                         {n: rng.standard_normal(s, dtype=np.float32) for n, s in zip(names, shapes)},
                         {n: np.abs(rng.standard_normal(s, dtype=np.float32)) for n, s in zip(names, shapes)})
    state = ck.TrainingState(step=7, total_steps=100, lr=2e-4, batch_size=8, grad_accum_steps=8, sequence_length=256,
                             model_path="/models/a", seed=3)
    path = str(tmp_path / "run.state.json")
    ck.save_training_checkpoint(path, state, adam)
    assert ck.moments_path(path) == str(tmp_path / "run.state.safetensors") and os.path.exists(ck.moments_path(path))
    doc = json.load(open(path))
    assert set(doc) == {"training_state", "optimizer_state", "grad_scaler_state"}
    assert doc["optimizer_state"]["AdamW"]["m_states"][names[0]] == {"shape": [32, 4], "data": []}
    assert doc["training_state"]["step"] == 7 and doc["training_state"]["task"] == "sft"
    from safetensors import safe_open
    with safe_open(ck.moments_path(path), framework="numpy") as f:
        assert f.metadata() == {"format": "ferrotensor-adamw-moments", "step": "7", "t": "7"}
        assert sorted(f.keys()) == sorted(["m/" + n for n in names] + ["v/" + n for n in names])
    state2, adam2 = ck.load_training_checkpoint(path)
    assert state2 == state and adam2.t == 7.0
    for n in names:
        np.testing.assert_array_equal(adam2.m_states[n], adam.m_states[n])
        np.testing.assert_array_equal(adam2.v_states[n], adam.v_states[n])
    # a JSON from another step than the moments file: refuse to resume
    doc["training_state"]["step"] = 8
    json.dump(doc, open(path, "w"))
    with pytest.raises(ValueError, match="interrupted while saving"):
        ck.load_training_checkpoint(path)


def test_not_a_safetensors_file(tmp_path):
    p = tmp_path / "junk.safetensors"
    p.write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00not json at all!!")
    with pytest.raises(ValueError):
        ck.read_safetensors(str(p))
    p.write_bytes(b"abc")
    with pytest.raises(ValueError):
        ck.read_safetensors(str(p))
