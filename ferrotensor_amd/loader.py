"""A Hugging Face model directory (config.json + safetensors) -> a resident `Lfm2Model`.

Follows `Lfm2Config` (ferrotensor-loader/src/lib.rs:74-142), `check_supported`
(ferrotensor-graph/src/model_builder.rs:186-222) and `Lfm2ModelBuilder::build`
(model_builder.rs:400-424, 505-550, 623-709) for Llama-style checkpoints: the
builder's transpose / f16 / tied-head rules themselves live in the library
(`ft_model_set_tensor`); this module reads the files and refuses what the step
does not compute. Tensors are read through a memory map, one at a time.
"""
import json
import os
import struct
from typing import Dict, Iterator, List, Optional, Tuple

import numpy as np

from .trainer import Lfm2Model, ModelConfig


class BuildError(ValueError):
    """`BuildError` of the reference's builder: the message names the field or tensor."""


def _rust_str(s: str) -> str:
    """`{:?}` of a Rust &str for the plain names that occur in configs."""
    return '"%s"' % s.replace("\\", "\\\\").replace('"', '\\"')


def check_supported(config: dict):
    """Refuses a config that asks for something the forward pass does not compute, with the
    reference's messages (model_builder.rs:186-222)."""
    act = config.get("hidden_act")
    if act is not None and act not in ("silu", "swish"):
        raise BuildError("hidden_act %s is not supported: the MLP computes SiLU (silu) only" % _rust_str(act))
    for field in ("rope_scaling", "rope_parameters"):
        rope = config.get(field)
        if rope is None:
            continue
        kind = rope.get("rope_type") or rope.get("type")
        if kind is None:
            kind = "default" if rope.get("factor") is None else "unnamed"
        if kind != "default":
            raise BuildError("%s type %s is not supported: RoPE runs unscaled" % (field, _rust_str(kind)))
    if config.get("use_sliding_window") is True:
        window = config.get("sliding_window")
        raise BuildError("sliding_window %s is not supported: attention always covers the whole sequence"
                         % ("unset" if window is None else window))


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def model_config(config: dict, tied: bool, f16_linears: bool = True, checkpoint_blocks: bool = False) -> ModelConfig:
    """`Lfm2Config` defaults: rms_norm_eps (alias norm_eps) 1e-5, kv heads = heads, RoPE base from
    rope_theta, else rope_parameters.rope_theta, else 10000 (model_builder.rs:541-546)."""
    check_supported(config)
    if (config.get("model_type") or "").lower() == "lfm2" or "conv" in (config.get("layer_types") or []):
        raise BuildError("LFM2 (convolution) blocks are not supported: Llama-style attention models only")
    heads = int(config["num_attention_heads"])
    kv = int(config.get("num_key_value_heads") or heads)
    hidden = int(config["hidden_size"])
    if heads == 0 or kv == 0 or heads % kv != 0:
        raise BuildError("num_attention_heads (%d) must be a positive multiple of num_key_value_heads (%d)"
                         % (heads, kv))
    head_dim = int(config.get("head_dim") or hidden // max(heads, 1))
    if head_dim > 128 or head_dim % 2 != 0:
        raise BuildError("head_dim %d is not supported (RoPE needs an even size, and the attention kernel "
                         "handles at most 128)" % head_dim)
    if head_dim * heads != hidden:
        raise BuildError("head_dim %d with %d heads does not match hidden_size %d" % (head_dim, heads, hidden))
    theta = config.get("rope_theta")
    if theta is None:
        theta = (config.get("rope_parameters") or {}).get("rope_theta")
    eps = config.get("rms_norm_eps", config.get("norm_eps", 1e-5))
    return ModelConfig(vocab_size=int(config["vocab_size"]), hidden_size=hidden,
                       intermediate_size=int(config["intermediate_size"]),
                       num_hidden_layers=int(config["num_hidden_layers"]), num_attention_heads=heads,
                       num_key_value_heads=kv, rms_norm_eps=float(eps), rope_theta=float(theta or 10000.0),
                       tie_word_embeddings=tied, f16_linears=f16_linears, checkpoint_blocks=checkpoint_blocks)


class SafetensorsFile:
    """Header of one safetensors file + lazy, memory-mapped access to its tensors as f32."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise BuildError("%s is not a safetensors file: too short" % path)
            (n,) = struct.unpack("<Q", head)
            if n > os.path.getsize(path) - 8:
                raise BuildError("%s is not a safetensors file: header length %d exceeds the file" % (path, n))
            try:
                self.header = json.loads(f.read(n).decode())
            except (UnicodeDecodeError, json.JSONDecodeError) as e:
                raise BuildError("%s is not a safetensors file: %s" % (path, e))
        self.metadata = self.header.pop("__metadata__", None) or {}
        self._base = 8 + n
        self._map = None

    def names(self) -> List[str]:
        return list(self.header)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.header[name]["shape"])

    def read(self, name: str) -> np.ndarray:
        info = self.header[name]
        if self._map is None:
            self._map = np.memmap(self.path, dtype=np.uint8, mode="r")
        b, e = info["data_offsets"]
        raw = self._map[self._base + b:self._base + e]
        dt = info["dtype"]
        if dt == "F32":
            a = raw.view("<f4").astype(np.float32)
        elif dt == "F16":
            a = raw.view("<f2").astype(np.float32)
        elif dt == "BF16":
            a = (raw.view("<u2").astype(np.uint32) << 16).view(np.float32)
        else:
            raise BuildError("%s in %s has dtype %s; F32, F16 or BF16 expected" % (name, self.path, dt))
        return np.ascontiguousarray(a).reshape(self.shape(name))


class WeightsContext:
    """`WeightsContext` of the reference loader: `model.safetensors`, or the shards listed in
    `model.safetensors.index.json`."""

    def __init__(self, model_dir: str):
        self.files: Dict[str, SafetensorsFile] = {}
        self.where: Dict[str, str] = {}
        index = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.exists(index):
            with open(index) as f:
                weight_map = json.load(f)["weight_map"]
            for name, shard in weight_map.items():
                if shard not in self.files:
                    self.files[shard] = SafetensorsFile(os.path.join(model_dir, shard))
                self.where[name] = shard
        else:
            single = os.path.join(model_dir, "model.safetensors")
            if not os.path.exists(single):
                raise BuildError("%s holds neither model.safetensors nor model.safetensors.index.json" % model_dir)
            self.files["model.safetensors"] = SafetensorsFile(single)
            for name in self.files["model.safetensors"].names():
                self.where[name] = "model.safetensors"

    def has(self, name: str) -> bool:
        return name in self.where

    def names(self) -> List[str]:
        return list(self.where)

    def read(self, name: str) -> np.ndarray:
        if name not in self.where:
            raise BuildError("the checkpoint has no tensor %s" % name)
        return self.files[self.where[name]].read(name)


_PROJ = (("self_attn", ("q_proj", "k_proj", "v_proj", "o_proj")), ("mlp", ("gate_proj", "up_proj", "down_proj")))


def expected_tensors(cfg: ModelConfig, tied: bool) -> List[str]:
    names = ["model.embed_tokens.weight", "model.norm.weight"]
    for l in range(cfg.num_hidden_layers):
        p = "model.layers.%d" % l
        names += [p + ".input_layernorm.weight", p + ".post_attention_layernorm.weight"]
        for sub, mods in _PROJ:
            names += ["%s.%s.%s.weight" % (p, sub, m) for m in mods]
    if not tied:
        names.append("lm_head.weight")
    return names


def load_model(ctx, model_dir: str, f16_linears: bool = True, checkpoint_blocks: bool = False) -> Lfm2Model:
    """The frozen base model of `model_dir`, resident on the GPU. The head is tied to the embedding
    when the checkpoint has no `lm_head.weight` (model_builder.rs:652-689)."""
    config = read_config(model_dir)
    weights = WeightsContext(model_dir)
    tied = not weights.has("lm_head.weight")
    cfg = model_config(config, tied, f16_linears, checkpoint_blocks)
    for l in range(cfg.num_hidden_layers):
        p = "model.layers.%d.self_attn." % l
        for unsupported in ("q_norm.weight", "k_norm.weight", "q_layernorm.weight"):
            if weights.has(p + unsupported):
                raise BuildError("%s%s: per-head norms are not supported" % (p, unsupported))
    model = Lfm2Model(ctx, cfg)
    try:
        for name in expected_tensors(cfg, tied):
            model.set_tensor(name, weights.read(name))
            # build_linear (model_builder.rs:454-469): a projection with a `<prefix>.bias` tensor gets it
            bias = name[:-len(".weight")] + ".bias"
            if ("_proj." in name or name == "lm_head.weight") and weights.has(bias):
                model.set_tensor(bias, weights.read(bias))
    except Exception:
        model.close()
        raise
    return model


def iter_weights(model_dir: str) -> Iterator[Tuple[str, np.ndarray]]:
    """(name, f32 array) for every tensor of the checkpoint, one at a time."""
    weights = WeightsContext(model_dir)
    for name in weights.names():
        yield name, weights.read(name)
