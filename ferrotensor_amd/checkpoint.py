"""Adapter and training-state files, in the formats the reference reads and writes
(ferrotensor-trainer/src/checkpoint.rs).

  * adapter file (`save_lora_checkpoint`, checkpoint.rs:124-162): F32 safetensors,
    tensors `<prefix>.lora_A.weight` [in, r] and `<prefix>.lora_B.weight` [r, out]
    (`Linear::named_params`, ferrotensor-graph/src/lib.rs:190-205), metadata
    `format = ferrotensor-lora`, `rank`, `alpha`, `target_modules` (`LoraMetadata::to_map`,
    checkpoint.rs:71-87);
  * training checkpoint (`TrainingCheckpoint::save`, checkpoint.rs:442-480): pretty JSON
    with `training_state`, `optimizer_state = {"AdamW": {...}}` (moment shapes only) and
    `grad_scaler_state`, plus the moments in `<name>.safetensors` next to it
    (`write_moments`, checkpoint.rs:537-566): tensors `m/<param>` and `v/<param>`,
    metadata `format = ferrotensor-adamw-moments`, `step`, `t`.

The safetensors container is written and parsed here (8-byte little-endian header
length, JSON header padded with spaces to a multiple of 8, raw little-endian data), so
the package needs no third-party library; every file goes through a temporary name
and a rename, as in the reference.
"""
import ctypes as C
import json
import os
import struct
from dataclasses import asdict, dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np

from ._lib import check

LORA_FORMAT = "ferrotensor-lora"
MOMENTS_FORMAT = "ferrotensor-adamw-moments"


def format_f32(x: float) -> str:
    """Rust's `f32::to_string()`: the shortest decimal that round-trips, positional, no trailing `.0`."""
    v = np.float32(x)
    if not np.isfinite(v):
        return "NaN" if np.isnan(v) else ("inf" if v > 0 else "-inf")
    return np.format_float_positional(v, unique=True, trim="-")


# ---------------------------------------------------------------------------
# safetensors container
# ---------------------------------------------------------------------------

def write_safetensors(path: str, tensors: Dict[str, np.ndarray], metadata: Optional[Dict[str, str]] = None):
    """F32 tensors + string metadata -> `path` (through `<path>.tmp`)."""
    header = {}
    if metadata is not None:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blobs, offset = [], 0
    for name in sorted(tensors):
        a = np.ascontiguousarray(tensors[name], dtype="<f4")
        header[name] = {"dtype": "F32", "shape": list(a.shape), "data_offsets": [offset, offset + a.nbytes]}
        blobs.append(a.tobytes())
        offset += a.nbytes
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for b in blobs:
            f.write(b)
    os.replace(tmp, path)


def _bf16_to_f32(raw: np.ndarray) -> np.ndarray:
    return (raw.astype(np.uint32) << 16).view(np.float32)


def read_safetensors(path: str) -> Tuple[Dict[str, np.ndarray], Dict[str, str]]:
    """(tensors as f32 arrays, metadata). F32, F16 and BF16 tensors are accepted, as in
    `load_lora_checkpoint` (checkpoint.rs:166-214)."""
    with open(path, "rb") as f:
        data = f.read()
    if len(data) < 8:
        raise ValueError("%s is not a safetensors file: too short" % path)
    (n,) = struct.unpack("<Q", data[:8])
    if n > len(data) - 8:
        raise ValueError("%s is not a safetensors file: header length %d exceeds the file" % (path, n))
    try:
        header = json.loads(data[8:8 + n].decode())
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise ValueError("%s is not a safetensors file: %s" % (path, e))
    metadata = header.pop("__metadata__", None) or {}
    body = memoryview(data)[8 + n:]
    out = {}
    for name, info in header.items():
        b, e = info["data_offsets"]
        shape = tuple(info["shape"])
        count = int(np.prod(shape)) if shape else 1
        dt = info["dtype"]
        if dt == "F32":
            a = np.frombuffer(body[b:e], dtype="<f4")
        elif dt == "F16":
            a = np.frombuffer(body[b:e], dtype="<f2").astype(np.float32)
        elif dt == "BF16":
            a = _bf16_to_f32(np.frombuffer(body[b:e], dtype="<u2"))
        else:
            raise ValueError("tensor %s in %s has dtype %s; F32, F16 or BF16 expected" % (name, path, dt))
        if a.size != count:
            raise ValueError("tensor %s in %s holds %d values for shape %s" % (name, path, a.size, list(shape)))
        out[name] = np.array(a, dtype=np.float32).reshape(shape)
    return out, metadata


# ---------------------------------------------------------------------------
# adapter files
# ---------------------------------------------------------------------------

@dataclass
class LoraMetadata:
    """checkpoint.rs:40-54."""
    rank: int
    alpha: float
    target_modules: List[str]
    trained_modules: Optional[str] = None

    def to_map(self) -> Dict[str, str]:
        m = {"format": "ferrotensor-weights" if self.trained_modules else LORA_FORMAT, "rank": str(self.rank),
             "alpha": format_f32(self.alpha), "target_modules": ",".join(self.target_modules)}
        if self.trained_modules:
            m["trained_modules"] = self.trained_modules
        return m

    @staticmethod
    def from_map(m: Dict[str, str]) -> Optional["LoraMetadata"]:
        try:
            return LoraMetadata(int(m["rank"]), float(m["alpha"]),
                                [s for s in m["target_modules"].split(",") if s], m.get("trained_modules") or None)
        except (KeyError, ValueError):
            return None


@dataclass
class LoraCheckpoint:
    tensors: Dict[str, np.ndarray]
    metadata: Optional[LoraMetadata]


def file_name(param: str) -> str:
    """`<prefix>.lora_a` -> `<prefix>.lora_A.weight` (graph/src/lib.rs:198-199)."""
    if param.endswith(".lora_a"):
        return param[:-len(".lora_a")] + ".lora_A.weight"
    if param.endswith(".lora_b"):
        return param[:-len(".lora_b")] + ".lora_B.weight"
    return param


def _param_shapes(model) -> Dict[str, Tuple[int, ...]]:
    """Shapes as the reference keeps them: A [in, r], B [r, out]; with a trainable base a linear weight in
    its stored [in, out] layout and a norm scale as a vector."""
    shapes = {}
    for name, numel in model.named_params():
        prefix, kind = name.rsplit(".", 1)
        if kind in ("lora_a", "lora_b"):
            i, o = model.linear_dims(prefix)
            shapes[name] = (i, numel // i) if kind == "lora_a" else (numel // o, o)
        elif prefix.endswith("norm"):
            shapes[name] = (numel,)
        else:
            shapes[name] = tuple(model.linear_dims(prefix))
    return shapes


def save_lora_checkpoint(model, path: str, metadata: Optional[LoraMetadata] = None):
    """Every adapter tensor of `model` -> an adapter file the reference's `eval`, `chat` and `merge` load."""
    shapes = _param_shapes(model)
    tensors = {file_name(n): v.reshape(shapes[n]) for n, v in model.params().items()}
    write_safetensors(path, tensors, metadata.to_map() if metadata else None)


def load_lora_checkpoint(path: str) -> LoraCheckpoint:
    tensors, meta = read_safetensors(path)
    return LoraCheckpoint(tensors, LoraMetadata.from_map(meta) if meta else None)


def apply_lora_checkpoint(model, ckpt: LoraCheckpoint, alpha: Optional[float] = None) -> int:
    """Attaches every (lora_A, lora_B) pair of the file to the linear it names; returns the number
    of adapters set. `alpha` defaults to the file's metadata."""
    if alpha is None:
        if ckpt.metadata is None:
            raise ValueError("the adapter file has no metadata: pass alpha")
        alpha = ckpt.metadata.alpha
    n = 0
    for name, a in sorted(ckpt.tensors.items()):
        if not name.endswith(".lora_A.weight"):
            continue
        prefix = name[:-len(".lora_A.weight")]
        b = ckpt.tensors.get(prefix + ".lora_B.weight")
        if b is None:
            raise ValueError("%s has no matching lora_B" % name)
        i, o = model.linear_dims(prefix)
        if a.shape[0] != i or b.shape[1] != o or a.shape[1] != b.shape[0]:
            raise ValueError("%s: shapes %s / %s do not fit a [%d, %d] linear" % (prefix, a.shape, b.shape, i, o))
        model.set_lora(prefix, a, b, alpha)
        n += 1
    return n


LLAMA_RENAMES = ((".input_layernorm.", ".operator_norm."), (".post_attention_layernorm.", ".ffn_norm."),
                 (".mlp.", ".feed_forward."))


def legacy_llama_name(name: str) -> Optional[str]:
    """The name a Llama-block parameter had in older adapter files (graph/src/lfm.rs:232-255), or None."""
    if not name.startswith("model.layers."):
        return None
    for new, old in LLAMA_RENAMES:
        if new in name:
            return name.replace(new, old, 1)
    return None


def apply_checkpoint(ckpt: LoraCheckpoint, model) -> int:
    """`apply_checkpoint` (ferrotensor-trainer/src/checkpoint.rs:210-286): overwrites every trainable tensor of
    `model` with the tensor of the same name (or of its old Llama name) in the file, in place. Strict both
    ways: a tensor the file lacks, a shape that differs, or a tensor in the file that the model does not
    have (a different rank, other LoRA targets) is an error and nothing is written. Returns the count."""
    shapes = _param_shapes(model)
    params = [(file_name(name), tuple(shapes[name])) for name, _ in model.named_params()]
    sources = []
    for index, (name, shape) in sorted(enumerate(params), key=lambda e: e[1][0]):
        legacy = legacy_llama_name(name)
        if legacy is not None and legacy not in ckpt.tensors:
            legacy = None
        if name in ckpt.tensors and legacy is not None:
            raise ValueError("checkpoint has both %s and its old name %s" % (name, legacy))
        key = name if name in ckpt.tensors else legacy
        if key is None:
            raise ValueError("checkpoint has no tensor %s" % name)
        have = tuple(ckpt.tensors[key].shape)
        if have != shape:
            raise ValueError("tensor %s: checkpoint has shape %s, model expects %s" % (key, list(have), list(shape)))
        sources.append((index, key))
    used = {key for _, key in sources}
    unused = sorted(k for k in ckpt.tensors if k not in used)
    if unused:
        raise ValueError("checkpoint has %d tensor(s) the model does not have, e.g. %s (a different rank, LoRA "
                         "targets or --train-modules?)" % (len(unused), unused[0]))
    for index, key in sources:
        model.write_param(index, ckpt.tensors[key])
    return len(sources)


# ---------------------------------------------------------------------------
# training checkpoints
# ---------------------------------------------------------------------------

@dataclass
class TrainingState:
    """checkpoint.rs:310-345 (serde field names)."""
    step: int = 0
    total_steps: int = 0
    best_loss: Optional[float] = None
    lr: float = 0.0
    epoch: int = 0
    batch_size: int = 1
    grad_accum_steps: int = 1
    sequence_length: int = 128
    fp16: bool = False
    train_modules: str = "lora"
    task: str = "sft"
    model_path: str = ""
    dataset_path: str = ""
    seed: int = 0


@dataclass
class AdamWState:
    """`AdamWCheckpoint` (autograd/src/lib.rs:1455-1472) with the moments as arrays."""
    lr: float
    beta1: float
    beta2: float
    eps: float
    weight_decay: float
    t: float
    m_states: Dict[str, np.ndarray] = field(default_factory=dict)
    v_states: Dict[str, np.ndarray] = field(default_factory=dict)


def moments_path(path: str) -> str:
    """`x.state.json` -> `x.state.safetensors` (checkpoint.rs:509-511)."""
    return os.path.splitext(path)[0] + ".safetensors"


def optimizer_state(trainer, hyper: Optional[Dict[str, float]] = None) -> AdamWState:
    """`AdamW::save_state`: moments keyed by the adapter-file names of the parameters."""
    lib, model = trainer._lib, trainer.model
    hyper = hyper or trainer.hyper
    shapes = _param_shapes(model)
    t = C.c_float()
    check(lib.ft_trainer_get_adam_t(trainer.handle, C.byref(t)))
    st = AdamWState(hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"], hyper["weight_decay"], t.value)
    for i, (name, numel) in enumerate(model.named_params()):
        m, v = np.empty(numel, np.float32), np.empty(numel, np.float32)
        check(lib.ft_trainer_read_moments(trainer.handle, i, m.ctypes.data_as(C.c_void_p),
                                          v.ctypes.data_as(C.c_void_p)))
        st.m_states[file_name(name)] = m.reshape(shapes[name])
        st.v_states[file_name(name)] = v.reshape(shapes[name])
    return st


def save_training_checkpoint(path: str, state: TrainingState, adam: Optional[AdamWState]):
    """`TrainingCheckpoint::save`: moments file first (it records step and t), then the JSON."""
    light = None
    if adam is not None:
        if adam.m_states or adam.v_states:
            tensors = {"m/" + n: a for n, a in adam.m_states.items()}
            tensors.update({"v/" + n: a for n, a in adam.v_states.items()})
            write_safetensors(moments_path(path), tensors,
                              {"format": MOMENTS_FORMAT, "step": str(state.step), "t": format_f32(adam.t)})
        shapes = lambda d: {n: {"shape": list(a.shape), "data": []} for n, a in d.items()}
        light = {"AdamW": {"lr": float(np.float32(adam.lr)), "beta1": float(np.float32(adam.beta1)),
                           "beta2": float(np.float32(adam.beta2)), "eps": float(np.float32(adam.eps)),
                           "weight_decay": float(np.float32(adam.weight_decay)), "t": float(np.float32(adam.t)),
                           "m_states": shapes(adam.m_states), "v_states": shapes(adam.v_states)}}
    doc = {"training_state": asdict(state), "optimizer_state": light, "grad_scaler_state": None}
    tmp = os.path.splitext(path)[0] + ".json.tmp"
    with open(tmp, "w") as f:
        json.dump(doc, f, indent=2)
    os.replace(tmp, path)


def load_training_checkpoint(path: str) -> Tuple[TrainingState, Optional[AdamWState]]:
    """`TrainingCheckpoint::load` + `read_moments`: a moments file from another step is an error."""
    with open(path) as f:
        doc = json.load(f)
    known = {f_ for f_ in TrainingState.__dataclass_fields__}
    state = TrainingState(**{k: v for k, v in doc["training_state"].items() if k in known})
    opt = doc.get("optimizer_state")
    if not opt:
        return state, None
    a = opt["AdamW"]
    adam = AdamWState(a["lr"], a["beta1"], a["beta2"], a["eps"], a["weight_decay"], a["t"])
    inline = {k: {n: np.asarray(t["data"], np.float32).reshape(t["shape"]) for n, t in a[k].items() if t["data"]}
              for k in ("m_states", "v_states")}
    missing = any(not t["data"] and int(np.prod(t["shape"])) > 0
                  for k in ("m_states", "v_states") for t in a[k].values())
    if missing:
        mp = moments_path(path)
        tensors, meta = read_safetensors(mp)
        if meta.get("format") != MOMENTS_FORMAT:
            raise ValueError("%s is not an optimizer moments file" % mp)
        try:
            saved_step, saved_t = int(meta.get("step", "")), float(meta.get("t", "nan"))
        except ValueError:
            saved_step, saved_t = -1, float("nan")
        if saved_step != state.step or np.float32(saved_t) != np.float32(adam.t):
            raise ValueError("optimizer moments in %s are from step %s, but the checkpoint is at step %d; "
                             "the run was probably interrupted while saving" % (mp, meta.get("step"), state.step))
        for key, pre in (("m_states", "m/"), ("v_states", "v/")):
            for n, t in a[key].items():
                if pre + n not in tensors:
                    raise ValueError("%s has no tensor %s" % (mp, pre + n))
                arr = tensors[pre + n]
                if list(arr.shape) != list(t["shape"]):
                    raise ValueError("%s in %s has shape %s, expected %s" % (pre + n, mp, list(arr.shape), t["shape"]))
                inline[key][n] = arr
    adam.m_states, adam.v_states = inline["m_states"], inline["v_states"]
    return state, adam


@dataclass(frozen=True)
class OptimizerLoad:
    """autograd/src/lib.rs:1427-1442: parameters that took both saved moments, parameters left without,
    and saved names no parameter has."""
    matched: int
    missing: int
    unused: int

    def is_complete(self) -> bool:
        return self.missing == 0 and self.unused == 0


def match_moments(shapes: Dict[str, Tuple[int, ...]], adam: AdamWState) -> Tuple[List[str], OptimizerLoad]:
    """`match_moments` (autograd/src/lib.rs:1669-1703): which saved moments belong to which parameters, without
    touching the device. A saved moment whose shape differs from its parameter's is an error that names it."""
    saved = sorted(set(adam.m_states) | set(adam.v_states))
    matched = []
    for name in saved:
        shape, m, v = shapes.get(name), adam.m_states.get(name), adam.v_states.get(name)
        if shape is None or m is None or v is None:
            continue
        for kind, moment in (("first", m), ("second", v)):
            if tuple(moment.shape) != tuple(shape):
                raise ValueError("saved %s moment of %s has shape %s (%d values), the parameter has shape %s"
                                 % (kind, name, list(moment.shape), moment.size, list(shape)))
        matched.append(name)
    return matched, OptimizerLoad(len(matched), len(shapes) - len(matched), len(saved) - len(matched))


def restore_optimizer(trainer, adam: AdamWState, step: Optional[int] = None) -> OptimizerLoad:
    """`AdamW::load_state` (autograd/src/lib.rs:1630-1662) and, given `step`, `Trainer::set_optimizer_steps`:
    every parameter with both saved moments of its shape takes them; a wrong shape raises before anything is
    changed; when nothing matches the optimizer is left as it was; otherwise the saved hyperparameters and
    step counter `t` come back too (parameters without saved moments start from zero moments)."""
    lib, model = trainer._lib, trainer.model
    names = [(file_name(name), numel) for name, numel in model.named_params()]
    shapes = {file_name(n): s for n, s in _param_shapes(model).items()}
    matched, report = match_moments(shapes, adam)
    if not matched:
        return report
    taken = set(matched)
    # hyperparameters and the step counter first: a value the trainer refuses (beta >= 1, negative eps,
    # a non-finite rate) raises here, before any moment on the device has been replaced
    check(lib.ft_trainer_set_adam_hyper(trainer.handle, adam.lr, adam.beta1, adam.beta2, adam.eps, adam.weight_decay))
    check(lib.ft_trainer_set_adam_t(trainer.handle, float(adam.t)))
    for i, (key, numel) in enumerate(names):
        if key in taken:
            m = np.ascontiguousarray(adam.m_states[key], np.float32)
            v = np.ascontiguousarray(adam.v_states[key], np.float32)
        else:
            m = v = np.zeros(numel, np.float32)
        check(lib.ft_trainer_write_moments(trainer.handle, i, m.ctypes.data_as(C.c_void_p),
                                           v.ctypes.data_as(C.c_void_p)))
    trainer.hyper.update(beta1=adam.beta1, beta2=adam.beta2, eps=adam.eps, weight_decay=adam.weight_decay)
    if trainer.lr_schedule == "constant":
        trainer.hyper["lr"] = adam.lr
    if step is not None:
        trainer.set_optimizer_steps(step)
    return report
