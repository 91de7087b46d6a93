#!/usr/bin/env python3
"""LoRA train step benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 360m|135m|1.7b|tiny|micro|probe]

A step is one full optimizer step (forward, masked cross-entropy, backward,
gradient norm, clip, AdamW) of the SmolLM2-360M-shaped model on 8 sequences x
256 tokens of synthetic, seeded input (BASELINE.json configs[3]); frozen f16
base weights, f32 LoRA rank 8 alpha 16 on q/k/v/o, AdamW lr 2e-4. Weights and
inputs are resident in HBM when the timed region starts, except the 2048 token
ids / targets / weights the step uploads itself (24 KiB).

Prints ONE JSON line: tokens/s (positions = B*S / step time; the reference CLI's
tok/s counts supervised tokens only: `supervised_tokens_per_s`), plus
  roofline     the dominant GEMM kernel: algorithmic 2*M*N*K flops per launch
               over its HIP-event duration (events on the library's stream,
               taken over K further steps identical to the timed ones), against
               the 157.3 TFLOP/s dense FP32 matrix peak;
  cpu_baseline the CPU oracle (oracle/) on this host's cores, on a bounded
               sample of the same workload (stated in `sample`).

--workload micro runs the kernel microbenchmark instead (BASELINE.json
configs[1]: the 2048x576x1536 LoRA GEMM and its two backward GEMMs, attention
forward + backward at 8 x 256 x 9/3 heads x 64, RMSNorm forward + backward on
2048 x 576, AdamW over 4M parameters) and prints one JSON line with every
kernel's HIP-event time against the roofline that bounds it.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (layers, hidden, heads, kv_heads, ffn, vocab, batch, seq, rank, alpha, targets, prompt range)
    "360m": dict(layers=32, hidden=960, heads=15, kv=5, ffn=2560, vocab=49152, B=8, S=256, rank=8, alpha=16.0,
                 targets=("q_proj", "k_proj", "v_proj", "o_proj"), prompt=(32, 128),
                 label="SmolLM2-360M-shaped LoRA step, 8x256 (BASELINE.json configs[3])"),
    "135m": dict(layers=30, hidden=576, heads=9, kv=3, ffn=1536, vocab=49152, B=8, S=256, rank=8, alpha=16.0,
                 targets=("q_proj", "k_proj", "v_proj", "o_proj"), prompt=(32, 128),
                 label="SmolLM2-135M-shaped LoRA step, 8x256 (BASELINE.json configs[2])"),
    "1.7b": dict(layers=24, hidden=2048, heads=32, kv=32, ffn=8192, vocab=49152, B=8, S=1024, rank=16, alpha=32.0,
                 targets=("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"),
                 prompt=(64, 512), checkpoint=True,
                 label="SmolLM2-1.7B-shaped LoRA step, 8x1024, per-layer activation checkpointing "
                       "(BASELINE.json configs[4])"),
    "tiny": dict(layers=2, hidden=64, heads=4, kv=2, ffn=128, vocab=256, B=2, S=32, rank=4, alpha=8.0,
                 targets=("q_proj", "k_proj", "v_proj", "o_proj"), prompt=(4, 8), label="tiny Llama (plumbing check)"),
}


def synthetic_tensors(w, seed=0):
    """Random-init N(0, 0.02) weights in Hugging Face layout ([out, in]); norm scales 1."""
    rng = np.random.default_rng(seed)
    H, F, V = w["hidden"], w["ffn"], w["vocab"]
    D = H // w["heads"]

    def n(*shape):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)

    yield "model.embed_tokens.weight", n(V, H)
    yield "model.norm.weight", np.ones(H, np.float32)
    for l in range(w["layers"]):
        p = f"model.layers.{l}"
        yield f"{p}.input_layernorm.weight", np.ones(H, np.float32)
        yield f"{p}.post_attention_layernorm.weight", np.ones(H, np.float32)
        yield f"{p}.self_attn.q_proj.weight", n(w["heads"] * D, H)
        yield f"{p}.self_attn.k_proj.weight", n(w["kv"] * D, H)
        yield f"{p}.self_attn.v_proj.weight", n(w["kv"] * D, H)
        yield f"{p}.self_attn.o_proj.weight", n(H, w["heads"] * D)
        yield f"{p}.mlp.gate_proj.weight", n(F, H)
        yield f"{p}.mlp.up_proj.weight", n(F, H)
        yield f"{p}.mlp.down_proj.weight", n(H, F)


def synthetic_batch(w, seed=1, B=None):
    """Token ids uniform over the vocabulary; targets = next token; the loss mask
    zeroes a prompt prefix whose length is uniform in the workload's range."""
    rng = np.random.default_rng(seed)
    B = B or w["B"]
    S, V = w["S"], w["vocab"]
    rows = rng.integers(0, V, (B, S)).astype(np.uint32)
    targets = np.concatenate([rows[:, 1:], rng.integers(0, V, (B, 1)).astype(np.uint32)], axis=1)
    masks = np.ones((B, S), np.uint8)
    lo, hi = w["prompt"]
    for b in range(B):
        masks[b, :int(rng.integers(lo, hi + 1))] = 0
    return rows, targets, masks


def lora_factors(model, w, seed=2):
    rng = np.random.default_rng(seed)
    for name in model.linear_prefixes(w["targets"]):
        i, o = model.linear_dims(name)
        a = rng.standard_normal((i, w["rank"]), dtype=np.float32) * np.float32(0.02)
        b = rng.standard_normal((w["rank"], o), dtype=np.float32) * np.float32(0.02)
        yield name, a, b


def step_flops(w, head_rows=None):
    """Algorithmic flops of one step, exactly the products that run: `2 M N K` for every forward GEMM on the
    frozen base and every input-gradient GEMM (the first block's q/k/v have none: their input is the frozen
    embedding), the head and its input gradient on `head_rows` rows (the supervised positions), the rank-r
    products of every adapter (forward x@A, t@B; backward dT, dT@A^T, dA, dB), attention forward + 2.5x
    backward (causal: 2 B H S^2 D forward)."""
    T = w["B"] * w["S"]
    H, F, V, L, r = w["hidden"], w["ffn"], w["vocab"], w["layers"], w["rank"]
    D = H // w["heads"]
    dims = {"q_proj": (H, w["heads"] * D), "k_proj": (H, w["kv"] * D), "v_proj": (H, w["kv"] * D),
            "o_proj": (w["heads"] * D, H), "gate_proj": (H, F), "up_proj": (H, F), "down_proj": (F, H)}
    head_rows = T if head_rows is None else head_rows
    total = 2 * 2.0 * head_rows * H * V
    for layer in range(L):
        for name, (i, o) in dims.items():
            dx = not (layer == 0 and name in ("q_proj", "k_proj", "v_proj"))
            total += 2.0 * T * i * o * (2 if dx else 1)
            if name in w["targets"]:
                total += 2.0 * T * r * (i + o) * (3 if dx else 2)
                if not dx:
                    total += 2.0 * T * r * o   # dT is still needed for dA
    total += 2.0 * w["B"] * w["heads"] * w["S"] ** 2 * D * 3.5 * L
    if w.get("checkpoint"):
        # every block but the last is run forward a second time before its backward
        for name, (i, o) in dims.items():
            total += (L - 1) * (2.0 * T * i * o + (2.0 * T * r * (i + o) if name in w["targets"] else 0.0))
        total += 2.0 * w["B"] * w["heads"] * w["S"] ** 2 * D * (L - 1)
    return total


def read_profile(ctx):
    lib = ctx._lib
    n = C.c_size_t()
    from ferrotensor_amd._lib import check
    check(lib.ft_profile_end(ctx.handle, C.byref(n)))
    out = []
    for i in range(n.value):
        name, launches = C.c_char_p(), C.c_uint64()
        ms, fl, by = C.c_double(), C.c_double(), C.c_double()
        check(lib.ft_profile_kernel(ctx.handle, i, C.byref(name), C.byref(launches), C.byref(ms), C.byref(fl),
                                    C.byref(by)))
        if launches.value:
            out.append(dict(name=name.value.decode(), launches=launches.value, ms=ms.value, flops=fl.value,
                            bytes=by.value))
    return sorted(out, key=lambda r: -r["ms"])


def cpu_baseline(w, seconds_budget=45.0):
    """The CPU oracle on this host: the same step on the same batch. One sequence is timed first; when the
    whole batch fits the budget it is timed too (median of up to 3 steps) and that is what is reported,
    otherwise the one-sequence figure (a bounded sample of the same workload, stated in `sample`)."""
    from oracle import cpu
    from oracle import reference_step as rs
    cfg = rs.ModelConfig(w["vocab"], w["hidden"], w["ffn"], w["layers"], w["heads"], w["kv"], 1e-5, 100000.0, True)
    tensors = dict(synthetic_tensors(w))
    model = rs.Model.from_hf_tensors(cfg, tensors, f16_linears=True)
    del tensors
    rng = np.random.default_rng(2)
    for name, lin in model.named_linears():
        if name.split(".")[-1] in w["targets"]:
            i, o = lin.weight.shape
            model.set_lora(name, rng.standard_normal((i, w["rank"]), dtype=np.float32) * np.float32(0.02),
                           rng.standard_normal((w["rank"], o), dtype=np.float32) * np.float32(0.02), w["alpha"])
    rows, targets, masks = synthetic_batch(w)
    opt = rs.AdamW(lr=2e-4, weight_decay=0.0)

    def timed(n):
        t0 = time.perf_counter()
        rs.train_chunk(model, opt, rows[:n], targets[:n], masks[:n], grad_accum_steps=w["B"], clip_grad_norm=1.0)
        return time.perf_counter() - t0

    t_all = time.perf_counter()
    one = timed(1)
    n, times = 1, [one]
    if one * w["B"] * 1.2 < seconds_budget:
        n, times = w["B"], []
        while len(times) < 3 and (not times or time.perf_counter() - t_all + times[-1] < seconds_budget):
            times.append(timed(n))
    t = float(np.median(times))
    return {"value": n * w["S"] / t, "unit": "tokens/s", "cores": cpu.num_threads(), "kind": "port",
            "sample": "%d of the %d sequences (%d tokens), all %d layers + head, fwd+bwd+AdamW, median of %d steps, "
                      "%.2f s/step, %d OpenMP threads" % (n, w["B"], n * w["S"], w["layers"], len(times), t,
                                                          cpu.num_threads())}


# What the rocprofv3 counters read for a plain 16 MiB device copy: FETCH_SIZE 8203.5 KiB for 16384 KiB read,
# WRITE_SIZE 16384.0 KiB for 16384 KiB written.
FETCH_SIZE_FACTOR = 16384.0 / 8203.5
WRITE_SIZE_FACTOR = 1.0


def source_hash():
    """Hash of the library's sources: names the build a stored profile was taken from."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "ferrotensor_amd", "csrc")
    for name in sorted(os.listdir(src)) + ["../../include/ferrotensor_hip.h"]:
        with open(os.path.join(src, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


TRAFFIC_PROFILE = os.path.join("profiles", "lora_step_360m_hbm_traffic.md")


def traffic_source():
    """Where `roofline.traffic` comes from: hardware counters cannot be read from inside this process, so the
    figure is the one the rocprofv3 --pmc runs of this same command recorded under profiles/. The profile
    names the source hash of the library it was taken from; `current` says whether that is this build."""
    recorded = None
    try:
        for line in open(os.path.join(ROOT, TRAFFIC_PROFILE)):
            if line.startswith("Library source hash:"):
                recorded = line.split(":", 1)[1].strip().strip("`")
    except OSError:
        pass
    return {"file": TRAFFIC_PROFILE, "library_source_hash": recorded, "current": recorded == source_hash()}


def measured_traffic(kernel, workload):
    """HBM-side bytes per launch of `kernel` (calibrated FETCH_SIZE + WRITE_SIZE, KiB per dispatch) as recorded
    by the rocprofv3 --pmc runs summarised under profiles/; None when there is no record for this kernel."""
    if workload != "360m":
        return None
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    # profile names -> kernel symbols: <.., layout, segments[, epilogue[, wave groups]]>
    name = kernel
    for tag, code in (("gate_up", "1, 1"), ("silu_bwd", "2, 1")):
        name = name.replace(", %s>" % tag, ", %s>" % code)
    if name == kernel and kernel.count(",") == 5:
        name = kernel[:-1] + ", 0, 1>"
    try:
        for line in open(path):
            cells = [c.strip() for c in line.split("|")]
            if len(cells) >= 5 and cells[1] == "`%s`" % name:
                return (FETCH_SIZE_FACTOR * float(cells[3]) + WRITE_SIZE_FACTOR * float(cells[4])) * 1024.0
    except (OSError, ValueError):
        pass
    return None


def micro_bench(args):
    """The kernel microbenchmark: each kernel `steps` times after `warmup` passes, timed by HIP events on the
    library's stream; algorithmic flops and bytes are the ones the library records per launch."""
    from ferrotensor_amd import AdamParams, AttentionOptions, ComputeEngine, HipContext, UnifiedTensor
    from ferrotensor_amd._lib import check

    ctx = HipContext(0)
    eng = ComputeEngine(ctx)
    rng = np.random.default_rng(0)

    def up(*shape, scale=1.0):
        return UnifiedTensor.new(ctx, rng.standard_normal(shape, dtype=np.float32) * np.float32(scale), list(shape))

    def empty(*shape):
        return UnifiedTensor.empty(ctx, list(shape))

    M, K, N, r, s = 2048, 576, 1536, 8, 2.0
    x, dy = up(M, K), up(M, N)
    w = UnifiedTensor.from_f32_as_f16(ctx, rng.standard_normal((K, N), dtype=np.float32), [K, N])
    a, b = up(K, r), up(r, N)
    t_, dt, y, dx = empty(M, r), empty(M, r), empty(M, N), empty(M, K)
    dw, da, db = empty(K, N), empty(K, r), empty(r, N)
    B, S, H, Hkv, D = 8, 256, 9, 3, 64
    q, k, v, do = up(B, S, H, D), up(B, S, Hkv, D), up(B, S, Hkv, D), up(B, S, H, D)
    o, stats = empty(B, S, H, D), empty(B * H * S, 2)
    dq, dk, dv = empty(B, S, H, D), empty(B, S, Hkv, D), empty(B, S, Hkv, D)
    opts = AttentionOptions(causal=True)
    nx, ng, nw = up(M, K), up(M, K), up(K)
    ny, ngx, ngw = empty(M, K), empty(M, K), empty(K)
    n = 4 * 1024 * 1024
    pw, pg, pm = up(n), up(n), up(n, scale=0.1)
    pv = UnifiedTensor.new(ctx, np.abs(rng.standard_normal(n, dtype=np.float32)) * np.float32(0.1), [n])
    adam = AdamParams(lr=2e-4, weight_decay=0.01, t=3.0)
    pcopy = empty(n)

    def one_pass():
        eng.lora_down(ctx, x, a, t_, s)                      # forward: y = x@W + (x@A * s)@B
        eng.lora_linear(ctx, x, w, t_, b, y)
        eng.lora_grad_down(ctx, dy, b, dt, s)                # backward 1: dx = dy@W^T + (dy@B^T * s)@A^T
        eng.lora_linear_dx(ctx, dy, w, dt, a, dx)
        eng.matmul_at(ctx, x, dy, dw)                        # backward 2: x^T@dy at full size, and the thin ones
        eng.lora_grad_a(ctx, x, dt, da)
        eng.lora_grad_b(ctx, t_, dy, db)
        eng.flash_attention_v2_with_stats(ctx, q, k, v, o, stats, opts)
        eng.flash_attention_v2_backward_with_stats(ctx, q, k, v, o, do, dq, dk, dv, stats, opts)
        eng.rms_norm_eps(ctx, nx, nw, ny, 1e-5)
        eng.rms_norm_backward(ctx, nx, nw, ng, ngx, ngw, 1e-5)
        eng.adamw_update(ctx, pw, pg, pm, pv, adam)
        eng.copy_tensor(ctx, pg, pcopy)                      # plain 16 MiB copy: the known-size kernel that
                                                             # hardware traffic counters are calibrated on

    for _ in range(args.warmup):
        one_pass()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_pass()
    ctx.synchronize()
    elapsed = time.perf_counter() - t0
    check(ctx._lib.ft_profile_begin(ctx.handle))
    for _ in range(args.steps):
        one_pass()
    kernels = []
    for rec in read_profile(ctx):
        us = rec["ms"] * 1e3 / rec["launches"]
        if rec["flops"] > 0:
            ach = rec["flops"] / (rec["ms"] * 1e-3) / 1e12
            kernels.append({"kernel": rec["name"], "bound": "mfma", "launches": rec["launches"] // args.steps,
                            "avg_us": us, "achieved": ach, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                            "frac": ach / FP32_MFMA_PEAK_TFLOPS})
        else:
            ach = rec["bytes"] / (rec["ms"] * 1e-3) / 1e9
            kernels.append({"kernel": rec["name"], "bound": "hbm", "launches": rec["launches"] // args.steps,
                            "avg_us": us, "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": ach / HBM_PEAK_GBS})
    gemm = max((k_ for k_ in kernels if k_["kernel"].startswith("gemm_")), key=lambda k_: k_["avg_us"] * k_["launches"])
    print(json.dumps({
        "metric": "kernel microbench (BASELINE.json configs[1]): FP32-MFMA TFLOP/s of the LoRA GEMM kernel",
        "value": gemm["achieved"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "kernel microbench: GEMM 2048x576x1536 (f16 B, rank-8 LoRA) fwd + 2 bwd; attention "
                               "8x256, 9/3 heads, 64; RMSNorm 2048x576 fwd+bwd; AdamW 4M"},
        "roofline": {"bound": "mfma", "kernel": gemm["kernel"], "achieved": gemm["achieved"],
                     "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": gemm["frac"], "traffic": None},
        "kernels": kernels}))


def mfma_probe(args):
    """What the FP32 matrix pipes sustain with no memory traffic at all: short and long launches, one to
    three waves per SIMD, dependent (1 chain) and independent (4 chains) accumulators."""
    from ferrotensor_amd import HipContext

    ctx = HipContext(0)
    runs = []
    for random_operands in (False, True):
        for waves in (1, 2, 3):
            for chains in (1, 4):
                for rounds in (100, 1000, 10000, 100000):
                    ctx.mfma_probe(rounds, waves, chains, random_operands)
                    best = None
                    for _ in range(3 if rounds < 100000 else 2):
                        s, f = ctx.mfma_probe(rounds, waves, chains, random_operands)
                        best = s if best is None or s < best else best
                    runs.append({"operands": "random" if random_operands else "ones", "waves_per_simd": waves,
                                 "chains": chains, "mfma_per_wave": rounds * 16, "us": best * 1e6,
                                 "tflops": f / best / 1e12})
    # A back-to-back train of 1.6 ms launches for about a second: the rate under continuous load.
    t0 = time.perf_counter()
    n, total_s, total_f = 0, 0.0, 0.0
    while time.perf_counter() - t0 < 1.0:
        s, f = ctx.mfma_probe(10000, 2, 4, True)
        total_s, total_f, n = total_s + s, total_f + f, n + 1
    sustained = total_f / total_s / 1e12
    best = max(r["tflops"] for r in runs)
    print(json.dumps({
        "metric": "FP32 MFMA rate of a register-only v_mfma_f32_32x32x2_f32 loop", "value": sustained,
        "unit": "TFLOP/s", "n_gpus": 1, "steps": n, "warmup": 0, "ms_per_step": total_s / n * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "matrix-pipe probe: %d launches of 160000 MFMAs per wave, 2 waves per SIMD, "
                               "4 independent accumulators, pseudo-random operands" % n},
        "roofline": {"bound": "mfma", "kernel": "mfma_probe_kernel<4>", "achieved": sustained,
                     "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": sustained / FP32_MFMA_PEAK_TFLOPS,
                     "traffic": None},
        "best_single_launch_tflops": best, "runs": runs}))


def engine_ops_path(ctx, cfg, w, rows, targets, masks, args, fused_loss):
    """The same workload through `ferrotensor_amd.engine_step`: every op of the step as its own call of the
    1:1 ComputeEngine entry point, in the order the reference's autograd tape issues them (six calls per LoRA
    linear, copy + scale, copy + RoPE, one sum-of-squares / clip / AdamW call per tensor). Same weights, batch
    and optimizer settings as the fused path; the head runs on every position, as in the reference."""
    from ferrotensor_amd.engine_step import EngineOpsModel, EngineOpsTrainer
    eo = EngineOpsModel(ctx, cfg, dict(synthetic_tensors(w)))
    rng = np.random.default_rng(2)
    dims = {"q_proj": (w["hidden"], w["hidden"]), "k_proj": (w["hidden"], w["hidden"] // w["heads"] * w["kv"]),
            "v_proj": (w["hidden"], w["hidden"] // w["heads"] * w["kv"]), "o_proj": (w["hidden"], w["hidden"]),
            "gate_proj": (w["hidden"], w["ffn"]), "up_proj": (w["hidden"], w["ffn"]), "down_proj": (w["ffn"], w["hidden"])}
    order = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    for layer in range(w["layers"]):          # the order lora_factors draws them in: layer by layer
        for name in order:
            if name in w["targets"]:
                i, o = dims[name]
                a = rng.standard_normal((i, w["rank"]), dtype=np.float32) * np.float32(0.02)
                b = rng.standard_normal((w["rank"], o), dtype=np.float32) * np.float32(0.02)
                eo.set_lora(layer, name, a, b, w["alpha"])
    tr = EngineOpsTrainer(eo, lr=2e-4, weight_decay=0.0, clip_grad_norm=1.0)
    steps = max(3, args.steps // 4)
    first_loss = None
    for _ in range(2):
        loss, norm, clip = tr.train_chunk(rows, targets, masks)
        first_loss = loss if first_loss is None else first_loss
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss, norm, clip = tr.train_chunk(rows, targets, masks)
    ctx.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    return {"ms_per_step": ms, "tokens_per_s": w["B"] * w["S"] / (ms * 1e-3), "steps": steps,
            "engine_calls_per_step": tr.calls, "first_step_loss": first_loss,
            "note": "1:1 ComputeEngine entry points in the reference's op order, driven from Python over ctypes; "
                    "loss of its first step next to the fused path's current loss (%.4f, after its own steps)" % fused_loss}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="360m", choices=sorted(WORKLOADS) + ["micro", "probe"])
    ap.add_argument("--micro-batch", type=int, default=0,
                    help="sequences per forward/backward pass (default: the whole batch); gradients accumulate "
                         "over the batch and one optimizer step follows, as `ferrotensor train --batch m --accum B/m`")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--path", default="fused", choices=["fused", "engine-ops"],
                    help="engine-ops: additionally time the same step composed only of the 1:1 ComputeEngine entry "
                         "points in the reference's op order (ferrotensor_amd.engine_step) and report it as "
                         "`engine_ops_path` next to the fused number")
    ap.add_argument("--breakdown", action="store_true", help="print the per-kernel event-time table to stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (one process, one HIP stream); --gpus %d is not supported. "
                 "The step would shard by data parallelism over sequences with one all-reduce of the LoRA "
                 "gradients, which is not built." % args.gpus)
    if args.workload == "micro":
        return micro_bench(args)
    if args.workload == "probe":
        return mfma_probe(args)
    w = WORKLOADS[args.workload]

    from ferrotensor_amd import HipContext
    from ferrotensor_amd.trainer import Lfm2Model, ModelConfig, Trainer

    ctx = HipContext(0)
    cfg = ModelConfig(vocab_size=w["vocab"], hidden_size=w["hidden"], intermediate_size=w["ffn"],
                      num_hidden_layers=w["layers"], num_attention_heads=w["heads"], num_key_value_heads=w["kv"],
                      rms_norm_eps=1e-5, rope_theta=100000.0, tie_word_embeddings=True, f16_linears=True,
                      checkpoint_blocks=bool(w.get("checkpoint", False)))
    model = Lfm2Model(ctx, cfg)
    for name, value in synthetic_tensors(w):
        model.set_tensor(name, value)
    for name, a, b in lora_factors(model, w):
        model.set_lora(name, a, b, w["alpha"])
    # CLI defaults of `ferrotensor train`: lr 2e-4, weight decay 0, clip 1.0, accumulation = batch.
    rows, targets, masks = synthetic_batch(w)
    mb = args.micro_batch or w["B"]
    if w["B"] % mb:
        sys.exit("bench.py: --micro-batch must divide the batch of %d sequences" % w["B"])
    # --micro-batch m: the reference's `--batch m --accum B/m` regime, one optimizer step per B sequences.
    trainer = Trainer(model, lr=2e-4, weight_decay=0.0, clip_grad_norm=1.0, grad_accum_steps=w["B"])

    def one_step():
        st = None
        for i in range(0, w["B"], mb):
            st = trainer.train_chunk(rows[i:i + mb], targets[i:i + mb], masks[i:i + mb])
        return st

    for _ in range(args.warmup):
        st = one_step()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        st = one_step()
    ctx.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    tokens = w["B"] * w["S"]
    value = tokens / (elapsed / args.steps)
    if not (np.isfinite(st.loss) and st.optimizer_step):
        sys.exit("bench.py: the step did not produce a finite loss / optimizer step: %r" % (st,))

    # The same steps with the head on every position, as the reference runs it (same results, more work).
    model.set_head_all_rows(True)
    one_step()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_step()
    ctx.synchronize()
    ms_all_rows = (time.perf_counter() - t0) / args.steps * 1e3
    model.set_head_all_rows(False)
    one_step()

    # Per-kernel HIP-event timing over the same number of identical steps.
    from ferrotensor_amd._lib import check
    check(ctx._lib.ft_profile_begin(ctx.handle))
    for _ in range(args.steps):
        one_step()
    prof = read_profile(ctx)
    gemms = [r for r in prof if r["name"].startswith("gemm_")]
    dom = gemms[0]
    achieved = dom["flops"] / (dom["ms"] * 1e-3) / 1e12
    all_gemm_ms = sum(r["ms"] for r in gemms)
    all_gemm_tf = sum(r["flops"] for r in gemms) / (all_gemm_ms * 1e-3) / 1e12
    kernel_ms = sum(r["ms"] for r in prof) / args.steps
    if args.breakdown:
        print("%-44s %8s %10s %9s %9s" % ("kernel", "launches", "ms/step", "TFLOP/s", "GB/s"), file=sys.stderr)
        for r in prof:
            print("%-44s %8d %10.3f %9.1f %9.0f" % (r["name"], r["launches"] // args.steps, r["ms"] / args.steps,
                                                    r["flops"] / (r["ms"] * 1e-3) / 1e12 if r["ms"] else 0,
                                                    r["bytes"] / (r["ms"] * 1e-3) / 1e9 if r["ms"] else 0),
                  file=sys.stderr)
        print("sum of kernel event time: %.3f ms/step; wall %.3f ms/step" % (kernel_ms, ms_per_step), file=sys.stderr)

    out = {
        "metric": ("LoRA train tokens/s at SmolLM2-360M shape, seq256x8; % FP32 MFMA peak" if args.workload == "360m"
                   else "LoRA train tokens/s, workload %s; %% FP32 MFMA peak" % args.workload),
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": w["label"], "global_batch": w["B"], "seq_len": w["S"], "micro_batch": mb,
                   "lora": "rank %d alpha %g on %s" % (w["rank"], w["alpha"], "/".join(w["targets"])),
                   "base_weights": "f16 storage, f32 arithmetic", "optimizer": "AdamW lr 2e-4 wd 0 clip 1.0",
                   "supervised_tokens": int(st.tokens), "loss": float(st.loss),
                   "head": "final norm, vocabulary head and loss on the %d supervised positions" % int(st.tokens)},
        "ms_per_step_head_all_rows": ms_all_rows, "tokens_per_s_head_all_rows": tokens / (ms_all_rows * 1e-3),
        "supervised_tokens_per_s": int(st.tokens) / (elapsed / args.steps),
        "step_tflops": step_flops(w, int(st.tokens)) / (elapsed / args.steps) / 1e12,
        "step_mfma_frac": step_flops(w, int(st.tokens)) / (elapsed / args.steps) / 1e12 / FP32_MFMA_PEAK_TFLOPS,
        "roofline": {"bound": "mfma", "kernel": dom["name"], "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
                     # the record is of the default batch: other micro-batch sizes have other launches
                     "traffic": measured_traffic(dom["name"], args.workload) if not args.micro_batch else None,
                     "traffic_source": traffic_source() if args.workload == "360m" and not args.micro_batch else None,
                     "launches_per_step": dom["launches"] // args.steps,
                     "avg_launch_us": dom["ms"] * 1e3 / dom["launches"],
                     "all_gemm_kernels_tflops": all_gemm_tf,
                     "all_gemm_kernels_frac": all_gemm_tf / FP32_MFMA_PEAK_TFLOPS,
                     "gemm_ms_per_step": all_gemm_ms / args.steps, "kernel_ms_per_step": kernel_ms},
    }
    if args.path == "engine-ops":
        out["engine_ops_path"] = engine_ops_path(ctx, cfg, w, rows, targets, masks, args, float(st.loss))
    if not args.no_cpu_baseline:
        trainer.close()
        model.close()
        ctx.close()
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
