"""Pins for each oracle kernel that do not come from the gradient fixture:
library routines (torch CPU), closed forms, golden JSON, special values.
A plausible mistake (dropped term, wrong sign/index, transposed operand)
fails at least one of these."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import cpu
from oracle import reference_step as rs

RNG = np.random.default_rng(1234)


def randn(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


# ---- f16 storage ---------------------------------------------------------

def test_f16_rounding_matches_ieee_rne():
    x = np.concatenate([
        randn(20000), randn(2000) * 1e-6, randn(2000) * 1e5,
        np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 6.1035156e-05,
                  5.9604645e-08, 2.9802322e-08, 2.98023224e-08 * 1.0001, 1e-10, np.inf, -np.inf,
                  1.0009765625, 1.00048828125, 1.00146484375], np.float32)])
    bits = cpu.pack_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(bits, want)
    np.testing.assert_array_equal(cpu.unpack_f16(bits).view(np.uint32),
                                  want.view(np.float16).astype(np.float32).view(np.uint32))
    assert np.isnan(cpu.unpack_f16(cpu.pack_f16(np.array([np.nan], np.float32))))[0]


def test_f16_every_bit_pattern_round_trips():
    bits = np.arange(65536, dtype=np.uint16)
    f = cpu.unpack_f16(bits)
    want = bits.view(np.float16).astype(np.float32)
    ok = ~np.isnan(want)
    np.testing.assert_array_equal(f[ok].view(np.uint32), want[ok].view(np.uint32))
    np.testing.assert_array_equal(cpu.pack_f16(f[ok]), bits[ok])


def test_f16_packing_is_little_endian_low_half_first():
    # tensor.rs:258-269: two values per 32-bit word, the first in the low half.
    bits = cpu.pack_f16(np.array([1.0, -2.0], np.float32))
    word = bits.view(np.uint32)[0]
    assert word & 0xFFFF == 0x3C00 and word >> 16 == 0xC000


# ---- matmul layouts ------------------------------------------------------

@pytest.mark.parametrize("M,K,N", [(1, 1, 1), (5, 7, 3), (33, 17, 65), (64, 576, 40), (130, 64, 129)])
def test_matmul_layouts_against_f64(M, K, N):
    a, b = randn(M, K), randn(K, N)
    want = a.astype(np.float64) @ b.astype(np.float64)
    tol = dict(rtol=1e-4, atol=1e-3)  # gpu_kernels.rs:989-1084 uses 1e-3 + 1e-4*|want|
    np.testing.assert_allclose(cpu.matmul(a, b), want, **tol)
    np.testing.assert_allclose(cpu.matmul_bt(a, np.ascontiguousarray(b.T)), want, **tol)
    np.testing.assert_allclose(cpu.matmul_at(np.ascontiguousarray(a.T), b), want, **tol)


def test_phase0_linear_and_rmsnorm_json(golden_dir):
    with open(os.path.join(golden_dir, "phase0_linear_rmsnorm.json")) as f:
        j = json.load(f)
    x = np.array(j["input"], np.float32)
    w_hf = np.array(j["linear_weight_hf_layout"], np.float32)
    want_lin = np.array(j["linear_output"], np.float32)
    got = cpu.matmul(x.reshape(-1, x.shape[-1]), cpu.transpose(w_hf))
    np.testing.assert_allclose(got.reshape(want_lin.shape), want_lin, rtol=1e-5, atol=1e-5)
    w = np.array(j["rms_weight"], np.float32)
    want_rms = np.array(j["rms_output"], np.float32)
    got = cpu.rms_norm(x, w, j["meta"]["eps"])
    np.testing.assert_allclose(got, want_rms, rtol=1e-5, atol=1e-5)


# ---- RMSNorm -------------------------------------------------------------

def test_rms_norm_backward_against_torch_autograd():
    x, w, g = randn(37, 96), randn(96), randn(37, 96)
    eps = 1e-5
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    y = xt * torch.rsqrt(xt.pow(2).mean(-1, keepdim=True) + eps) * wt
    y.backward(torch.tensor(g, dtype=torch.float64))
    np.testing.assert_allclose(cpu.rms_norm(x, w, eps), y.detach().numpy(), rtol=1e-5, atol=1e-5)
    gx, gw = cpu.rms_norm_backward(x, w, g, eps)
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=1e-4, atol=1e-4)


# ---- RoPE ----------------------------------------------------------------

def test_rope_closed_form_and_inverse():
    B, S, heads, D, theta, pos0 = 2, 9, 3, 8, 10000.0, 5
    x = randn(B, S, heads * D)
    got = cpu.rope(x, D, pos0, theta)
    x4 = x.reshape(B, S, heads, D).astype(np.float64)
    i = np.arange(D // 2)
    ang = (pos0 + np.arange(S))[:, None] * theta ** (-2.0 * i / D)[None, :]
    c, s = np.cos(ang)[None, :, None, :], np.sin(ang)[None, :, None, :]
    x1, x2 = x4[..., :D // 2], x4[..., D // 2:]
    want = np.concatenate([x1 * c - x2 * s, x1 * s + x2 * c], -1).reshape(B, S, heads * D)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    back = cpu.rope(got, D, pos0, theta, inverse=True)
    np.testing.assert_allclose(back, x, rtol=1e-5, atol=1e-5)
    # position 0 is the identity (autograd/src/lib.rs:1899-1912)
    one = randn(1, 1, D)
    np.testing.assert_array_equal(cpu.rope(one, D, 0, theta), one)


# ---- attention -----------------------------------------------------------

def _sdpa(q, k, v, causal, offset=0):
    B, Sq, H, D = q.shape
    Hkv = k.shape[2]
    qt = torch.tensor(q, dtype=torch.float64, requires_grad=True)
    kt = torch.tensor(k, dtype=torch.float64, requires_grad=True)
    vt = torch.tensor(v, dtype=torch.float64, requires_grad=True)
    qh = qt.transpose(1, 2)
    kh = kt.transpose(1, 2).repeat_interleave(H // Hkv, dim=1)
    vh = vt.transpose(1, 2).repeat_interleave(H // Hkv, dim=1)
    s = qh @ kh.transpose(-1, -2) / math.sqrt(D)
    Sk = k.shape[1]
    if causal:
        vis = torch.arange(Sk)[None, :] <= (torch.arange(Sq)[:, None] + offset)
        s = s.masked_fill(~vis, float("-inf"))
    lse = torch.logsumexp(s, -1)
    out = (s.softmax(-1) @ vh).transpose(1, 2)
    return qt, kt, vt, out, lse


@pytest.mark.parametrize("B,S,H,Hkv,D,causal", [(2, 13, 4, 2, 8, True), (1, 40, 6, 6, 16, True),
                                               (2, 17, 3, 1, 64, False), (1, 1, 2, 1, 4, True)])
def test_attention_forward_backward_against_torch(B, S, H, Hkv, D, causal):
    q, k, v, do = randn(B, S, H, D), randn(B, S, Hkv, D), randn(B, S, Hkv, D), randn(B, S, H, D)
    qt, kt, vt, out, lse = _sdpa(q, k, v, causal)
    out.backward(torch.tensor(do, dtype=torch.float64))
    got, got_lse = cpu.attention(q, k, v, causal=causal)
    np.testing.assert_allclose(got, out.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(got_lse, lse.detach().numpy(), rtol=1e-5, atol=1e-5)
    dq, dk, dv = cpu.attention_backward(q, k, v, got, do, causal=causal)
    np.testing.assert_allclose(dq, qt.grad.numpy(), rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(dk, kt.grad.numpy(), rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(dv, vt.grad.numpy(), rtol=1e-3, atol=1e-5)


def test_attention_is_causal_bit_exact():
    # changing later tokens must not change earlier outputs at all
    # (ferrotensor-graph/tests/model_correctness.rs:281-300)
    q, k, v = randn(1, 12, 2, 8), randn(1, 12, 1, 8), randn(1, 12, 1, 8)
    a, _ = cpu.attention(q, k, v)
    k2, v2 = k.copy(), v.copy()
    k2[:, 7:], v2[:, 7:] = randn(1, 5, 1, 8), randn(1, 5, 1, 8)
    b, _ = cpu.attention(q, k2, v2)
    np.testing.assert_array_equal(a[:, :7], b[:, :7])


# ---- SiLU gate -----------------------------------------------------------

def test_silu_gate_against_torch():
    a, b, g = randn(1000) * 3, randn(1000), randn(1000)
    at = torch.tensor(a, dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    y = torch.nn.functional.silu(at) * bt
    y.backward(torch.tensor(g, dtype=torch.float64))
    np.testing.assert_allclose(cpu.silu_gate(a, b), y.detach().numpy(), rtol=1e-5, atol=1e-6)
    ga, gb = cpu.silu_gate_backward(a, b, g)
    np.testing.assert_allclose(ga, at.grad.numpy(), rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(gb, bt.grad.numpy(), rtol=1e-4, atol=1e-6)


# ---- masked CE -----------------------------------------------------------

def test_masked_cross_entropy_against_torch():
    rows, vocab = 12, 50
    logits = randn(rows, vocab) * 4
    targets = RNG.integers(0, vocab, rows).astype(np.uint32)
    weights = RNG.random(rows).astype(np.float32)
    targets[[2, 7]] = rs.MASKED_CE_SKIP
    lt = torch.tensor(logits, dtype=torch.float64, requires_grad=True)
    keep = targets != rs.MASKED_CE_SKIP
    tt = torch.tensor(np.where(keep, targets, 0).astype(np.int64))
    per = torch.nn.functional.cross_entropy(lt, tt, reduction="none")
    wt = torch.tensor(np.where(keep, weights, 0.0), dtype=torch.float64)
    (per * wt).sum().backward()
    grad, row_loss = cpu.masked_cross_entropy(logits, targets, weights)
    np.testing.assert_allclose(row_loss[keep], per.detach().numpy()[keep], rtol=1e-5, atol=1e-5)
    assert (row_loss[~keep] == 0).all() and (grad[~keep] == 0).all()
    np.testing.assert_allclose(grad, lt.grad.numpy(), rtol=1e-4, atol=1e-6)


def test_targets_and_weights_are_exact():
    # trainer/src/lib.rs:695-722: out-of-vocab or masked rows are skipped;
    # weight = 1 / supervised tokens of the row's own sequence.
    tg = np.array([[1, 2, 99, 4], [5, 6, 7, 8]], np.uint32)
    mk = np.array([[0, 1, 1, 1], [1, 1, 1, 0]], np.uint8)
    t, w, tokens = rs.build_targets_and_weights(tg, mk, 2, vocab=10)
    np.testing.assert_array_equal(t, np.array([0xFFFFFFFF, 2, 0xFFFFFFFF, 4, 5, 6, 7, 0xFFFFFFFF], np.uint32))
    np.testing.assert_array_equal(tokens, [2, 3])
    np.testing.assert_array_equal(w, np.array([0, .5, 0, .5, np.float32(1) / np.float32(3),
                                               np.float32(1) / np.float32(3), np.float32(1) / np.float32(3), 0],
                                              np.float32))


# ---- grad norm, AdamW ----------------------------------------------------

def test_sum_squares_partial_chunks():
    x = randn(4096 * 2 + 100)
    out = np.zeros(8, np.float32)
    n = cpu.sum_squares_partial(x, out, 3)
    assert n == 3 and (out[:3] == 0).all() and (out[6:] == 0).all()
    want = [np.sum(x[i * 4096:(i + 1) * 4096].astype(np.float64) ** 2) for i in range(3)]
    np.testing.assert_allclose(out[3:6], want, rtol=1e-5)
    assert abs(float(rs.global_grad_norm([x])) - np.linalg.norm(x.astype(np.float64))) < 1e-3


@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_adamw_against_torch_optim(wd):
    n = 257
    w0, grads = randn(n), [randn(n) for _ in range(4)]
    wt = torch.nn.Parameter(torch.tensor(w0, dtype=torch.float64))
    opt = torch.optim.AdamW([wt], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd)
    w, m, v = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t, g in enumerate(grads, 1):
        wt.grad = torch.tensor(g, dtype=torch.float64)
        opt.step()
        cpu.adamw_update(w, g, m, v, 1e-3, 0.9, 0.999, 1e-8, wd, float(t))
        np.testing.assert_allclose(w, wt.detach().numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("max_norm,wd", [(0.5, 0.0), (1.0, 0.01), (1e9, 0.0)])
def test_apply_gradients_clips_like_torch_clip_grad_norm(max_norm, wd):
    """The clip of `apply_gradients` (max / (norm + 1e-6) when norm > max, trainer/src/lib.rs:336-343) is
    the rule of `torch.nn.utils.clip_grad_norm_`; followed by AdamW it must track torch over several
    steps, with tensors that span more than one 4096-element partial-sum chunk."""
    shapes = [(5000,), (33, 7), (4096,), (3,)]
    names = [f"p{i}" for i in range(len(shapes))]
    w = {n: randn(*s) for n, s in zip(names, shapes)}
    tw = [torch.nn.Parameter(torch.tensor(w[n], dtype=torch.float64)) for n in names]
    topt = torch.optim.AdamW(tw, lr=1e-2, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd)
    opt = rs.AdamW(lr=1e-2, weight_decay=wd)
    params = [(n, w[n]) for n in names]
    for step in range(4):
        grads = {n: randn(*s) * np.float32(0.02 * (step + 1)) for n, s in zip(names, shapes)}
        for p, n in zip(tw, names):
            p.grad = torch.tensor(grads[n], dtype=torch.float64)
        total = float(torch.nn.utils.clip_grad_norm_(tw, max_norm))
        topt.step()
        stats = rs.StepStats(0.0, [], None, False)
        rs.apply_gradients(params, grads, opt, stats, clip_grad_norm=max_norm)
        assert stats.optimizer_step and opt.t == step + 1
        assert abs(stats.grad_norm - total) <= 1e-5 * total
        if total > max_norm:
            assert abs(stats.clip_scale - max_norm / (total + 1e-6)) <= 1e-6 * stats.clip_scale
            for p, n in zip(tw, names):      # the gradients are clipped in place
                np.testing.assert_allclose(grads[n], p.grad.numpy(), rtol=1e-5, atol=1e-9)
        else:
            assert stats.clip_scale is None
        for p, n in zip(tw, names):
            np.testing.assert_allclose(w[n], p.detach().numpy(), rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("bad", [np.nan, np.inf])
def test_apply_gradients_skips_a_non_finite_norm(bad):
    """trainer/src/lib.rs:330-335: a NaN / Inf norm returns before the clip, the schedule and the
    optimizer: weights, moments, t and the schedule stay where they were; the next clean call steps."""
    w = {"a": randn(300), "b": randn(17, 5)}
    params = list(w.items())
    opt = rs.AdamW(lr=1e-2, weight_decay=0.0)
    sched = rs.WarmupCosineScheduler(1e-2, 1e-3, 2, 6)
    stats = rs.StepStats(0.0, [], None, False)
    rs.apply_gradients(params, {n: randn(*v.shape) for n, v in w.items()}, opt, stats, 1.0, sched)
    assert stats.optimizer_step and opt.t == 1.0 and sched.current == 1
    before = ({n: v.copy() for n, v in w.items()}, {n: v.copy() for n, v in opt.m.items()},
              {n: v.copy() for n, v in opt.v.items()}, opt.lr)
    grads = {n: randn(*v.shape) for n, v in w.items()}
    grads["b"][3, 2] = bad
    stats = rs.StepStats(0.0, [], None, False)
    rs.apply_gradients(params, grads, opt, stats, 1.0, sched)
    assert not stats.optimizer_step and not np.isfinite(stats.grad_norm) and stats.clip_scale is None
    assert opt.t == 1.0 and sched.current == 1 and opt.lr == before[3] and stats.lr is None
    for n in w:
        np.testing.assert_array_equal(w[n], before[0][n])
        np.testing.assert_array_equal(opt.m[n], before[1][n])
        np.testing.assert_array_equal(opt.v[n], before[2][n])
    stats = rs.StepStats(0.0, [], None, False)
    rs.apply_gradients(params, {n: randn(*v.shape) for n, v in w.items()}, opt, stats, 1.0, sched)
    assert stats.optimizer_step and opt.t == 2.0 and sched.current == 2


def test_embedding_out_of_range_row_is_zero():
    table = randn(5, 3)
    out = cpu.embedding(table, np.array([[0, 4, 5, 1000]], np.uint32))
    np.testing.assert_array_equal(out[0, 0], table[0])
    np.testing.assert_array_equal(out[0, 1], table[4])
    assert (out[0, 2:] == 0).all()


def test_lr_schedulers_follow_the_reference_curves():
    """The vectors of `schedulers_follow_their_curves` (autograd/src/lib.rs:1914-1941)."""
    cosine = rs.CosineAnnealingLR(1.0, 0.0, 10)
    assert cosine.get_lr() == 1.0
    for _ in range(5):
        cosine.step()
    assert abs(cosine.get_lr() - 0.5) < 1e-6
    for _ in range(5):
        cosine.step()
    assert cosine.get_lr() == 0.0 and cosine.current == 10

    warm = rs.WarmupCosineScheduler(1.0, 0.1, 4, 14)
    lrs = []
    for _ in range(15):
        lrs.append(warm.get_lr())
        warm.step()
    assert lrs[:5] == [0.0, 0.25, 0.5, 0.75, 1.0]
    assert abs(lrs[9] - 0.55) < 1e-6
    assert lrs[14] == np.float32(0.1)
    # monotone: up through the warm-up, down afterwards, never below min_lr
    assert all(a < b for a, b in zip(lrs[:4], lrs[1:5]))
    assert all(a > b for a, b in zip(lrs[4:14], lrs[5:15]))


def test_lora_seed_pinned_values():
    """`lora_seed_is_pinned` (model_builder.rs:869-876)."""
    assert rs.lora_seed(1, "q_proj") == 0x5f28d61921d3ddb3
    assert rs.lora_seed(1, "o_proj") == 0xfabfd7977f143d7c
    assert rs.lora_seed(2, "q_proj") == 0x4bae9242648e2fc1
    assert rs.lora_seed(0, "lm_head") == 0x6d1a1dffacc30def


def test_lora_init_a_is_xorshift64star_uniform():
    """`LoRAAdapter::new_seeded` (graph/src/lib.rs:59-92) at seed 7, in 4, out 3, rank 2. The expected values
    were worked out apart from the oracle, in C with native wrapping 64-bit arithmetic typed from the Rust:
    state0 = (7 * 0x9E3779B97F4A7C15 + (4 << 32 | 3 << 8 | 2)) | 1 = 0x538454167b096795, then per element
    xorshift64* (shifts 12, 25, 27), bits = (state * 0x2545F4914F6CDD1D) >> 40, value = (bits / 2^24 * 2 - 1) / 2.
    A seed other than 0 pins the golden-ratio mixing of the seed. Beyond that the matrix is uniform in
    +-1/sqrt(in), differs between seeds and shapes, and is not rank-1."""
    bits = [0x7b8ec6, 0xb151b4, 0x5238fe, 0x68cc18, 0xaaf8c4, 0xb4f168, 0xfd7741, 0xb72c0e]
    want = np.array([(np.float32(b) / np.float32(1 << 24) * np.float32(2) - np.float32(1)) * np.float32(0.5)
                     for b in bits], np.float32).reshape(4, 2)
    np.testing.assert_array_equal(rs.lora_init_a(4, 3, 2, 7), want)
    np.testing.assert_allclose(want.reshape(-1), [-0.0173527002, 0.192652941, -0.178817868, -0.0906357765,
                                                  0.167858362, 0.206808567, 0.49010092, 0.215515971], rtol=1e-7)
    a = rs.lora_init_a(960, 320, 8, rs.lora_seed(3, "k_proj"))
    bound = 1.0 / math.sqrt(960)
    assert a.shape == (960, 8) and np.all(np.abs(a) <= bound) and abs(float(a.mean())) < 0.05 * bound
    assert abs(float(a.std()) - bound / math.sqrt(3)) < 0.03 * bound          # uniform: sigma = bound / sqrt 3
    assert np.linalg.matrix_rank(a.astype(np.float64)) == 8
    b = rs.lora_init_a(960, 320, 8, rs.lora_seed(4, "k_proj"))
    c = rs.lora_init_a(960, 960, 8, rs.lora_seed(3, "k_proj"))
    assert not np.array_equal(a, b) and not np.array_equal(a, c)
    np.testing.assert_array_equal(a, rs.lora_init_a(960, 320, 8, rs.lora_seed(3, "k_proj")))
