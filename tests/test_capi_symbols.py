"""The C-ABI library loads and exports every symbol include/ferrotensor_hip.h declares
(no compute calls: runs without a GPU), and fails loudly when asked for a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ferrotensor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ft_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_hot_compute_engine_methods():
    syms = declared_symbols()
    for name in ["ft_matmul", "ft_matmul_bt", "ft_matmul_at", "ft_matmul_f16b", "ft_matmul_bt_f16b",
                 "ft_rms_norm_eps", "ft_rms_norm_backward", "ft_rope_theta", "ft_rope_theta_inverse",
                 "ft_flash_attention_v2_with_stats", "ft_flash_attention_v2_backward_with_stats", "ft_add",
                 "ft_add_backward", "ft_silu_gate_fused", "ft_silu_gate_backward", "ft_gradient_scale",
                 "ft_clip_grad_by_norm", "ft_sum_squares_partial", "ft_masked_cross_entropy_weighted",
                 "ft_adamw_update", "ft_copy_tensor", "ft_synchronize", "ft_trainer_train_chunk"]:
        assert name in syms, name


def test_library_exports_every_declared_symbol():
    from ferrotensor_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing
    # and the ctypes table covers the header
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_no_cpu_fallback_without_a_device():
    """Without a GPU the product raises; it never computes on the host."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from ferrotensor_amd import FtError, HipContext
    with pytest.raises(FtError):
        HipContext(0)


def test_product_does_not_import_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "ferrotensor_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("the oracle", ""), os.path.join(dirpath, f)


def test_lr_schedule_entry_point_matches_the_oracle():
    """ft_lr_schedule is host arithmetic (no GPU): compared with the restated schedulers step by step."""
    from ferrotensor_amd.trainer import lr_schedule
    from oracle import reference_step as rs
    import numpy as np
    for peak, low, warm, total in [(1.0, 0.1, 4, 14), (2e-4, 2e-5, 100, 1000), (3e-4, 0.0, 0, 50), (1e-3, 1e-4, 7, 7)]:
        w = rs.WarmupCosineScheduler(peak, low, warm, total)
        c = rs.CosineAnnealingLR(peak, low, total)
        for k in range(total + 3):
            got = lr_schedule("warmup_cosine", peak, low, warm, total, k)
            assert abs(got - w.get_lr()) <= 2e-7 * peak, (peak, low, warm, total, k, got, w.get_lr())
            got = lr_schedule("cosine", peak, low, warm, total, k)
            assert abs(got - c.get_lr()) <= 2e-7 * peak
            assert lr_schedule("constant", peak, low, warm, total, k) == np.float32(peak)
            w.step()
            c.step()


def test_lora_seed_and_init_entry_points_are_bit_exact():
    """Integer hashing and the xorshift64* draws (host arithmetic, no GPU) against the reference's pinned
    seeds and against the restated generator, bit for bit."""
    from ferrotensor_amd.trainer import lora_seed, lora_init_a
    from oracle import reference_step as rs
    import numpy as np
    assert lora_seed(1, "q_proj") == 0x5f28d61921d3ddb3
    assert lora_seed(1, "o_proj") == 0xfabfd7977f143d7c
    assert lora_seed(2, "q_proj") == 0x4bae9242648e2fc1
    assert lora_seed(0, "lm_head") == 0x6d1a1dffacc30def
    for in_dim, out_dim, rank, seed in [(1, 0, 1, 0), (32, 64, 4, 7), (960, 320, 8, lora_seed(3, "k_proj")),
                                        (576, 1536, 16, lora_seed(30, "up_proj"))]:
        np.testing.assert_array_equal(lora_init_a(in_dim, out_dim, rank, seed),
                                      rs.lora_init_a(in_dim, out_dim, rank, seed))
