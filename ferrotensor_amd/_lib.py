"""ctypes binding of libferrotensor_hip.so (the C ABI of include/ferrotensor_hip.h).

The library is the product: there is no fallback. Importing this module
without the built library raises, and every failing call raises FtError with
the library's message.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libferrotensor_hip.so")


class FtError(RuntimeError):
    pass


class AttentionOptionsC(C.Structure):
    _fields_ = [("causal", C.c_int32), ("causal_offset", C.c_uint32), ("window", C.c_uint32),
                ("dropout_prob", C.c_float), ("seed", C.c_uint64)]


class LoraLinearDescC(C.Structure):
    _fields_ = [("w", C.c_void_p), ("w_dtype", C.c_int32), ("t", C.c_void_p), ("b", C.c_void_p),
                ("residual", C.c_void_p), ("y", C.c_void_p), ("N", C.c_size_t), ("r", C.c_size_t),
                ("rope_table", C.c_void_p), ("rope_seq", C.c_size_t)]


class LoraDxDescC(C.Structure):
    _fields_ = [("dy", C.c_void_p), ("w", C.c_void_p), ("w_dtype", C.c_int32), ("dt", C.c_void_p),
                ("a", C.c_void_p), ("N", C.c_size_t), ("r", C.c_size_t)]


class AdamParamsC(C.Structure):
    _fields_ = [("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("eps", C.c_float),
                ("weight_decay", C.c_float), ("t", C.c_float)]


class ModelConfigC(C.Structure):
    _fields_ = [("vocab_size", C.c_uint32), ("hidden_size", C.c_uint32), ("intermediate_size", C.c_uint32),
                ("num_hidden_layers", C.c_uint32), ("num_attention_heads", C.c_uint32),
                ("num_key_value_heads", C.c_uint32), ("rms_norm_eps", C.c_float), ("rope_theta", C.c_float),
                ("tie_word_embeddings", C.c_int32), ("f16_linears", C.c_int32), ("checkpoint_blocks", C.c_int32),
                ("head_all_rows", C.c_int32), ("trainable_base", C.c_int32)]


class TrainerConfigC(C.Structure):
    _fields_ = [("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("eps", C.c_float),
                ("weight_decay", C.c_float), ("clip_grad_norm", C.c_float), ("grad_accum_steps", C.c_uint32),
                ("lr_schedule", C.c_uint32), ("warmup_steps", C.c_uint32), ("total_steps", C.c_uint32),
                ("min_lr", C.c_float)]


class StepStatsC(C.Structure):
    _fields_ = [("loss", C.c_float), ("grad_norm", C.c_float), ("clip_scale", C.c_float),
                ("supervised_tokens", C.c_uint32), ("optimizer_step", C.c_int32), ("lr", C.c_float)]


_P = C.c_void_p
_SZ = C.c_size_t
_F = C.c_float
_I = C.c_int

# name -> argtypes (restype is int unless listed in _RESTYPES)
SIGNATURES = {
    "ft_last_error": [],
    "ft_context_create": [_I, C.POINTER(_P)],
    "ft_context_create_on_stream": [_I, _P, C.POINTER(_P)],
    "ft_context_destroy": [_P],
    "ft_synchronize": [_P],
    "ft_flush": [_P],
    "ft_context_stream": [_P],
    "ft_profile_begin": [_P],
    "ft_profile_end": [_P, C.POINTER(_SZ)],
    "ft_profile_kernel": [_P, _SZ, C.POINTER(C.c_char_p), C.POINTER(C.c_uint64), C.POINTER(C.c_double),
                          C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "ft_mfma_probe": [_P, _SZ, _SZ, _SZ, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "ft_alloc": [_P, _SZ, C.POINTER(_P)],
    "ft_free": [_P, _P],
    "ft_pool_trim": [_P],
    "ft_pool_stats": [_P, C.POINTER(_SZ), C.POINTER(_SZ)],
    "ft_zero": [_P, _P, _SZ],
    "ft_upload": [_P, _P, _P, _SZ],
    "ft_download": [_P, _P, _P, _SZ],
    "ft_upload_f32_as_f16": [_P, _P, _P, _SZ],
    "ft_upload_f32_transposed": [_P, _P, _P, _SZ, _SZ, _I],
    "ft_copy_tensor": [_P, _P, _SZ, _P, _SZ],
    "ft_matmul": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_matmul_bt": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_matmul_at": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_matmul_f16b": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_matmul_bt_f16b": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_lora_down": [_P, _P, _P, _P, _SZ, _SZ, _SZ, _F],
    "ft_lora_linear_group": [_P, _P, C.POINTER(LoraLinearDescC), _SZ, _SZ, _SZ],
    "ft_lora_linear_dx_group": [_P, C.POINTER(LoraDxDescC), _SZ, _P, _P, _SZ, _SZ],
    "ft_rope_table": [_P, _P, _SZ, _SZ, _SZ, _F],
    "ft_rope_apply": [_P, _P, _P, _SZ, _SZ, _SZ, _SZ, _P, _I],
    "ft_mlp_gate_up": [_P, _P, _P, _P, _I, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_mlp_down_backward": [_P, _P, _P, _I, _P, _P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_lora_linear": [_P, _P, _P, _I, _P, _P, _P, _P, _SZ, _SZ, _SZ, _SZ],
    "ft_lora_grad_down": [_P, _P, _P, _P, _SZ, _SZ, _SZ, _F],
    "ft_lora_linear_dx": [_P, _P, _P, _I, _P, _P, _P, _P, _SZ, _SZ, _SZ, _SZ],
    "ft_lora_grad_b": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_lora_grad_a": [_P, _P, _P, _P, _SZ, _SZ, _SZ],
    "ft_rms_norm_eps": [_P, _P, _P, _P, _SZ, _SZ, _F],
    "ft_rms_norm_backward": [_P, _P, _P, _P, _P, _P, _SZ, _SZ, _F],
    "ft_rms_norm_backward_noalloc": [_P, _P, _P, _P, _P, _P, _SZ, _SZ, _F],
    "ft_rope_theta": [_P, _P, _SZ, _SZ, _SZ, _SZ, _SZ, _F],
    "ft_rope_theta_inverse": [_P, _P, _SZ, _SZ, _SZ, _SZ, _SZ, _F],
    "ft_rope_theta_to": [_P, _P, _P, _SZ, _SZ, _SZ, _SZ, _SZ, _F, _I],
    "ft_train_batch_select": [_P, _P, _P, _P, _SZ, _SZ, C.POINTER(_SZ), C.POINTER(_SZ)],
    "ft_train_batch_plan": [_SZ, _SZ, _SZ, C.POINTER(_SZ), C.POINTER(_SZ)],
    "ft_chunk_padded_len": [C.POINTER(_SZ), C.POINTER(_SZ), _SZ, _SZ, C.POINTER(_SZ)],
    "ft_pad_chunk": [C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), C.POINTER(_SZ), C.POINTER(_SZ), C.POINTER(_SZ),
                     _SZ, _SZ, _P, _P, _P],
    "ft_flash_attention_v2_with_stats": [_P, _P, _P, _P, _P, _P, _SZ, _SZ, _SZ, _SZ, _SZ, _SZ,
                                         C.POINTER(AttentionOptionsC)],
    "ft_flash_attention_v2_backward_with_stats": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _SZ, _SZ, _SZ,
                                                  _SZ, _SZ, C.POINTER(AttentionOptionsC)],
    "ft_add": [_P, _P, _P, _P, _SZ],
    "ft_add_backward": [_P, _P, _P, _P, _SZ],
    "ft_silu_gate_fused": [_P, _P, _P, _P, _SZ],
    "ft_silu_gate_backward": [_P, _P, _P, _P, _P, _P, _SZ],
    "ft_gradient_scale": [_P, _P, _SZ, _F],
    "ft_clip_grad_by_norm": [_P, _P, _SZ, _F],
    "ft_gradient_accumulate": [_P, _P, _P, _SZ],
    "ft_sum_squares_partial": [_P, _P, _SZ, _P, _SZ, C.POINTER(_SZ)],
    "ft_masked_cross_entropy_weighted": [_P, _P, _P, _P, _P, _P, _SZ, _SZ, _F],
    "ft_adamw_update": [_P, _P, _P, _P, _P, _SZ, C.POINTER(AdamParamsC)],
    "ft_adamw_update_multi": [_P, C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), C.POINTER(_SZ), _SZ,
                              C.POINTER(AdamParamsC), _F],
    "ft_embedding": [_P, _P, _SZ, _SZ, _P, _SZ, _P],
    "ft_model_create": [_P, C.POINTER(ModelConfigC), C.POINTER(_P)],
    "ft_model_destroy": [_P],
    "ft_model_set_tensor": [_P, C.c_char_p, _P, C.POINTER(_SZ), _I],
    "ft_model_set_lora": [_P, C.c_char_p, _P, _P, _SZ, _F],
    "ft_model_param_count": [_P, C.POINTER(_SZ)],
    "ft_model_param_info": [_P, _SZ, C.POINTER(C.c_char_p), C.POINTER(_SZ)],
    "ft_model_read_param": [_P, _SZ, _P],
    "ft_model_write_param": [_P, _SZ, _P],
    "ft_model_read_grad": [_P, _SZ, _P],
    "ft_model_forward_logits": [_P, _P, _SZ, _SZ, _P],
    "ft_model_eval_chunk": [_P, _P, _P, _P, _SZ, _SZ, _P, _P],
    "ft_trainer_create": [_P, C.POINTER(TrainerConfigC), C.POINTER(_P)],
    "ft_trainer_destroy": [_P],
    "ft_trainer_read_moments": [_P, _SZ, _P, _P],
    "ft_trainer_write_moments": [_P, _SZ, _P, _P],
    "ft_trainer_get_adam_t": [_P, C.POINTER(_F)],
    "ft_trainer_set_adam_t": [_P, _F],
    "ft_trainer_set_adam_hyper": [_P, _F, _F, _F, _F, _F],
    "ft_trainer_optimizer_steps": [_P, C.POINTER(_SZ)],
    "ft_trainer_step_in_accum": [_P, C.POINTER(_SZ)],
    "ft_trainer_set_optimizer_steps": [_P, _SZ],
    "ft_lora_seed": [C.c_uint64, C.c_char_p],
    "ft_lora_init_a": [_P, _SZ, _SZ, _SZ, C.c_uint64],
    "ft_model_add_lora": [_P, C.c_char_p, _SZ, _F],
    "ft_model_set_head_all_rows": [_P, _I],
    "ft_lr_schedule": [C.c_uint32, _F, _F, C.c_uint32, C.c_uint32, C.c_uint32],
    "ft_trainer_train_chunk": [_P, _P, _P, _P, _SZ, _SZ, _I, C.POINTER(StepStatsC), _P],
}
_RESTYPES = {"ft_last_error": C.c_char_p, "ft_context_stream": _P, "ft_lr_schedule": C.c_float, "ft_lora_seed": C.c_uint64}

_lib = None


def load():
    """The loaded library; raises FtError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FtError("%s is missing: build it with `python -m ferrotensor_amd.build` "
                      "(there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, C.c_int)
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        msg = load().ft_last_error()
        raise FtError("ferrotensor_hip error %d: %s" % (rc, msg.decode() if msg else ""))
