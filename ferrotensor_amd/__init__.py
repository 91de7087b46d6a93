"""MI355X (gfx950) implementation of Ferrotensor's LoRA training step.

`engine` mirrors the reference's kernel boundary (ComputeEngine, UnifiedTensor,
context) over the C ABI of include/ferrotensor_hip.h; `trainer` mirrors
Lfm2Model / Trainer over the library's step driver. All arithmetic runs in
libferrotensor_hip.so; there is no CPU path.
"""
from ._lib import FtError, LIB_PATH  # noqa: F401
from .engine import (AdamParams, AttentionOptions, ComputeEngine, DType, HipContext,  # noqa: F401
                     MASKED_CE_SKIP, SUM_SQUARES_CHUNK, UnifiedTensor)
