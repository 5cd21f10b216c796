"""rustorch_amd: MI355X (gfx950) attention engine behind rustorch's attention call surfaces.

Host mirror of the reference interface (`attention`, `gqa`, `llm_kernels`) over the C ABI of
librt_attn_hip.so (include/rt_attn.h).  All arithmetic runs in hand-written HIP kernels; there is
no CPU fallback.
"""
from . import _lib
from .attention import (AttentionShape, Mask, flash_backward, flash_backward_f32_dev, flash_backward_saved_f32_dev,
                        flash_forward_stats_f32_dev,
                        flash_backward_workspace_bytes, flash_forward, flash_forward_bf16_dev, flash_forward_bnhd_bf16_dev,
                        flash_forward_bnhd_f32_dev, flash_forward_f32_dev, flash_forward_masked,
                        flash_forward_varlen_bf16_dev, flash_forward_window_bf16_dev, mha_attention_f32, mha_attention_route, mha_flash_forward_f32, mha_forward_masked_bf16_dev, mha_forward_masked_f32_dev,
                        mha_forward_masked_f32)
from .device import (HipStorage, Stream, debug_force_bf16_prefill_kernel, i32_add_dev, init, set_strict_non_finite_v,
                     shutdown, synchronize)
from .errors import (AttentionError, BufferShapeMismatch, DeviceError, GQAError, HeadCountMismatch, KVCacheError,
                     KVWrongInputLen, LayerOutOfRange,
                     MaskError, OutputShapeMismatch, Overflow, PaddingLengthMismatch, PositionOverflow, RoPEError,
                     RopeWrongInputLen, WrongInputLen, ZeroDim)
from .gqa import gqa_forward_f32, gqa_forward_f32_dev
from .kv_cache import KVCache
from .llm_kernels import LlmKernels
from .masks import MASK_NEG, bool_to_additive, causal_mask, sliding_window_mask
from .rope import RoPE

__all__ = [n for n in dir() if not n.startswith("_")]
