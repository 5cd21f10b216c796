"""Additive attention masks of crates/rustorch-nn/src/masks.rs:22-80: 0.0 keeps a position, MASK_NEG (-1e4, not
-inf, so that a fully masked row softmaxes to finite weights instead of NaN) masks it.  Plain float32 arrays, to be
passed as `attn_mask` to `mha_forward_masked_f32`."""
from __future__ import annotations

import numpy as np

MASK_NEG = np.float32(-1.0e4)


def causal_mask(seq_len: int) -> np.ndarray:
    """[seq_len, seq_len]: 0 where j <= i, MASK_NEG above the diagonal (masks.rs:30-40)."""
    i = np.arange(seq_len)[:, None]
    j = np.arange(seq_len)[None, :]
    return np.where(j > i, MASK_NEG, np.float32(0.0)).astype(np.float32)


def sliding_window_mask(seq_len: int, window: int) -> np.ndarray:
    """[seq_len, seq_len]: 0 iff j <= i and i - j < window (masks.rs:52-65); window must be >= 1."""
    if window < 1:
        raise ValueError("sliding_window_mask: window must be >= 1")  # an assert (panic) in the reference
    i = np.arange(seq_len)[:, None]
    j = np.arange(seq_len)[None, :]
    keep = (j <= i) & (np.maximum(i - j, 0) < window)
    return np.where(keep, np.float32(0.0), MASK_NEG).astype(np.float32)


def bool_to_additive(mask) -> np.ndarray:
    """Keep-mask with values in {0.0, 1.0} -> additive bias: 0.0 where the value is >= 0.5, MASK_NEG elsewhere
    (masks.rs:73-82); the shape is kept."""
    m = np.asarray(mask, dtype=np.float32)
    return np.where(m >= 0.5, np.float32(0.0), MASK_NEG).astype(np.float32)
