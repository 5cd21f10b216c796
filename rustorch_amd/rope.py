"""Host side of rotary position embeddings: `RoPE` of crates/rustorch-nn/src/rope.rs:33-205.

The tables are built on the host exactly as `RoPE::new` builds them (f32 throughout) and uploaded once; the
device kernel behind `LlmKernels.qk_norm_rope_kv_append_bf16` reads them.  `apply_inplace_half_split` and
`apply_inplace` of the reference are host loops over f32 slices; here they validate like the reference and run
as numpy expressions with the same per-element arithmetic.
"""
from __future__ import annotations

import numpy as np

from .device import HipStorage
from .errors import PositionOverflow, RopeWrongInputLen


class RoPE:
    def __init__(self, head_dim: int, max_seq: int, base: float = 10000.0):
        if head_dim % 2 != 0:
            raise ValueError(f"RoPE: head_dim must be even, got {head_dim}")  # rope.rs:64-68 (a panic there)
        self.head_dim, self.max_seq = head_dim, max_seq
        half = head_dim // 2
        # theta_k = 1 / base^(2k / head_dim), angle = p * theta_k: every step in f32 (rope.rs:72-83).  powf, cos
        # and sin are evaluated in float64 on the f32 argument and rounded, which is what a correctly rounding
        # f32 libm returns (numpy's own float32 routines are a few ulp off, and an ulp of theta is 5e-4 rad at
        # position 8192).
        expo = (2 * np.arange(half)).astype(np.float32) / np.float32(head_dim)
        powed = np.power(np.float64(np.float32(base)), expo.astype(np.float64)).astype(np.float32)
        inv_theta = np.float32(1.0) / powed
        angle = np.arange(max_seq, dtype=np.float32)[:, None] * inv_theta[None, :]
        self.cos = np.cos(angle.astype(np.float64)).astype(np.float32).reshape(-1)
        self.sin = np.sin(angle.astype(np.float64)).astype(np.float32).reshape(-1)
        self._dev = None

    def device_tables(self):
        """(cos, sin) as device buffers, uploaded on first use."""
        if self._dev is None:
            self._dev = (HipStorage.from_numpy(self.cos), HipStorage.from_numpy(self.sin))
        return self._dev

    def _check(self, x, batch, n_heads, seq, position_offset):
        expected = batch * n_heads * seq * self.head_dim
        if x.size != expected:
            raise RopeWrongInputLen(expected, x.size)
        if position_offset + seq > self.max_seq:
            raise PositionOverflow(self.max_seq, position_offset + seq)

    def _tables(self, seq, position_offset):
        half = self.head_dim // 2
        sl = slice(position_offset * half, (position_offset + seq) * half)
        return self.cos[sl].reshape(1, 1, seq, half), self.sin[sl].reshape(1, 1, seq, half)

    def apply_inplace_half_split(self, x: np.ndarray, batch: int, n_heads: int, seq: int, position_offset: int):
        """rope.rs:162-205 on a float32 array viewed as [batch, n_heads, seq, head_dim]."""
        self._check(x, batch, n_heads, seq, position_offset)
        half = self.head_dim // 2
        v = x.reshape(batch, n_heads, seq, self.head_dim)
        c, s = self._tables(seq, position_offset)
        x0, x1 = v[..., :half].copy(), v[..., half:].copy()
        v[..., :half] = x0 * c - x1 * s
        v[..., half:] = x1 * c + x0 * s

    def apply_inplace(self, x: np.ndarray, batch: int, n_heads: int, seq: int, position_offset: int):
        """rope.rs:96-142: pairs (2k, 2k+1)."""
        self._check(x, batch, n_heads, seq, position_offset)
        v = x.reshape(batch, n_heads, seq, self.head_dim)
        c, s = self._tables(seq, position_offset)
        x0, x1 = v[..., 0::2].copy(), v[..., 1::2].copy()
        v[..., 0::2] = x0 * c - x1 * s
        v[..., 1::2] = x0 * s + x1 * c
