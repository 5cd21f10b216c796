"""Device-resident mirror of `KVCache` / `KVLayerCache` (crates/rustorch-nn/src/kv_cache.rs:49-256).

Same object protocol as the reference -- `append(layer, seq_added, new_k, new_v)` for every layer, then
`advance(seq_added)` -- with the per-layer `[batch, n_heads, max_seq, head_dim]` buffers living in HBM (bf16 by
default, the storage type of the decode kernels; f32 on request) and the copies enqueued on a stream.  The
buffers are what `LlmKernels.gqa_decode_batched_bf16` and `qk_norm_rope_kv_append_bf16` take as caches: nothing
is trimmed or copied out before attention.
"""
from __future__ import annotations

import ctypes as C

from . import _lib as L
from .device import HipStorage, dev_ptr
from .errors import LayerOutOfRange, Overflow, raise_for

_ELEM = {"bf16": 2, "f32": 4}


class KVCache:
    def __init__(self, num_layers: int, batch: int, n_heads: int, head_dim: int, max_seq: int, dtype: str = "bf16"):
        """`KVCache::new` (kv_cache.rs:131-146; note the argument order: head_dim before max_seq).  The buffers
        start zeroed, like the reference's `vec![0.0; n]`."""
        if dtype not in _ELEM:
            raise ValueError(f"dtype must be 'bf16' or 'f32', got {dtype!r}")
        self.dtype, self.elem_bytes = dtype, _ELEM[dtype]
        self._dims = (batch, n_heads, max_seq, head_dim)
        self._max_seq = max_seq
        self._current_len = 0
        n_bytes = batch * n_heads * max_seq * head_dim * self.elem_bytes
        self._layers = [(HipStorage.zeros(n_bytes), HipStorage.zeros(n_bytes)) for _ in range(num_layers)]

    def num_layers(self) -> int:
        return len(self._layers)

    def max_seq(self) -> int:
        return self._max_seq

    def current_len(self) -> int:
        return self._current_len

    def clear(self) -> None:
        """Length back to zero; contents become stale, the allocation stays (kv_cache.rs:165-167)."""
        self._current_len = 0

    def append(self, layer_idx: int, seq_added: int, new_k, new_v, stream=None) -> None:
        """kv_cache.rs:172-190 then :77-112.  new_k / new_v are device buffers (`HipStorage`) holding
        `[batch, n_heads, seq_added, head_dim]` elements of the cache's dtype; their element counts are checked
        like the reference checks slice lengths."""
        if not 0 <= layer_idx < len(self._layers):
            raise LayerOutOfRange(layer_idx, len(self._layers))
        batch, n_heads, max_seq, head_dim = self._dims
        k, v = self._layers[layer_idx]
        err = L.RtErr()
        raise_for(L.lib().rt_kv_cache_append_dev(stream, dev_ptr(k), dev_ptr(v), dev_ptr(new_k),
                                                 new_k.byte_len // self.elem_bytes, dev_ptr(new_v),
                                                 new_v.byte_len // self.elem_bytes, batch, n_heads, max_seq, head_dim,
                                                 self._current_len, seq_added, self.elem_bytes, C.byref(err)), err)

    def advance(self, seq_added: int) -> None:
        """kv_cache.rs:194-204."""
        new_len = self._current_len + seq_added
        if new_len > self._max_seq:
            raise Overflow(new_len, self._max_seq)
        self._current_len = new_len

    def k_buffer(self, layer_idx: int):
        """The full `[batch, n_heads, max_seq, head_dim]` device buffer of the layer, or None (kv_cache.rs:210-212)."""
        return self._layers[layer_idx][0] if 0 <= layer_idx < len(self._layers) else None

    def v_buffer(self, layer_idx: int):
        return self._layers[layer_idx][1] if 0 <= layer_idx < len(self._layers) else None

    def dims(self):
        """`(batch, n_heads, max_seq, head_dim)`, or None without layers (kv_cache.rs:223-226)."""
        return self._dims if self._layers else None
