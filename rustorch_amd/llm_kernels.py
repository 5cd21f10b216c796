"""Host-side mirror of the attention part of `LlmKernels`
(crates/rustorch-cuda/src/llm_kernels.rs:874-958): raw device addresses, i32 dims and a stream;
calls enqueue and return."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .device import dev_ptr
from .errors import Overflow, PositionOverflow, raise_for


class LlmKernels:
    def __init__(self):
        L.lib()  # fail here, loudly, if the HIP library is not built

    @staticmethod
    def kv_append_bf16(stream, k_cache, v_cache, k_in, v_in, pos, n_kv, head_dim, max_seq):
        err = L.RtErr()
        raise_for(L.lib().rt_kv_append_bf16(stream, dev_ptr(k_cache), dev_ptr(v_cache), dev_ptr(k_in),
                                            dev_ptr(v_in), pos, n_kv, head_dim, max_seq, C.byref(err)), err)

    @staticmethod
    def qk_norm_rope_kv_append_bf16(stream, q, k_in, v_in, k_cache, v_cache, positions, rope, batch, n_heads, n_kv,
                                    head_dim, max_seq, q_gamma=None, k_gamma=None, eps=1e-6, seq=1):
        """Steps 2a, 2b, 3 of decode_step (crates/rustorch-llm/src/model.rs:575-636) in one launch: per-head
        RMSNorm of q and k (device f32 gammas, or None), half-split RoPE with `rope`'s tables, cache append.
        `seq` new tokens per sequence ([batch, heads, seq, head_dim] buffers; 1 when decoding).  `positions` is a
        device int32[batch] buffer (position of each sequence's first new token), or an int used for every
        sequence (checked on the host)."""
        err = L.RtErr()
        if isinstance(positions, (int, np.integer)):
            pos_ptr, pos = None, int(positions)
            # the reference's checks, before anything touches the device (rope.rs:179-184, kv_cache.rs:88-95)
            if pos < 0 or pos + seq > rope.max_seq:
                raise PositionOverflow(rope.max_seq, pos + seq)
            if pos + seq > max_seq:
                raise Overflow(pos + seq, max_seq)
        else:
            pos_ptr, pos = dev_ptr(positions), 0
        cos, sin = rope.device_tables()
        raise_for(L.lib().rt_qk_norm_rope_kv_append_bf16(
            stream, dev_ptr(q), dev_ptr(k_in), dev_ptr(v_in), dev_ptr(k_cache), dev_ptr(v_cache), pos_ptr, pos,
            dev_ptr(q_gamma) if q_gamma is not None else None, dev_ptr(k_gamma) if k_gamma is not None else None,
            eps, dev_ptr(cos), dev_ptr(sin), rope.max_seq, batch, seq, n_heads, n_kv, head_dim, max_seq, C.byref(err)), err)

    @staticmethod
    def gqa_decode_online_bf16(stream, q, k_cache, v_cache, out, n_heads, n_kv, kv_len, head_dim, max_seq):
        err = L.RtErr()
        raise_for(L.lib().rt_gqa_decode_online_bf16(stream, dev_ptr(q), dev_ptr(k_cache), dev_ptr(v_cache),
                                                    dev_ptr(out), n_heads, n_kv, kv_len, head_dim, max_seq,
                                                    C.byref(err)), err)

    @staticmethod
    def gqa_decode_naive_bf16(stream, q, k_cache, v_cache, out, n_heads, n_kv, kv_len, head_dim, max_seq):
        """llm_kernels.rs:990-1042: the reference's three-pass decode launcher; same function, same kernels here."""
        err = L.RtErr()
        raise_for(L.lib().rt_gqa_decode_naive_bf16(stream, dev_ptr(q), dev_ptr(k_cache), dev_ptr(v_cache),
                                                   dev_ptr(out), n_heads, n_kv, kv_len, head_dim, max_seq,
                                                   C.byref(err)), err)

    @staticmethod
    def gqa_decode_workspace_bytes(batch, n_heads, n_kv, head_dim, max_seq) -> int:
        return L.lib().rt_gqa_decode_workspace_bytes(batch, n_heads, n_kv, head_dim, max_seq)

    @staticmethod
    def gqa_decode_batched_bf16(stream, q, k_cache, v_cache, out, kv_lens, batch, n_heads, n_kv, head_dim, max_seq,
                                workspace, workspace_bytes):
        """Ragged batch: q/out [B,Hq,D], caches [B,Hkv,max_seq,D], kv_lens device int32[B]."""
        err = L.RtErr()
        raise_for(L.lib().rt_gqa_decode_batched_bf16(stream, dev_ptr(q), dev_ptr(k_cache), dev_ptr(v_cache),
                                                     dev_ptr(out), dev_ptr(kv_lens), batch, n_heads, n_kv,
                                                     head_dim, max_seq, dev_ptr(workspace), workspace_bytes,
                                                     C.byref(err)), err)

    @staticmethod
    def gqa_decode_batched_bf16_noalloc(stream, q, k_cache, v_cache, out, kv_lens, batch, n_heads, n_kv, head_dim,
                                        max_seq):
        """gqa_decode_batched_bf16 without a workspace argument: the partials go to a fixed block of device memory
        inside the library, and the call allocates nothing (for callers under graph capture or in loops that must
        not call hipMalloc).  Calls that overlap on one GPU race."""
        err = L.RtErr()
        raise_for(L.lib().rt_gqa_decode_batched_bf16_noalloc(stream, dev_ptr(q), dev_ptr(k_cache), dev_ptr(v_cache),
                                                             dev_ptr(out), dev_ptr(kv_lens), batch, n_heads, n_kv,
                                                             head_dim, max_seq, C.byref(err)), err)

    @staticmethod
    def gqa_decode_chunk_bf16(stream, q, k_cache, v_cache, out, kv_lens, batch, seq_new, n_heads, n_kv, head_dim,
                              max_seq):
        """`seq_new` consecutive new positions per sequence against the cache, causally masked (the bf16, batched form
        of gqa_decode_batched_f32, crates/rustorch-metal/src/kernels.rs:14432-14516): q/out [B,seq_new,Hq,D], caches
        [B,Hkv,max_seq,D] already holding the new positions; `kv_lens` a device int32[B] buffer of key counts that
        include the new positions, or an int used for every sequence."""
        err = L.RtErr()
        if isinstance(kv_lens, (int, np.integer)):
            lens_ptr, kv_len = None, int(kv_lens)
        else:
            lens_ptr, kv_len = dev_ptr(kv_lens), 0
        raise_for(L.lib().rt_gqa_decode_chunk_bf16(stream, dev_ptr(q), dev_ptr(k_cache), dev_ptr(v_cache), dev_ptr(out),
                                                   lens_ptr, kv_len, batch, seq_new, n_heads, n_kv, head_dim, max_seq,
                                                   C.byref(err)), err)
