"""Host-side mirror of the attention part of `LlmKernels`
(crates/rustorch-cuda/src/llm_kernels.rs:874-958): raw device addresses, i32 dims and a stream;
calls enqueue and return."""
from __future__ import annotations

import ctypes as C

from . import _lib as L
from .device import dev_ptr
from .errors import raise_for


class LlmKernels:
    def __init__(self):
        L.lib()  # fail here, loudly, if the HIP library is not built

    @staticmethod
    def kv_append_bf16(stream, k_cache, v_cache, k_in, v_in, pos, n_kv, head_dim, max_seq):
        err = L.RtErr()
        raise_for(L.lib().rt_kv_append_bf16(stream, dev_ptr(k_cache), dev_ptr(v_cache), dev_ptr(k_in),
                                            dev_ptr(v_in), pos, n_kv, head_dim, max_seq, C.byref(err)), err)

    @staticmethod
    def gqa_decode_online_bf16(stream, q, k_cache, v_cache, out, n_heads, n_kv, kv_len, head_dim, max_seq):
        err = L.RtErr()
        raise_for(L.lib().rt_gqa_decode_online_bf16(stream, dev_ptr(q), dev_ptr(k_cache), dev_ptr(v_cache),
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
