"""Host-side mirror of `rustorch_nn::gqa` (crates/rustorch-nn/src/gqa.rs:94-210) over the HIP library."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .errors import raise_for


def gqa_forward_f32(q, k, v, out, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim):
    """Same argument order as the reference.  q/out [B,Hq,Sq,D], k/v [B,Hkv,Skv,D], flat f32;
    `out` (numpy f32, C-contiguous) is fully overwritten and returned."""
    def f32(a):
        a = np.ascontiguousarray(np.ravel(a), dtype=np.float32)
        return a, a.ctypes.data_as(C.POINTER(C.c_float))

    q, qp = f32(q)
    k, kp = f32(k)
    v, vp = f32(v)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    err = L.RtErr()
    rc = L.lib().rt_gqa_forward_f32(qp, q.size, kp, k.size, vp, v.size, out.ctypes.data_as(C.POINTER(C.c_float)),
                                    out.size, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, C.byref(err))
    raise_for(rc, err)
    return out


def gqa_forward_f32_dev(q, k, v, out, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, stream=None):
    """The same on device-resident f32 tensors; enqueues on `stream` and returns."""
    from .device import dev_ptr

    err = L.RtErr()
    rc = L.lib().rt_gqa_forward_f32_dev(stream, dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(out), batch, n_heads,
                                        n_kv_heads, seq_q, seq_kv, head_dim, C.byref(err))
    raise_for(rc, err)
