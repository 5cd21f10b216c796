"""Host-side mirror of `rustorch_attention` (crates/rustorch-attention/src/{cpu_forward,mask}.rs)
over the HIP library: same names, argument meaning and errors; the arithmetic runs on the GPU.

    shape = AttentionShape.new(B, H, N, D)
    out = flash_forward_masked(shape, q, k, v, Mask.causal())      # numpy f32 in, numpy f32 out
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib as L
from .device import dev_ptr
from .errors import raise_for


@dataclass
class AttentionShape:
    """cpu_forward.rs:49-89."""
    batch: int
    heads: int
    seq: int
    dim: int
    br: int = 64
    bc: int = 64

    @classmethod
    def new(cls, batch, heads, seq, dim):
        return cls(batch, heads, seq, dim, 64, 64)

    def buffer_len(self) -> int:
        return self.batch * self.heads * self.seq * self.dim

    def strides(self):
        s_n = self.dim
        s_h = self.seq * s_n
        return self.heads * s_h, s_h, s_n

    def _c(self):
        return L.RtShape(self.batch, self.heads, self.seq, self.dim, self.br, self.bc)


class Mask:
    """mask.rs:26-66: Mask::None | Mask::Causal | Mask::Padding(keep)."""

    def __init__(self, kind: int, keep=None):
        self.kind = kind
        self.keep = None if keep is None else np.ascontiguousarray(np.asarray(keep, dtype=np.bool_)).view(np.uint8)

    @classmethod
    def none(cls):
        return cls(L.RT_MASK_NONE)

    @classmethod
    def causal(cls):
        return cls(L.RT_MASK_CAUSAL)

    @classmethod
    def padding(cls, keep):
        return cls(L.RT_MASK_PADDING, keep)

    def is_masked(self, qi: int, kj: int) -> bool:
        if self.kind == L.RT_MASK_CAUSAL:
            return kj > qi
        if self.kind == L.RT_MASK_PADDING:
            return kj < self.keep.size and not self.keep[kj]
        return False


def _f32(a):
    a = np.ascontiguousarray(np.ravel(a), dtype=np.float32)
    return a, a.ctypes.data_as(C.POINTER(C.c_float))


def flash_forward_masked(shape: AttentionShape, q, k, v, mask: Mask, out=None):
    """cpu_forward.rs:193-242.  q, k, v: flat f32 [B,H,N,D]; returns (and fills) flat f32 `out`."""
    q, qp = _f32(q)
    k, kp = _f32(k)
    v, vp = _f32(v)
    if out is None:
        out = np.zeros(shape.buffer_len(), dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    keep_p, keep_n = None, 0
    if mask.kind == L.RT_MASK_PADDING:
        keep_p, keep_n = mask.keep.ctypes.data_as(C.POINTER(C.c_uint8)), mask.keep.size
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_masked_f32(C.byref(s), qp, q.size, kp, k.size, vp, v.size, mask.kind, keep_p,
                                             keep_n, out.ctypes.data_as(C.POINTER(C.c_float)), out.size,
                                             C.byref(err))
    raise_for(rc, err)
    return out


def flash_forward(shape: AttentionShape, q, k, v, out=None):
    """cpu_forward.rs:175-183."""
    return flash_forward_masked(shape, q, k, v, Mask.none(), out)


def flash_backward(shape: AttentionShape, q, k, v, d_out, dq=None, dk=None, dv=None):
    """rustorch_attention::flash_backward (crates/rustorch-attention/src/cpu_backward.rs:46-185): gradients of
    unmasked attention.  q, k, v, d_out: flat f32 [B,H,N,D]; fills (overwrites) and returns flat f32 (dq, dk, dv)."""
    ins = [_f32(a) for a in (q, k, v, d_out)]
    outs = [np.zeros(shape.buffer_len(), dtype=np.float32) if o is None else o for o in (dq, dk, dv)]
    args = []
    for a, ptr in ins:
        args += [ptr, a.size]
    for o in outs:
        assert o.dtype == np.float32 and o.flags.c_contiguous
        args += [o.ctypes.data_as(C.POINTER(C.c_float)), o.size]
    err = L.RtErr()
    s = shape._c()
    raise_for(L.lib().rt_flash_backward_f32(C.byref(s), *args, C.byref(err)), err)
    return tuple(outs)


def flash_backward_workspace_bytes(shape: AttentionShape) -> int:
    s = shape._c()
    return int(L.lib().rt_flash_backward_workspace_bytes(C.byref(s)))


def flash_backward_f32_dev(shape, q, k, v, d_out, dq, dk, dv, workspace, workspace_bytes, stream=None):
    """flash_backward on device-resident f32 [B,H,N,D] tensors; enqueues on `stream` and returns."""
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_backward_f32_dev(stream, C.byref(s), dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(d_out),
                                           dev_ptr(dq), dev_ptr(dk), dev_ptr(dv), dev_ptr(workspace),
                                           workspace_bytes, C.byref(err))
    raise_for(rc, err)


def flash_forward_stats_f32_dev(shape, q, k, v, out, lse, stream=None):
    """Unmasked f32 forward that also writes lse[b,h,i] = m_i + ln(l_i): what flash_backward_saved_f32_dev takes back."""
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_stats_f32_dev(stream, C.byref(s), dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(out),
                                                dev_ptr(lse), C.byref(err))
    raise_for(rc, err)


def flash_backward_saved_f32_dev(shape, q, k, v, out, lse, d_out, dq, dk, dv, workspace, workspace_bytes, stream=None):
    """The backward from a saved forward (cpu_backward.rs:3-4, :29-35); workspace: batch*heads*seq floats."""
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_backward_saved_f32_dev(stream, C.byref(s), dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(out),
                                                 dev_ptr(lse), dev_ptr(d_out), dev_ptr(dq), dev_ptr(dk), dev_ptr(dv),
                                                 dev_ptr(workspace), workspace_bytes, C.byref(err))
    raise_for(rc, err)


# ---- device-resident tensors (torch GPU tensors, HipStorage, or raw addresses) ---------------------------


def flash_forward_f32_dev(shape, q, k, v, out, mask: Mask = None, keep_dev=None, n_kv_heads=0, stream=None):
    mask = mask or Mask.none()
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_f32_dev(stream, C.byref(s), n_kv_heads, dev_ptr(q), dev_ptr(k), dev_ptr(v),
                                          mask.kind, dev_ptr(keep_dev), dev_ptr(out), C.byref(err))
    raise_for(rc, err)


def flash_forward_bf16_dev(shape, q, k, v, out, mask: Mask = None, keep_dev=None, n_kv_heads=0, stream=None):
    """bf16 [B,H,N,D] device tensors; enqueues on `stream` and returns."""
    mask = mask or Mask.none()
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_bf16_dev(stream, C.byref(s), n_kv_heads, dev_ptr(q), dev_ptr(k), dev_ptr(v),
                                           mask.kind, dev_ptr(keep_dev), dev_ptr(out), C.byref(err))
    raise_for(rc, err)


def flash_forward_window_bf16_dev(shape, q, k, v, out, window: int, n_kv_heads=0, bnhd=False, stream=None):
    """Causal attention with a sliding window (position i sees keys j <= i with i - j < window: the mask of
    rustorch_nn::masks::sliding_window_mask, crates/rustorch-nn/src/masks.rs:41-60, never materialised) on bf16 device
    tensors [B,H,N,D], or [B,N,H,D] with `bnhd`.  Enqueues on `stream` and returns."""
    err = L.RtErr()
    s = shape._c()
    fn = L.lib().rt_flash_forward_window_bnhd_bf16_dev if bnhd else L.lib().rt_flash_forward_window_bf16_dev
    raise_for(fn(stream, C.byref(s), n_kv_heads, dev_ptr(q), dev_ptr(k), dev_ptr(v), int(window), dev_ptr(out),
                 C.byref(err)), err)


def flash_forward_varlen_bf16_dev(shape, q, k, v, seq_lens_dev, out, zero_padded_rows=True, n_kv_heads=0,
                                  stream=None):
    """Padded-batch causal prefill: per-sequence valid lengths (device int32[batch])."""
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_varlen_bf16_dev(stream, C.byref(s), n_kv_heads, dev_ptr(q), dev_ptr(k),
                                                  dev_ptr(v), dev_ptr(seq_lens_dev), int(bool(zero_padded_rows)),
                                                  dev_ptr(out), C.byref(err))
    raise_for(rc, err)


# ---- [batch, seq, heads, dim] tensors: the layout MultiHeadAttention keeps its projections in --------------


def mha_flash_forward_f32(q, k, v, batch: int, seq: int, heads: int, head_dim: int, out=None):
    """rustorch_nn::attention::mha_flash_forward_f32 (crates/rustorch-nn/src/attention.rs:452-495): q, k, v flat
    f32 [B,T,H,hd]; returns flat f32 [B,T,H*hd].  Unmasked attention per (batch, head); no transposed copies."""
    q, qp = _f32(q)
    k, kp = _f32(k)
    v, vp = _f32(v)
    if out is None:
        out = np.zeros(batch * seq * heads * head_dim, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    err = L.RtErr()
    rc = L.lib().rt_mha_flash_forward_f32(qp, q.size, kp, k.size, vp, v.size,
                                          out.ctypes.data_as(C.POINTER(C.c_float)), out.size, batch, seq, heads,
                                          head_dim, C.byref(err))
    raise_for(rc, err)
    return out


def mha_forward_masked_f32(q, k, v, batch: int, t_q: int, t_kv: int, heads: int, head_dim: int, attn_mask=None,
                           out=None):
    """Steps 2-8 of `MultiHeadAttention::forward`'s composed path (crates/rustorch-nn/src/attention.rs:371-399):
    softmax((Q.K^T)/sqrt(hd) + attn_mask).V per (batch, head) on the projected tensors q [B,t_q,H*hd], k, v
    [B,t_kv,H*hd] (flat f32; t_q != t_kv is cross-attention).  `attn_mask` is an additive f32 bias with t_q*t_kv
    ([T,T] / [1,T,T]) or B*H*t_q*t_kv ([B*H,T,T]) elements, e.g. from `masks.causal_mask`, or None.  Returns flat
    f32 [B,t_q,H*hd]."""
    q, qp = _f32(q)
    k, kp = _f32(k)
    v, vp = _f32(v)
    m, mp = (None, None) if attn_mask is None else _f32(np.ravel(attn_mask))
    if out is None:
        out = np.zeros(batch * t_q * heads * head_dim, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    err = L.RtErr()
    rc = L.lib().rt_mha_forward_masked_f32(qp, q.size, kp, k.size, vp, v.size, mp, 0 if m is None else m.size,
                                           out.ctypes.data_as(C.POINTER(C.c_float)), out.size, batch, t_q, t_kv, heads,
                                           head_dim, C.byref(err))
    raise_for(rc, err)
    return out


def mha_forward_masked_f32_dev(q, k, v, out, batch: int, t_q: int, t_kv: int, heads: int, head_dim: int, attn_mask=None,
                               mask_len: int = 0, stream=None):
    """`mha_forward_masked_f32` on device-resident f32 tensors ([B,t,H*hd]); `attn_mask` is a device buffer of
    `mask_len` elements (t_q*t_kv or B*H*t_q*t_kv) or None.  Enqueues on `stream` and returns."""
    err = L.RtErr()
    rc = L.lib().rt_mha_forward_masked_f32_dev(stream, dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(attn_mask),
                                               mask_len if attn_mask is not None else 0, dev_ptr(out), batch, t_q, t_kv,
                                               heads, head_dim, C.byref(err))
    raise_for(rc, err)


def mha_forward_masked_bf16_dev(q, k, v, out, batch: int, t_q: int, t_kv: int, heads: int, head_dim: int, attn_mask=None,
                                mask_len: int = 0, stream=None):
    """The same composed path on bf16 device tensors ([B,t,H*hd] bit patterns) with an f32 device mask of `mask_len`
    elements (t_q*t_kv or B*H*t_q*t_kv) or None; bf16 out.  Enqueues on `stream` and returns."""
    err = L.RtErr()
    rc = L.lib().rt_mha_forward_masked_bf16_dev(stream, dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(attn_mask),
                                                mask_len if attn_mask is not None else 0, dev_ptr(out), batch, t_q, t_kv,
                                                heads, head_dim, C.byref(err))
    raise_for(rc, err)


def mha_attention_route(t_q: int, t_kv: int, has_mask: bool) -> str:
    """Which branch `MultiHeadAttention::forward` takes for the attention between its projections, under no_grad on
    contiguous f32 tensors (crates/rustorch-nn/src/attention.rs:325-333, :347-356): "identity" for the single-token
    shortcut (softmax over one position is 1, the context is V), "flash" for unmasked self-attention of equal lengths,
    "composed" when a mask is given or the lengths differ."""
    if not has_mask and t_q == 1 and t_kv == 1:
        return "identity"
    if not has_mask and t_q == t_kv:
        return "flash"
    return "composed"


def mha_attention_f32(q, k, v, batch: int, t_q: int, t_kv: int, heads: int, head_dim: int, attn_mask=None):
    """The attention between the projections of `MultiHeadAttention::forward` with the reference's routing
    (attention.rs:325-399): projected q [B,t_q,H*hd], k, v [B,t_kv,H*hd] -> context [B,t_q,H*hd], flat f32."""
    route = mha_attention_route(t_q, t_kv, attn_mask is not None)
    if route == "identity":
        v, _ = _f32(v)
        if v.size != batch * heads * head_dim:
            raise ValueError(f"v has {v.size} elements, expected {batch * heads * head_dim}")
        return v.copy()
    if route == "flash":
        return mha_flash_forward_f32(q, k, v, batch, t_q, heads, head_dim)
    return mha_forward_masked_f32(q, k, v, batch, t_q, t_kv, heads, head_dim, attn_mask)


def flash_forward_bnhd_f32_dev(shape, q, k, v, out, mask: Mask = None, keep_dev=None, n_kv_heads=0, stream=None):
    """f32 [B,N,H,D] device tensors (k, v: [B,N,Hkv,D]); `shape` is still (batch, heads, seq, dim)."""
    mask = mask or Mask.none()
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_bnhd_f32_dev(stream, C.byref(s), n_kv_heads, dev_ptr(q), dev_ptr(k), dev_ptr(v),
                                               mask.kind, dev_ptr(keep_dev), dev_ptr(out), C.byref(err))
    raise_for(rc, err)


def flash_forward_bnhd_bf16_dev(shape, q, k, v, out, mask: Mask = None, keep_dev=None, n_kv_heads=0, stream=None):
    """bf16 [B,N,H,D] device tensors (k, v: [B,N,Hkv,D]); `shape` is still (batch, heads, seq, dim)."""
    mask = mask or Mask.none()
    err = L.RtErr()
    s = shape._c()
    rc = L.lib().rt_flash_forward_bnhd_bf16_dev(stream, C.byref(s), n_kv_heads, dev_ptr(q), dev_ptr(k), dev_ptr(v),
                                                mask.kind, dev_ptr(keep_dev), dev_ptr(out), C.byref(err))
    raise_for(rc, err)
