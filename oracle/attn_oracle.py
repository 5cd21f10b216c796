"""ctypes binding of the CPU oracle (``libattn_oracle.so``, built from ``attn_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker.  The shipped
package (``rustorch_amd``) never imports it.

Each wrapper keeps the name of the reference function it restates
(``crates/rustorch-attention/src/cpu_forward.rs``, ``mask.rs``,
``online_softmax.rs``; ``crates/rustorch-nn/src/gqa.rs``, ``kv_cache.rs``;
``crates/rustorch-cuda/src/llm_kernels.rs``); the C file cites the lines.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libattn_oracle.so")

MASK_NONE, MASK_CAUSAL, MASK_PADDING = 0, 1, 2

OK = 0
ERR_ZERO_DIM = 1
ERR_BUFFER_SHAPE_MISMATCH = 2
ERR_OUTPUT_SHAPE_MISMATCH = 3
ERR_PADDING_LENGTH_MISMATCH = 4
ERR_HEAD_COUNT_MISMATCH = 5
ERR_WRONG_INPUT_LEN = 6
ERR_KV_OVERFLOW = 7
ERR_KV_WRONG_INPUT_LEN = 8
ERR_ROPE_WRONG_INPUT_LEN = 9
ERR_ROPE_POSITION_OVERFLOW = 10

WHICH = {0: "q", 1: "k", 2: "v", 3: "out", 4: "flash_forward", 6: "do", -1: ""}


class _Shape(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("batch", "heads", "seq", "dim", "br", "bc")]


class _Err(C.Structure):
    _fields_ = [("which", C.c_int32), ("expected", C.c_uint64), ("got", C.c_uint64), ("got2", C.c_uint64)]


class _Osm(C.Structure):
    _fields_ = [("m", C.c_float), ("l", C.c_float)]


@dataclass
class OracleError(Exception):
    code: int
    which: str = ""
    expected: int = 0
    got: int = 0
    got2: int = 0

    def __str__(self):
        return f"oracle error code={self.code} which={self.which!r} expected={self.expected} got={self.got}"


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile (gcc); returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        fp, u8p, u16p, i32p = (C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_uint16),
                               C.POINTER(C.c_int32))
        sz = C.c_size_t
        fwd_args = [C.POINTER(_Shape), fp, sz, fp, sz, fp, sz, C.c_int, u8p, sz, fp, sz, C.POINTER(_Err)]
        L.ro_flash_forward_masked.argtypes = fwd_args + [C.c_int]
        L.ro_flash_forward_scalar.argtypes = fwd_args
        L.ro_naive_forward_masked.argtypes = fwd_args
        L.ro_mask_is_masked.argtypes = [C.c_int, u8p, sz, sz, sz]
        L.ro_gqa_forward_f32.argtypes = [fp, sz, fp, sz, fp, sz, fp, sz, sz, sz, sz, sz, sz, sz, C.POINTER(_Err),
                                         C.c_int]
        L.ro_kv_cache_append.argtypes = [fp, fp, sz, sz, sz, sz, sz, sz, fp, sz, fp, sz, C.POINTER(_Err)]
        L.ro_kv_trim.argtypes = [fp, fp, sz, sz, sz, sz]
        L.ro_kv_trim.restype = None
        L.ro_f32_to_bf16_array.argtypes = [fp, u16p, sz]
        L.ro_f32_to_bf16_array.restype = None
        L.ro_bf16_to_f32_array.argtypes = [u16p, fp, sz]
        L.ro_bf16_to_f32_array.restype = None
        L.ro_kv_append_bf16.argtypes = [u16p, u16p, u16p, u16p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.ro_kv_append_bf16.restype = None
        L.ro_gqa_decode_online_bf16.argtypes = [u16p, u16p, u16p, u16p] + [C.c_int] * 5
        L.ro_gqa_decode_online_bf16.restype = None
        L.ro_gqa_decode_batched_bf16.argtypes = [u16p, u16p, u16p, i32p, fp] + [C.c_int] * 6
        L.ro_gqa_decode_batched_bf16.restype = None
        L.ro_gqa_decode_chunk_bf16.argtypes = [u16p, u16p, u16p, i32p, fp] + [C.c_int] * 7
        L.ro_gqa_decode_chunk_bf16.restype = None
        for name in ("ro_osm_empty",):
            getattr(L, name).argtypes = [C.POINTER(_Osm)]
            getattr(L, name).restype = None
        L.ro_osm_from_scalar.argtypes = [C.POINTER(_Osm), C.c_float]
        L.ro_osm_from_scalar.restype = None
        L.ro_osm_absorb.argtypes = [C.POINTER(_Osm), C.c_float]
        L.ro_osm_absorb.restype = None
        L.ro_osm_is_empty.argtypes = [C.POINTER(_Osm)]
        L.ro_osm_combine.argtypes = [C.POINTER(_Osm)] * 3
        L.ro_osm_combine.restype = None
        L.ro_osm_full.argtypes = [fp, sz, C.POINTER(_Osm)]
        L.ro_osm_full.restype = None
        L.ro_max_threads.restype = C.c_int
        L.ro_causal_mask.argtypes = [sz, fp]
        L.ro_causal_mask.restype = None
        L.ro_sliding_window_mask.argtypes = [sz, sz, fp]
        L.ro_sliding_window_mask.restype = None
        L.ro_bool_to_additive.argtypes = [fp, fp, sz]
        L.ro_bool_to_additive.restype = None
        L.ro_softmax_row.argtypes = [fp, fp, sz]
        L.ro_softmax_row.restype = None
        L.ro_mha_forward_masked.argtypes = [fp, fp, fp, fp, sz, fp, sz, sz, sz, sz, sz]
        L.ro_mha_forward_masked.restype = None
        L.ro_rope_tables.argtypes = [C.c_int, C.c_int, C.c_float, fp, fp]
        L.ro_rope_tables.restype = None
        rope_args = [fp, sz, sz, sz, sz, sz, sz, fp, fp, sz, C.POINTER(_Err)]
        L.ro_rope_half_split.argtypes = rope_args
        L.ro_rope_interleaved.argtypes = rope_args
        L.ro_rms_norm_per_head.argtypes = [fp, fp, sz, sz, C.c_float]
        L.ro_rms_norm_per_head.restype = None
        L.ro_decode_prepare_bf16.argtypes = [u16p, u16p, u16p, u16p, u16p, i32p, fp, fp, C.c_float, fp, fp] + \
            [C.c_int] * 7 + [C.POINTER(_Err)]
        L.ro_flash_backward.argtypes = [C.POINTER(_Shape)] + [fp, sz] * 7 + [C.POINTER(_Err)]
        _lib = L
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(C.POINTER(C.c_float))


def _raise(code, err):
    if code != OK:
        raise OracleError(code, WHICH.get(err.which, ""), err.expected, err.got, err.got2)


@dataclass
class AttentionShape:
    """``AttentionShape`` of cpu_forward.rs:49-89 (``new`` => br = bc = 64)."""
    batch: int
    heads: int
    seq: int
    dim: int
    br: int = 64
    bc: int = 64

    def buffer_len(self) -> int:
        return self.batch * self.heads * self.seq * self.dim

    def _c(self):
        return _Shape(self.batch, self.heads, self.seq, self.dim, self.br, self.bc)


def _mask_args(mask):
    """mask: None | "causal" | ("padding", keep-array)."""
    if mask is None or mask == "none":
        return MASK_NONE, None, 0, None
    if mask == "causal":
        return MASK_CAUSAL, None, 0, None
    kind, keep = mask
    assert kind == "padding"
    keep = np.ascontiguousarray(np.asarray(keep, dtype=np.uint8))
    return MASK_PADDING, keep.ctypes.data_as(C.POINTER(C.c_uint8)), keep.size, keep


def _forward(fn, shape, q, k, v, mask, out_len, extra):
    q, qp = _f32(np.ravel(q))
    k, kp = _f32(np.ravel(k))
    v, vp = _f32(np.ravel(v))
    n_out = shape.buffer_len() if out_len is None else out_len
    out = np.zeros(n_out, dtype=np.float32)
    kind, keep_p, keep_n, _keep = _mask_args(mask)
    err = _Err()
    s = shape._c()
    code = fn(C.byref(s), qp, q.size, kp, k.size, vp, v.size, kind, keep_p, keep_n,
              out.ctypes.data_as(C.POINTER(C.c_float)), out.size, C.byref(err), *extra)
    _raise(code, err)
    return out


def flash_forward_masked(shape, q, k, v, mask=None, threads=None, out_len=None):
    """cpu_forward.rs:193-425 (tiled forward).  Returns the flat ``out`` array."""
    t = lib().ro_max_threads() if threads is None else threads
    return _forward(lib().ro_flash_forward_masked, shape, q, k, v, mask, out_len, (t,))


def flash_forward(shape, q, k, v, threads=None, out_len=None):
    """cpu_forward.rs:175-183."""
    return flash_forward_masked(shape, q, k, v, None, threads, out_len)


def flash_forward_scalar(shape, q, k, v, mask=None):
    """cpu_forward.rs:594-686 (row-by-row statement of the same recurrence)."""
    return _forward(lib().ro_flash_forward_scalar, shape, q, k, v, mask, None, ())


def naive_forward_masked(shape, q, k, v, mask=None):
    """cpu_forward.rs:702-763."""
    return _forward(lib().ro_naive_forward_masked, shape, q, k, v, mask, None, ())


def naive_forward(shape, q, k, v):
    return naive_forward_masked(shape, q, k, v, None)


def flash_backward(shape, q, k, v, d_out, out_lens=None):
    """cpu_backward.rs:46-185.  Returns flat ``(dq, dk, dv)``; ``out_lens`` overrides the three output lengths
    (to exercise the length checks)."""
    ins = [_f32(np.ravel(a)) for a in (q, k, v, d_out)]
    lens = [shape.buffer_len()] * 3 if out_lens is None else list(out_lens)
    outs = [np.zeros(n, dtype=np.float32) for n in lens]
    err = _Err()
    s = shape._c()
    args = []
    for a, ptr in ins:
        args += [ptr, a.size]
    for o in outs:
        args += [o.ctypes.data_as(C.POINTER(C.c_float)), o.size]
    _raise(lib().ro_flash_backward(C.byref(s), *args, C.byref(err)), err)
    return tuple(outs)


def mask_is_masked(mask, qi, kj) -> bool:
    kind, keep_p, keep_n, _keep = _mask_args(mask)
    return bool(lib().ro_mask_is_masked(kind, keep_p, keep_n, qi, kj))


def gqa_forward_f32(q, k, v, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, threads=None, out_len=None):
    """gqa.rs:94-270.  Returns flat out [batch, n_heads, seq_q, head_dim]."""
    q, qp = _f32(np.ravel(q))
    k, kp = _f32(np.ravel(k))
    v, vp = _f32(np.ravel(v))
    n_out = batch * n_heads * seq_q * head_dim if out_len is None else out_len
    out = np.zeros(n_out, dtype=np.float32)
    err = _Err()
    t = lib().ro_max_threads() if threads is None else threads
    code = lib().ro_gqa_forward_f32(qp, q.size, kp, k.size, vp, v.size, out.ctypes.data_as(C.POINTER(C.c_float)),
                                    out.size, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, C.byref(err), t)
    _raise(code, err)
    return out


def kv_cache_append(k_cache, v_cache, batch, n_heads, max_seq, head_dim, current_len, seq_added, new_k, new_v):
    """kv_cache.rs:77-112, in place on the two float32 cache arrays."""
    assert k_cache.dtype == np.float32 and v_cache.dtype == np.float32
    nk, nkp = _f32(np.ravel(new_k))
    nv, nvp = _f32(np.ravel(new_v))
    err = _Err()
    code = lib().ro_kv_cache_append(k_cache.ctypes.data_as(C.POINTER(C.c_float)),
                                    v_cache.ctypes.data_as(C.POINTER(C.c_float)), batch, n_heads, max_seq,
                                    head_dim, current_len, seq_added, nkp, nk.size, nvp, nv.size, C.byref(err))
    _raise(code, err)


def kv_trim(cache, n_kv_heads, max_seq, kv_len, head_dim):
    """model.rs:638-650."""
    cache, cp = _f32(np.ravel(cache))
    out = np.zeros(n_kv_heads * kv_len * head_dim, dtype=np.float32)
    lib().ro_kv_trim(cp, out.ctypes.data_as(C.POINTER(C.c_float)), n_kv_heads, max_seq, kv_len, head_dim)
    return out


def f32_to_bf16(x):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    x, xp = _f32(np.ravel(x))
    y = np.empty(x.size, dtype=np.uint16)
    lib().ro_f32_to_bf16_array(xp, y.ctypes.data_as(C.POINTER(C.c_uint16)), x.size)
    return y


def bf16_to_f32(y):
    y = np.ascontiguousarray(np.ravel(y), dtype=np.uint16)
    x = np.empty(y.size, dtype=np.float32)
    lib().ro_bf16_to_f32_array(y.ctypes.data_as(C.POINTER(C.c_uint16)), x.ctypes.data_as(C.POINTER(C.c_float)),
                               y.size)
    return x


def _u16(a):
    a = np.ascontiguousarray(np.ravel(a), dtype=np.uint16)
    return a, a.ctypes.data_as(C.POINTER(C.c_uint16))


def kv_append_bf16(k_cache, v_cache, k_in, v_in, pos, n_kv, head_dim, max_seq):
    """llm_kernels.rs:353-372, in place on the uint16 cache arrays."""
    assert k_cache.dtype == np.uint16 and v_cache.dtype == np.uint16
    ki, kip = _u16(k_in)
    vi, vip = _u16(v_in)
    lib().ro_kv_append_bf16(k_cache.ctypes.data_as(C.POINTER(C.c_uint16)),
                            v_cache.ctypes.data_as(C.POINTER(C.c_uint16)), kip, vip, pos, n_kv, head_dim, max_seq)


def gqa_decode_online_bf16(q, k_cache, v_cache, n_heads, n_kv, kv_len, head_dim, max_seq):
    """llm_kernels.rs:396-457.  bf16 bit patterns in, bf16 bit patterns out [n_heads*head_dim]."""
    q, qp = _u16(q)
    kc, kp = _u16(k_cache)
    vc, vp = _u16(v_cache)
    out = np.zeros(n_heads * head_dim, dtype=np.uint16)
    lib().ro_gqa_decode_online_bf16(qp, kp, vp, out.ctypes.data_as(C.POINTER(C.c_uint16)), n_heads, n_kv, kv_len,
                                    head_dim, max_seq)
    return out


def gqa_decode_batched_bf16(q, k_cache, v_cache, kv_lens, batch, n_heads, n_kv, head_dim, max_seq, threads=None):
    """The CPU decode path (trim + decode_attn_row) per sequence with its own length, f32 on
    bf16-rounded inputs.  Returns float32 [batch*n_heads*head_dim]."""
    q, qp = _u16(q)
    kc, kp = _u16(k_cache)
    vc, vp = _u16(v_cache)
    lens = np.ascontiguousarray(kv_lens, dtype=np.int32)
    out = np.zeros(batch * n_heads * head_dim, dtype=np.float32)
    t = lib().ro_max_threads() if threads is None else threads
    lib().ro_gqa_decode_batched_bf16(qp, kp, vp, lens.ctypes.data_as(C.POINTER(C.c_int32)),
                                     out.ctypes.data_as(C.POINTER(C.c_float)), batch, n_heads, n_kv, head_dim,
                                     max_seq, t)
    return out


def gqa_decode_chunk_bf16(q, k_cache, v_cache, kv_lens, batch, seq_new, n_heads, n_kv, head_dim, max_seq, threads=None):
    """gqa_decode_batched_f32 (crates/rustorch-metal/src/kernels.rs:14432-14516) per sequence: `seq_new` consecutive
    query positions, position s of sequence b seeing keys [0, kv_lens[b] - seq_new + s].  q bf16 bits
    [B,seq_new,Hq,D], caches bf16 bits [B,Hkv,max_seq,D]; returns float32 [B*seq_new*Hq*D]."""
    q, qp = _u16(q)
    kc, kp = _u16(k_cache)
    vc, vp = _u16(v_cache)
    lens = np.ascontiguousarray(kv_lens, dtype=np.int32)
    out = np.zeros(batch * seq_new * n_heads * head_dim, dtype=np.float32)
    t = lib().ro_max_threads() if threads is None else threads
    lib().ro_gqa_decode_chunk_bf16(qp, kp, vp, lens.ctypes.data_as(C.POINTER(C.c_int32)),
                                   out.ctypes.data_as(C.POINTER(C.c_float)), batch, seq_new, n_heads, n_kv, head_dim,
                                   max_seq, t)
    return out


def varlen_causal_forward(q, k, v, seq_lens, batch, heads, max_seq, dim, zero_padded_rows=True, threads=None):
    """Padded-batch causal prefill: for sequence b the valid rows [0, len_b) equal the
    reference's ``flash_forward_masked(Mask::Causal)`` on the truncated (1,H,len_b,D)
    problem (causal already hides keys >= len_b from valid queries); rows >= len_b are
    0.0 (or NaN when ``zero_padded_rows`` is False, the reference's no-visible-key rule,
    cpu_forward.rs:411-420)."""
    q = np.asarray(q, dtype=np.float32).reshape(batch, heads, max_seq, dim)
    k = np.asarray(k, dtype=np.float32).reshape(batch, heads, max_seq, dim)
    v = np.asarray(v, dtype=np.float32).reshape(batch, heads, max_seq, dim)
    fill = 0.0 if zero_padded_rows else np.nan
    out = np.full((batch, heads, max_seq, dim), fill, dtype=np.float32)
    for b in range(batch):
        n = int(seq_lens[b])
        if n == 0:
            continue
        sh = AttentionShape(1, heads, n, dim)
        o = flash_forward_masked(sh, q[b, :, :n], k[b, :, :n], v[b, :, :n], "causal", threads)
        out[b, :, :n] = o.reshape(heads, n, dim)
    return out.ravel()


class OnlineSoftmaxState:
    """online_softmax.rs:44-151."""

    def __init__(self, m=-np.inf, l=0.0):
        self._s = _Osm(m, l)

    @property
    def m(self):
        return self._s.m

    @property
    def l(self):
        return self._s.l

    @classmethod
    def from_scalar(cls, x):
        st = cls()
        lib().ro_osm_from_scalar(C.byref(st._s), x)
        return st

    def absorb(self, x):
        lib().ro_osm_absorb(C.byref(self._s), x)

    def is_empty(self):
        return bool(lib().ro_osm_is_empty(C.byref(self._s)))


def combine_tiles(a: OnlineSoftmaxState, b: OnlineSoftmaxState) -> OnlineSoftmaxState:
    r = OnlineSoftmaxState()
    lib().ro_osm_combine(C.byref(a._s), C.byref(b._s), C.byref(r._s))
    return r


def online_softmax_full(xs) -> OnlineSoftmaxState:
    xs, xp = _f32(np.ravel(xs))
    r = OnlineSoftmaxState()
    lib().ro_osm_full(xp, xs.size, C.byref(r._s))
    return r


class RoPE:
    """RoPE::new and its two apply functions (crates/rustorch-nn/src/rope.rs:63-205) on float32 arrays."""

    def __init__(self, head_dim: int, max_seq: int, base: float = 10000.0):
        if head_dim % 2 != 0:
            raise ValueError(f"RoPE: head_dim must be even, got {head_dim}")  # rope.rs:64-68 panics
        self.head_dim, self.max_seq = head_dim, max_seq
        half = head_dim // 2
        self.cos = np.zeros(max_seq * half, dtype=np.float32)
        self.sin = np.zeros(max_seq * half, dtype=np.float32)
        lib().ro_rope_tables(head_dim, max_seq, base, self.cos.ctypes.data_as(C.POINTER(C.c_float)),
                             self.sin.ctypes.data_as(C.POINTER(C.c_float)))

    def _apply(self, fn, x, batch, n_heads, seq, position_offset):
        x = np.ascontiguousarray(np.ravel(x), dtype=np.float32).copy()
        err = _Err()
        fp = C.POINTER(C.c_float)
        rc = fn(x.ctypes.data_as(fp), x.size, batch, n_heads, seq, self.head_dim, position_offset,
                self.cos.ctypes.data_as(fp), self.sin.ctypes.data_as(fp), self.max_seq, C.byref(err))
        _raise(rc, err)
        return x

    def apply_half_split(self, x, batch, n_heads, seq, position_offset):
        return self._apply(lib().ro_rope_half_split, x, batch, n_heads, seq, position_offset)

    def apply_interleaved(self, x, batch, n_heads, seq, position_offset):
        return self._apply(lib().ro_rope_interleaved, x, batch, n_heads, seq, position_offset)


def rms_norm_per_head(x, gamma, n_heads, head_dim, eps):
    """model.rs:862-897; returns a new float32 array."""
    x, _ = _f32(x)
    x = x.copy()
    g, gp = _f32(gamma)
    assert x.size == n_heads * head_dim and g.size == head_dim
    lib().ro_rms_norm_per_head(x.ctypes.data_as(C.POINTER(C.c_float)), gp, n_heads, head_dim, eps)
    return x


def decode_prepare_bf16(q, k_in, v_in, k_cache, v_cache, positions, q_gamma, k_gamma, eps, rope, batch, n_heads, n_kv,
                        head_dim, max_seq, seq=1):
    """Steps 2a, 2b, 3 of decode_step (model.rs:575-636) on bf16 bit patterns, `seq` new tokens per sequence
    ([batch, heads, seq, head_dim] inputs): returns the new q; the caches (uint16 arrays) are updated in place."""
    assert k_cache.dtype == np.uint16 and v_cache.dtype == np.uint16
    q, qp = _u16(q)
    q = q.copy()
    qp = q.ctypes.data_as(C.POINTER(C.c_uint16))
    ki, kip = _u16(k_in)
    vi, vip = _u16(v_in)
    pos = np.ascontiguousarray(positions, dtype=np.int32)
    fp = C.POINTER(C.c_float)
    qg = gp_q = None
    if q_gamma is not None:
        qg, gp_q = _f32(q_gamma)
    kg = gp_k = None
    if k_gamma is not None:
        kg, gp_k = _f32(k_gamma)
    err = _Err()
    rc = lib().ro_decode_prepare_bf16(qp, kip, vip, k_cache.ctypes.data_as(C.POINTER(C.c_uint16)),
                                      v_cache.ctypes.data_as(C.POINTER(C.c_uint16)),
                                      pos.ctypes.data_as(C.POINTER(C.c_int32)), gp_q, gp_k, eps,
                                      rope.cos.ctypes.data_as(fp), rope.sin.ctypes.data_as(fp), batch, seq, n_heads,
                                      n_kv, head_dim, max_seq, rope.max_seq, C.byref(err))
    _raise(rc, err)
    return q


MASK_NEG = np.float32(-1.0e4)


def causal_mask(seq_len):
    """masks.rs:30-40."""
    out = np.zeros(seq_len * seq_len, dtype=np.float32)
    lib().ro_causal_mask(seq_len, out.ctypes.data_as(C.POINTER(C.c_float)))
    return out.reshape(seq_len, seq_len)


def sliding_window_mask(seq_len, window):
    """masks.rs:52-65."""
    assert window >= 1
    out = np.zeros(seq_len * seq_len, dtype=np.float32)
    lib().ro_sliding_window_mask(seq_len, window, out.ctypes.data_as(C.POINTER(C.c_float)))
    return out.reshape(seq_len, seq_len)


def bool_to_additive(mask):
    """masks.rs:73-82."""
    m, mp = _f32(np.asarray(mask, dtype=np.float32))
    out = np.zeros(m.size, dtype=np.float32)
    lib().ro_bool_to_additive(mp, out.ctypes.data_as(C.POINTER(C.c_float)), m.size)
    return out.reshape(m.shape)


def softmax_row(x):
    """softmax_row_online_f32 (crates/rustorch-cpu/src/kernels/softmax.rs:146-180)."""
    x, xp = _f32(np.ravel(x))
    out = np.zeros(x.size, dtype=np.float32)
    lib().ro_softmax_row(xp, out.ctypes.data_as(C.POINTER(C.c_float)), x.size)
    return out


def mha_forward_masked(q, k, v, batch, t_q, t_kv, heads, head_dim, attn_mask=None):
    """Steps 2-8 of the composed MultiHeadAttention path (attention.rs:371-399); q [B,t_q,H*hd], k, v [B,t_kv,H*hd];
    attn_mask None, t_q*t_kv elements, or B*H*t_q*t_kv elements.  Returns flat float32 [B,t_q,H*hd]."""
    q, qp = _f32(np.ravel(q))
    k, kp = _f32(np.ravel(k))
    v, vp = _f32(np.ravel(v))
    assert q.size == batch * t_q * heads * head_dim and k.size == v.size == batch * t_kv * heads * head_dim
    mp, stride = None, 0
    if attn_mask is not None:
        m, mp = _f32(np.ravel(attn_mask))
        assert m.size in (t_q * t_kv, batch * heads * t_q * t_kv)
        stride = t_q * t_kv if (m.size == batch * heads * t_q * t_kv and batch * heads > 1) else 0
    out = np.zeros(q.size, dtype=np.float32)
    lib().ro_mha_forward_masked(qp, kp, vp, mp, stride, out.ctypes.data_as(C.POINTER(C.c_float)), batch, t_q, t_kv,
                                heads, head_dim)
    return out


def max_threads() -> int:
    return lib().ro_max_threads()


# ---------------------------------------------------------------------------------------------------------------
# Comparison rule of the bf16 parity checks (no reference arithmetic here: a rule about two result arrays)
BF16_MAX_ABS = 2e-2    # the absolute bar
BF16_REL_FRO = 1e-2    # the scale-aware bar beside it, per block of rows


def rel_fro_blocks(got, want, dim, slab_rows=None, block_rows=256, min_elems=512):
    """Largest relative Frobenius error ``||got - want||_F / ||want||_F`` over blocks of ``block_rows`` consecutive
    rows of ``dim`` elements, blocks never crossing a slab of ``slab_rows`` rows (one (batch, head) pair; default:
    the whole array is one slab).  The reference's own equivalence test carries a Frobenius criterion beside the
    max-abs one (crates/rustorch-attention/tests/equivalence.rs:79-112: ``frob < tol * sqrt(n)``); this is its
    scale-aware form, local in the rows: late rows of a long causal prefill average thousands of V rows and are
    small (std 1/sqrt(N)), so an absolute bar alone cannot see a dropped key tile there, the relative one does.
    Elements that are NaN in ``want`` are left out (NaN patterns are compared exactly elsewhere); a block whose
    ``want`` is all zero must be reproduced exactly (the result is inf otherwise).  Blocks of fewer than
    ``min_elems`` elements are too small for a norm ratio to mean anything: the array is then taken as one block.
    Decode outputs are compared per (sequence, head) row: ``block_rows=1, min_elems=64``."""
    got = np.asarray(got, dtype=np.float64).reshape(-1, dim)
    want = np.asarray(want, dtype=np.float64).reshape(-1, dim)
    assert got.shape == want.shape
    rows = want.shape[0]
    if rows == 0:
        return 0.0
    slab_rows = slab_rows or rows
    assert rows % slab_rows == 0
    nan = np.isnan(want)
    with np.errstate(invalid="ignore"):
        diff = np.where(nan | (got == want), 0.0, got - want)  # equal infinities agree
    diff2 = (np.nan_to_num(diff, nan=np.inf, posinf=np.inf, neginf=np.inf) ** 2).sum(axis=1)
    ref2 = np.where(nan | np.isinf(want), 0.0, want ** 2).sum(axis=1)
    blk = min(block_rows, slab_rows)
    if blk * dim < min_elems:
        num, den = np.array([diff2.sum()]), np.array([ref2.sum()])
    else:
        n_blk = -(-slab_rows // blk)
        pad = n_blk * blk - slab_rows
        d2 = np.pad(diff2.reshape(-1, slab_rows), ((0, 0), (0, pad))).reshape(-1, n_blk, blk)
        r2 = np.pad(ref2.reshape(-1, slab_rows), ((0, 0), (0, pad))).reshape(-1, n_blk, blk)
        num, den = d2.sum(axis=2).ravel(), r2.sum(axis=2).ravel()
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(den > 0, np.sqrt(num / den), np.where(num > 0, np.inf, 0.0))
    return float(rel.max())
