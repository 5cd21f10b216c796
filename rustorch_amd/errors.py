"""The reference's error enums for the attention path, as Python exceptions.

AttentionError / MaskError: crates/rustorch-attention/src/cpu_forward.rs:93-114, mask.rs:70-78.
GQAError: crates/rustorch-nn/src/gqa.rs:37-55.  KVCacheError: crates/rustorch-nn/src/kv_cache.rs:229-256.
RoPEError: crates/rustorch-nn/src/rope.rs:208-241.
DeviceError stands where the reference has CudaError (NoDeviceFound / Driver / Unsupported).
"""
from __future__ import annotations

from . import _lib as L


class AttentionError(Exception):
    pass


class ZeroDim(AttentionError):
    def __str__(self):
        return "dim must be > 0"


class BufferShapeMismatch(AttentionError):
    def __init__(self, which, expected, got):
        self.which, self.expected, self.got = which, expected, got

    def __str__(self):
        return f"{self.which} buffer has {self.got} elements, expected {self.expected}"


class OutputShapeMismatch(AttentionError):
    def __init__(self, expected, got):
        self.expected, self.got = expected, got

    def __str__(self):
        return f"output buffer has {self.got} elements, expected {self.expected}"


class MaskError(AttentionError):
    pass


class PaddingLengthMismatch(MaskError):
    def __init__(self, expected, got):
        self.expected, self.got = expected, got

    def __str__(self):
        return f"mask error: padding mask len {self.got}, expected {self.expected}"


class GQAError(Exception):
    pass


class HeadCountMismatch(GQAError):
    def __init__(self, n_heads, n_kv_heads):
        self.n_heads, self.n_kv_heads = n_heads, n_kv_heads

    def __str__(self):
        return f"gqa: n_heads {self.n_heads} not divisible by n_kv_heads {self.n_kv_heads}"


class WrongInputLen(GQAError):
    def __init__(self, which, expected, got):
        self.which, self.expected, self.got = which, expected, got

    def __str__(self):
        return f"gqa: {self.which} expected {self.expected} f32, got {self.got}"


class KVCacheError(Exception):
    pass


class Overflow(KVCacheError):
    def __init__(self, requested, max):
        self.requested, self.max = requested, max

    def __str__(self):
        return f"kv_cache overflow: requested {self.requested} positions, max {self.max}"


class KVWrongInputLen(KVCacheError):
    def __init__(self, expected, got_k, got_v):
        self.expected, self.got_k, self.got_v = expected, got_k, got_v

    def __str__(self):
        return f"kv_cache append: expected {self.expected}, got K={self.got_k} V={self.got_v}"


class LayerOutOfRange(KVCacheError):
    def __init__(self, layer, num_layers):
        self.layer, self.num_layers = layer, num_layers

    def __str__(self):
        return f"kv_cache layer {self.layer} out of range (have {self.num_layers})"


class RoPEError(Exception):
    pass


class RopeWrongInputLen(RoPEError):
    def __init__(self, expected, got):
        self.expected, self.got = expected, got

    def __str__(self):
        return f"rope: expected buffer of {self.expected} f32, got {self.got}"


class PositionOverflow(RoPEError):
    def __init__(self, max_seq, requested):
        self.max_seq, self.requested = max_seq, requested

    def __str__(self):
        return f"rope: position {self.requested} exceeds max_seq {self.max_seq}"


class DeviceError(Exception):
    """NoDeviceFound / Driver / Unsupported / workspace and pointer errors of the HIP library."""

    def __init__(self, status, message, hip_error=0, expected=0, got=0):
        self.status, self.message, self.hip_error, self.expected, self.got = status, message, hip_error, expected, got

    def __str__(self):
        return f"{L.status_name(self.status)}: {self.message}"


def raise_for(status: int, err: "L.RtErr"):
    """Turn a C-ABI status + detail into the matching exception."""
    if status == L.RT_OK:
        return
    which = L.WHICH.get(err.which, "")
    if status == L.RT_ERR_ZERO_DIM:
        raise ZeroDim()
    if status == L.RT_ERR_BUFFER_SHAPE_MISMATCH:
        raise BufferShapeMismatch(which, err.expected, err.got)
    if status == L.RT_ERR_OUTPUT_SHAPE_MISMATCH:
        raise OutputShapeMismatch(err.expected, err.got)
    if status == L.RT_ERR_PADDING_LENGTH_MISMATCH:
        raise PaddingLengthMismatch(err.expected, err.got)
    if status == L.RT_ERR_HEAD_COUNT_MISMATCH:
        raise HeadCountMismatch(err.expected, err.got)
    if status == L.RT_ERR_WRONG_INPUT_LEN:
        raise WrongInputLen(which, err.expected, err.got)
    if status == L.RT_ERR_KV_OVERFLOW:
        raise Overflow(err.got, err.expected)
    if status == L.RT_ERR_KV_WRONG_INPUT_LEN:
        raise KVWrongInputLen(err.expected, err.got, err.got2)
    if status == L.RT_ERR_ROPE_WRONG_INPUT_LEN:
        raise RopeWrongInputLen(err.expected, err.got)
    if status == L.RT_ERR_ROPE_POSITION_OVERFLOW:
        raise PositionOverflow(err.expected, err.got)
    raise DeviceError(status, err.message.decode(errors="replace"), err.hip_error, err.expected, err.got)
