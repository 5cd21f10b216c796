"""Shared test helpers: the reference's deterministic input generators and comparison rules."""
import numpy as np


def lcg_buffer(n, seed, span=2.0):
    """The reference tests' LCG fixture (crates/rustorch-attention/tests/equivalence.rs:23-31 with
    span 2.0; cpu_forward.rs:769-779 with span 3.0):
    s0 = seed * 2654435761; s_{i+1} = s_i * 1664525 + 1013904223 (mod 2^32);
    x_i = (s_i as f32 / u32::MAX as f32 - 0.5) * span."""
    if n == 0:
        return np.zeros(0, dtype=np.float32)
    a = np.uint32(1664525)
    c = np.uint32(1013904223)
    s0 = np.uint32((seed * 2654435761) & 0xFFFFFFFF)
    with np.errstate(over="ignore"):
        pw = np.cumprod(np.full(n, a, dtype=np.uint32), dtype=np.uint32)  # a^1 .. a^n
        geo = np.cumsum(np.concatenate([[np.uint32(1)], pw[:-1]]).astype(np.uint32), dtype=np.uint32)  # sum a^0..a^(i-1)
        s = pw * s0 + c * geo
    sf = s.astype(np.float32)  # `as f32`: round to nearest
    x = (sf / np.float32(4294967296.0) - np.float32(0.5)) * np.float32(span)
    return x.astype(np.float32)


def hash_buffer(n, mult):
    """Inputs of the reference's proptest (cpu_forward.rs:1076-1078):
    ((i as u32) * mult * 2654435761) as f32 / u32::MAX as f32 - 0.5) * 2."""
    i = np.arange(n, dtype=np.uint64)
    s = ((i * np.uint64(mult)) & np.uint64(0xFFFFFFFF)) * np.uint64(2654435761) & np.uint64(0xFFFFFFFF)
    sf = s.astype(np.uint32).astype(np.float32)
    return ((sf / np.float32(4294967296.0) - np.float32(0.5)) * np.float32(2.0)).astype(np.float32)


def close_ref(a, b, atol, rtol=1e-4):
    """The reference's `close` (cpu_forward.rs:790-795): NaN==NaN, else |a-b| <= atol + rtol*max(|a|,|b|)."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    both_nan = np.isnan(a) & np.isnan(b)
    with np.errstate(invalid="ignore"):
        ok = np.abs(a - b) <= atol + rtol * np.maximum(np.abs(a), np.abs(b))
    return bool(np.all(ok | both_nan))


def attention_f64(q, k, v, mask=None):
    """Brute-force float64 attention on [B,H,N,D] arrays; mask None | "causal" | ("padding", keep)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, H, N, D = q.shape
    s = np.einsum("bhid,bhjd->bhij", q, k) / np.sqrt(np.float64(np.float32(D)))
    if mask == "causal":
        s = np.where(np.triu(np.ones((N, N), dtype=bool), 1)[None, None], -np.inf, s)
    elif mask is not None:
        keep = np.asarray(mask[1], dtype=bool)
        s = np.where(~keep[None, None, None, :], -np.inf, s)
    with np.errstate(invalid="ignore"):
        m = s.max(axis=-1, keepdims=True)
        p = np.exp(s - m)
        out = np.einsum("bhij,bhjd->bhid", p / p.sum(axis=-1, keepdims=True), v)
    return out


def seeded_normal(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
