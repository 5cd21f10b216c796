"""Pins the oracle's additive masks, row softmax and the masked MultiHeadAttention core, and checks the host mask
builders of rustorch_amd against them.  Reference tests restated: crates/rustorch-nn/src/masks.rs:88-208.
Independent anchors: float64 brute force, torch's softmax and scaled_dot_product_attention with an additive mask,
closed forms (zero scores + causal mask => prefix means; a row masked everywhere with -1e4 => uniform weights)."""
import numpy as np
import pytest
import torch

import rustorch_amd as ra


# ---- reference tests (masks.rs:88-208) ----------------------------------------------------------------------


@pytest.mark.parametrize("mod", ["oracle", "host"])
def test_mask_builders(oracle, mod):
    m = oracle if mod == "oracle" else ra
    neg = np.float32(-1.0e4)
    c = m.causal_mask(4)
    for i in range(4):
        for j in range(4):
            assert c[i, j] == (0.0 if j <= i else neg)
    s = m.sliding_window_mask(8, 3)  # truth table: columns max(0, i-2) .. i are kept
    for i in range(8):
        for j in range(8):
            assert s[i, j] == (0.0 if max(0, i - 2) <= j <= i else neg)
    assert np.array_equal(m.sliding_window_mask(5, 100), m.causal_mask(5))
    d = m.sliding_window_mask(4, 1)
    assert np.array_equal(d == 0.0, np.eye(4, dtype=bool))
    add = m.bool_to_additive(np.array([[1.0, 0.0], [1.0, 1.0]], dtype=np.float32))
    assert add.shape == (2, 2) and add.tolist() == [[0.0, float(neg)], [0.0, 0.0]]
    assert c.dtype == np.float32 and s.dtype == np.float32


def test_host_window_must_be_positive():
    with pytest.raises(ValueError):
        ra.sliding_window_mask(4, 0)


def test_causal_mask_zeroes_softmax_above_diagonal(oracle):
    n = 3
    masked = np.zeros((n, n), dtype=np.float32) + oracle.causal_mask(n)
    p = np.stack([oracle.softmax_row(masked[i]) for i in range(n)])
    assert abs(p[0, 0] - 1.0) < 1e-3 and abs(p[0, 1]) < 1e-3 and abs(p[0, 2]) < 1e-3
    assert np.abs(p[2] - 1.0 / n).max() < 1e-3


# ---- independent anchors ------------------------------------------------------------------------------------


def test_softmax_row_against_torch_and_edge_rows(oracle):
    rng = np.random.default_rng(0)
    for n in (1, 2, 7, 64, 1000):
        x = (rng.standard_normal(n) * 5).astype(np.float32)
        want = torch.softmax(torch.from_numpy(x).double(), 0).numpy()
        assert np.abs(oracle.softmax_row(x) - want).max() < 1e-6
    assert oracle.softmax_row(np.array([], dtype=np.float32)).size == 0
    # every entry masked with -1e4: finite, uniform (the reason masks.rs uses -1e4)
    u = oracle.softmax_row(np.full(4, -1.0e4, dtype=np.float32))
    assert np.array_equal(u, np.full(4, 0.25, dtype=np.float32))
    # every entry -inf: NaN, as exp(-inf - -inf) makes it (softmax.rs:158-165)
    assert np.isnan(oracle.softmax_row(np.full(3, -np.inf, dtype=np.float32))).all()
    # one huge entry: one-hot without overflow
    h = oracle.softmax_row(np.array([0.0, 1.0e6, -1.0e6], dtype=np.float32))
    assert h.tolist() == [0.0, 1.0, 0.0]


def _f64_reference(q, k, v, b, tq, tkv, h, d, mask):
    q4 = q.astype(np.float64).reshape(b, tq, h, d).transpose(0, 2, 1, 3)
    k4 = k.astype(np.float64).reshape(b, tkv, h, d).transpose(0, 2, 1, 3)
    v4 = v.astype(np.float64).reshape(b, tkv, h, d).transpose(0, 2, 1, 3)
    s = q4 @ k4.transpose(0, 1, 3, 2) / np.sqrt(d)
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64).reshape(-1, tq, tkv).reshape((1, 1, tq, tkv) if np.size(mask) == tq * tkv
                                                                               else (b, h, tq, tkv))
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(-1, keepdims=True)
    return (p @ v4).transpose(0, 2, 1, 3).reshape(-1)


@pytest.mark.parametrize("b,tq,tkv,h,d,mask_kind", [
    (1, 1, 1, 1, 4, None), (2, 5, 5, 3, 8, "causal"), (1, 7, 7, 2, 16, "window"), (2, 4, 9, 2, 8, None),
    (2, 6, 3, 2, 4, "rand_shared"), (2, 5, 5, 2, 8, "rand_per_head"), (1, 33, 70, 1, 32, "rand_shared")])
def test_mha_core_against_float64_and_torch(oracle, b, tq, tkv, h, d, mask_kind):
    rng = np.random.default_rng(3)
    q = rng.standard_normal(b * tq * h * d).astype(np.float32)
    k = rng.standard_normal(b * tkv * h * d).astype(np.float32)
    v = rng.standard_normal(b * tkv * h * d).astype(np.float32)
    mask = {None: None, "causal": lambda: oracle.causal_mask(tq), "window": lambda: oracle.sliding_window_mask(tq, 3),
            "rand_shared": lambda: np.where(rng.random((tq, tkv)) > 0.3, 0.0, -1.0e4).astype(np.float32),
            "rand_per_head": lambda: (rng.standard_normal((b * h, tq, tkv)) * 2).astype(np.float32)}[mask_kind]
    mask = mask() if mask is not None else None
    got = oracle.mha_forward_masked(q, k, v, b, tq, tkv, h, d, mask)
    assert np.abs(got - _f64_reference(q, k, v, b, tq, tkv, h, d, mask)).max() < 5e-6
    # torch's library routine with an additive float mask, on [B,H,T,D] views
    tq4 = torch.from_numpy(q).double().reshape(b, tq, h, d).transpose(1, 2)
    tk4 = torch.from_numpy(k).double().reshape(b, tkv, h, d).transpose(1, 2)
    tv4 = torch.from_numpy(v).double().reshape(b, tkv, h, d).transpose(1, 2)
    tm = None
    if mask is not None:
        tm = torch.from_numpy(np.asarray(mask)).double()
        tm = tm.reshape(1, 1, tq, tkv) if tm.numel() == tq * tkv else tm.reshape(b, h, tq, tkv)
    want = torch.nn.functional.scaled_dot_product_attention(tq4, tk4, tv4, attn_mask=tm).transpose(1, 2).reshape(-1).numpy()
    assert np.abs(got - want).max() < 5e-6


def test_mha_core_closed_forms(oracle):
    # zero queries and keys + causal mask: row i is the mean of V[0..i] (the -1e4 entries weigh exp(-1e4) = 0)
    b, t, h, d = 1, 6, 2, 4
    rng = np.random.default_rng(5)
    v = rng.standard_normal(b * t * h * d).astype(np.float32)
    z = np.zeros_like(v)
    got = oracle.mha_forward_masked(z, z, v, b, t, t, h, d, oracle.causal_mask(t)).reshape(t, h, d)
    v4 = v.reshape(t, h, d).astype(np.float64)
    for i in range(t):
        assert np.abs(got[i] - v4[: i + 1].mean(0)).max() < 1e-6
    # a row masked everywhere attends uniformly instead of turning into NaN (masks.rs:9-15)
    m = np.zeros((t, t), dtype=np.float32)
    m[2, :] = -1.0e4
    got = oracle.mha_forward_masked(z, z, v, b, t, t, h, d, m).reshape(t, h, d)
    assert np.abs(got[2] - v4.mean(0)).max() < 1e-6 and np.isfinite(got).all()
    # without a mask and with t_q == t_kv the core is the unmasked flash forward on transposed tensors
    q = rng.standard_normal(b * t * h * d).astype(np.float32)
    k = rng.standard_normal(b * t * h * d).astype(np.float32)
    tr = lambda x: np.ascontiguousarray(x.reshape(b, t, h, d).transpose(0, 2, 1, 3)).ravel()
    flash = oracle.flash_forward(oracle.AttentionShape(b, h, t, d), tr(q), tr(k), tr(v)).reshape(b, h, t, d)
    core = oracle.mha_forward_masked(q, k, v, b, t, t, h, d).reshape(b, t, h, d).transpose(0, 2, 1, 3)
    assert np.abs(flash - core).max() < 1e-6
    # no keys at all: rows of zeros (an empty softmax times an empty V)
    out = oracle.mha_forward_masked(q, np.zeros(0, np.float32), np.zeros(0, np.float32), b, t, 0, h, d)
    assert not out.any()
