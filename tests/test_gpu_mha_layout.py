"""GPU parity of the [batch, seq, heads, dim] entry points (rt_mha_flash_forward_f32,
rt_flash_forward_bnhd_f32_dev, rt_flash_forward_bnhd_bf16_dev): the MultiHeadAttention call surface of
crates/rustorch-nn/src/attention.rs:452-495 without its four transposes.  The expected value is the oracle's
flash forward on explicitly transposed copies, transposed back, which is what the reference computes."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_bf16_parity, assert_close_nan, bf16_round, dev
from _util import seeded_normal

pytestmark = pytest.mark.gpu


def to_bhnd(x, b, n, h, d):
    return np.ascontiguousarray(x.reshape(b, n, h, d).transpose(0, 2, 1, 3)).ravel()


def to_bnhd(x, b, h, n, d):
    return np.ascontiguousarray(x.reshape(b, h, n, d).transpose(0, 2, 1, 3)).ravel()


@pytest.mark.parametrize("b,n,h,d", [(1, 1, 1, 4), (2, 5, 3, 8), (1, 64, 4, 32), (2, 130, 2, 64), (1, 300, 3, 128),
                                     (3, 33, 5, 20)])
def test_mha_flash_forward_f32_matches_reference_path(oracle, b, n, h, d):
    q, k, v = (seeded_normal((b, n, h, d), s).ravel() for s in (11, 12, 13))
    got = ra.mha_flash_forward_f32(q, k, v, b, n, h, d)
    want_bhnd = oracle.flash_forward(oracle.AttentionShape(b, h, n, d), to_bhnd(q, b, n, h, d), to_bhnd(k, b, n, h, d),
                                     to_bhnd(v, b, n, h, d))
    assert_close_nan(got, to_bnhd(want_bhnd, b, h, n, d), 1e-5, f"mha f32 {b},{n},{h},{d}")


def test_mha_flash_forward_f32_errors_follow_flash_forward():
    z = np.zeros(24, dtype=np.float32)
    with pytest.raises(ra.ZeroDim):
        ra.mha_flash_forward_f32(z, z, z, 1, 2, 3, 0)
    with pytest.raises(ra.BufferShapeMismatch) as e:
        ra.mha_flash_forward_f32(z[:23], z, z, 1, 2, 3, 4)
    assert (e.value.which, e.value.expected, e.value.got) == ("q", 24, 23)
    with pytest.raises(ra.BufferShapeMismatch) as e:
        ra.mha_flash_forward_f32(z, z, z[:5], 1, 2, 3, 4)
    assert e.value.which == "v"
    with pytest.raises(ra.OutputShapeMismatch):
        ra.mha_flash_forward_f32(z, z, z, 1, 2, 3, 4, out=np.zeros(25, dtype=np.float32))
    # seq == 0: Ok, nothing touched
    out = np.full(0, 7.0, dtype=np.float32)
    ra.mha_flash_forward_f32(z[:0], z[:0], z[:0], 2, 0, 3, 4, out=out)


@pytest.mark.parametrize("kernel", ["auto", "wide"])
@pytest.mark.parametrize("mask_name", ["none", "causal", "padding"])
@pytest.mark.parametrize("b,n,h,hkv,d", [(2, 200, 4, 4, 64), (1, 513, 6, 2, 128), (2, 64, 8, 1, 128), (1, 700, 8, 2, 64)])
def test_flash_bnhd_bf16_matches_oracle(oracle, b, n, h, hkv, d, mask_name, kernel):
    """(kernel "wide": the 64-rows-per-wave kernel where it applies, head dim 64 without a padding mask; else as "auto")"""
    ra.debug_force_bf16_prefill_kernel(kernel)
    try:
        _bnhd_bf16_case(oracle, b, n, h, hkv, d, mask_name)
    finally:
        ra.debug_force_bf16_prefill_kernel("auto")


def _bnhd_bf16_case(oracle, b, n, h, hkv, d, mask_name):
    (qb, qf) = bf16_round(seeded_normal((b, n, h, d), 21).ravel())
    (kb, kf) = bf16_round(seeded_normal((b, n, hkv, d), 22).ravel())
    (vb, vf) = bf16_round(seeded_normal((b, n, hkv, d), 23).ravel())
    keep = np.random.default_rng(n).random(n) < 0.7
    keep[0] = True
    mask, om, keep_dev = {"none": (ra.Mask.none(), None, None), "causal": (ra.Mask.causal(), "causal", None),
                          "padding": (ra.Mask.padding(keep), ("padding", keep), dev(keep.astype(np.uint8)))}[mask_name]
    out = ra.HipStorage(b * n * h * d * 2)
    ra.flash_forward_bnhd_bf16_dev(ra.AttentionShape.new(b, h, n, d), dev(qb), dev(kb), dev(vb), out, mask,
                                   keep_dev=keep_dev, n_kv_heads=hkv)
    ra.synchronize()
    got = oracle.bf16_to_f32(out.download(np.uint16))
    # oracle on [B,H,N,D] copies, k/v heads replicated per group as gqa.rs does
    g = h // hkv
    k_rep = np.repeat(kf.reshape(b, n, hkv, d), g, axis=2).ravel()
    v_rep = np.repeat(vf.reshape(b, n, hkv, d), g, axis=2).ravel()
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), to_bhnd(qf, b, n, h, d),
                                       to_bhnd(k_rep, b, n, h, d), to_bhnd(v_rep, b, n, h, d), om)
    assert_bf16_parity(got, to_bnhd(want, b, h, n, d), d, None, f"bnhd bf16 {b},{n},{h},{hkv},{d} {mask_name}")


@pytest.mark.parametrize("b,n,h,d", [(2, 100, 3, 48), (1, 257, 2, 128)])
def test_flash_bnhd_f32_dev_matches_oracle(oracle, b, n, h, d):
    q, k, v = (seeded_normal((b, n, h, d), s).ravel() for s in (31, 32, 33))
    out = ra.HipStorage(b * n * h * d * 4)
    ra.flash_forward_bnhd_f32_dev(ra.AttentionShape.new(b, h, n, d), dev(q), dev(k), dev(v), out, ra.Mask.causal())
    ra.synchronize()
    got = out.download(np.float32)
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), to_bhnd(q, b, n, h, d),
                                       to_bhnd(k, b, n, h, d), to_bhnd(v, b, n, h, d), "causal")
    assert_close_nan(got, to_bnhd(want, b, h, n, d), 1e-5, f"bnhd f32 {b},{n},{h},{d}")
