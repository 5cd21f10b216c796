"""rt_mha_forward_masked_f32 (the masked / cross-attention core of MultiHeadAttention::forward,
crates/rustorch-nn/src/attention.rs:371-399) against the oracle: max-abs <= 1e-5, NaN patterns exact."""
import numpy as np
import pytest

import rustorch_amd as ra

pytestmark = pytest.mark.gpu


def _run(oracle, b, tq, tkv, h, d, mask, seed=0):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal(b * tq * h * d).astype(np.float32)
    k = rng.standard_normal(b * tkv * h * d).astype(np.float32)
    v = rng.standard_normal(b * tkv * h * d).astype(np.float32)
    got = ra.mha_forward_masked_f32(q, k, v, b, tq, tkv, h, d, attn_mask=mask)
    want = oracle.mha_forward_masked(q, k, v, b, tq, tkv, h, d, mask)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.nanmax(np.abs(got - want)) <= 1e-5 if got.size else True
    return got


@pytest.mark.parametrize("b,t,h,d", [(1, 1, 1, 4), (2, 5, 3, 8), (2, 128, 4, 64), (1, 70, 2, 96), (1, 33, 1, 130), (2, 257, 2, 32)])
@pytest.mark.parametrize("kind", ["none", "causal", "window", "bool", "per_head"])
def test_self_attention_with_masks(oracle, b, t, h, d, kind):
    rng = np.random.default_rng(7)
    mask = {"none": None, "causal": ra.causal_mask(t), "window": ra.sliding_window_mask(t, 3),
            "bool": ra.bool_to_additive((rng.random((t, t)) > 0.4).astype(np.float32)),
            "per_head": (rng.standard_normal((b * h, t, t)) * 2).astype(np.float32)}[kind]
    _run(oracle, b, t, t, h, d, mask)


@pytest.mark.parametrize("b,tq,tkv,h,d", [(2, 4, 9, 2, 8), (1, 100, 7, 3, 64), (2, 1, 300, 2, 128), (1, 6, 1, 1, 16),
                                          (2, 70, 333, 3, 80), (1, 257, 64, 2, 20), (1, 33, 1000, 1, 128), (2, 40, 65, 2, 6),
                                          (1, 31, 97, 2, 132), (8, 16, 512, 8, 64)])
def test_cross_attention(oracle, b, tq, tkv, h, d):
    rng = np.random.default_rng(9)
    _run(oracle, b, tq, tkv, h, d, None)
    _run(oracle, b, tq, tkv, h, d, np.where(rng.random((tq, tkv)) > 0.3, 0.0, -1.0e4).astype(np.float32))
    _run(oracle, b, tq, tkv, h, d, (rng.standard_normal((b * h, tq, tkv))).astype(np.float32))


def test_masked_rows_and_edge_cases(oracle):
    b, t, h, d = 1, 6, 2, 4
    m = np.zeros((t, t), dtype=np.float32)
    m[2, :] = -1.0e4  # masked everywhere with the reference's value: uniform weights, finite
    got = _run(oracle, b, t, t, h, d, m)
    assert np.isfinite(got).all()
    m[3, :] = -np.inf  # masked everywhere with -inf: that row is NaN, as in the reference's softmax
    got = _run(oracle, b, t, t, h, d, m).reshape(b, t, h * d)
    assert np.isnan(got[0, 3]).all() and np.isfinite(np.delete(got[0], 3, axis=0)).all()
    # no keys: rows of zeros; no queries: nothing
    z = np.zeros(0, np.float32)
    q = np.ones(b * t * h * d, np.float32)
    assert not ra.mha_forward_masked_f32(q, z, z, b, t, 0, h, d).any()
    assert ra.mha_forward_masked_f32(z, q, q, b, 0, t, h, d).size == 0
    # [1,T,T] and [T,T] are the same bytes
    c = ra.causal_mask(t)
    assert np.array_equal(_run(oracle, b, t, t, h, d, c), _run(oracle, b, t, t, h, d, c.reshape(1, t, t)))


def test_without_mask_equals_the_flash_path():
    rng = np.random.default_rng(11)
    b, t, h, d = 2, 64, 4, 32
    q, k, v = (rng.standard_normal(b * t * h * d).astype(np.float32) for _ in range(3))
    a = ra.mha_forward_masked_f32(q, k, v, b, t, t, h, d)
    f = ra.mha_flash_forward_f32(q, k, v, b, t, h, d)
    assert np.abs(a - f).max() <= 2e-6


def test_error_order():
    z = lambda n: np.zeros(n, np.float32)
    b, tq, tkv, h, d = 1, 2, 3, 2, 4
    nq, nk = b * tq * h * d, b * tkv * h * d
    with pytest.raises(ra.ZeroDim):
        ra.mha_forward_masked_f32(z(0), z(0), z(0), b, tq, tkv, h, 0)
    for args, which, exp, got in (((z(nq - 1), z(nk), z(nk)), "q", nq, nq - 1), ((z(nq), z(nk + 1), z(nk)), "k", nk, nk + 1),
                                  ((z(nq), z(nk), z(nk - 2)), "v", nk, nk - 2)):
        with pytest.raises(ra.BufferShapeMismatch) as e:
            ra.mha_forward_masked_f32(*args, b, tq, tkv, h, d)
        assert (e.value.which, e.value.expected, e.value.got) == (which, exp, got)
    with pytest.raises(ra.OutputShapeMismatch):
        ra.mha_forward_masked_f32(z(nq), z(nk), z(nk), b, tq, tkv, h, d, out=z(nq + 1))
    with pytest.raises(ra.WrongInputLen) as e:
        ra.mha_forward_masked_f32(z(nq), z(nk), z(nk), b, tq, tkv, h, d, attn_mask=z(5))
    assert (e.value.which, e.value.expected, e.value.got) == ("mask", tq * tkv, 5)


def test_routing_of_multi_head_attention(oracle):
    """attention.rs:325-399: single token without mask -> the context is V; unmasked equal lengths -> the flash path;
    a mask or unequal lengths -> the composed path.  All three agree with the oracle's composed core."""
    rng = np.random.default_rng(11)
    for b, tq, tkv, h, d, masked in [(3, 1, 1, 2, 8, False), (2, 40, 40, 2, 32, False), (2, 40, 40, 2, 32, True),
                                     (1, 5, 9, 2, 16, False), (2, 1, 1, 2, 8, True)]:
        q = rng.standard_normal(b * tq * h * d).astype(np.float32)
        k = rng.standard_normal(b * tkv * h * d).astype(np.float32)
        v = rng.standard_normal(b * tkv * h * d).astype(np.float32)
        mask = ra.causal_mask(tq) if masked and tq == tkv else None
        route = ra.mha_attention_route(tq, tkv, mask is not None)
        got = ra.mha_attention_f32(q, k, v, b, tq, tkv, h, d, mask)
        want = oracle.mha_forward_masked(q, k, v, b, tq, tkv, h, d, mask)
        assert np.abs(got - want).max() <= 1e-5, route
        if route == "identity":
            assert np.array_equal(got, v)


@pytest.mark.parametrize("b,tq,tkv,h,d,kind", [(2, 40, 40, 2, 32, "causal"), (1, 70, 333, 3, 80, "per_head"),
                                                (2, 33, 9, 2, 6, "none"), (1, 5, 64, 2, 130, "shared")])
def test_device_entry_matches_host_entry(b, tq, tkv, h, d, kind):
    """rt_mha_forward_masked_f32_dev on a stream of its own gives the bits of the host-slice entry (same kernels)."""
    from _gpu import dev

    rng = np.random.default_rng(13)
    q = rng.standard_normal(b * tq * h * d).astype(np.float32)
    k = rng.standard_normal(b * tkv * h * d).astype(np.float32)
    v = rng.standard_normal(b * tkv * h * d).astype(np.float32)
    mask = {"none": None, "causal": ra.causal_mask(tq) if tq == tkv else None,
            "shared": np.where(rng.random((tq, tkv)) > 0.3, 0.0, -1.0e4).astype(np.float32),
            "per_head": rng.standard_normal((b * h, tq, tkv)).astype(np.float32)}[kind]
    want = ra.mha_forward_masked_f32(q, k, v, b, tq, tkv, h, d, mask)
    st = ra.Stream()
    dq, dk, dv = dev(q), dev(k), dev(v)
    dm = dev(mask.ravel()) if mask is not None else None
    dout = ra.HipStorage.zeros(q.nbytes)
    ra.mha_forward_masked_f32_dev(dq, dk, dv, dout, b, tq, tkv, h, d, dm, 0 if mask is None else mask.size, stream=st)
    st.synchronize()
    assert np.array_equal(dout.download(np.float32), want)
