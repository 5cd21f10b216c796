"""GPU parity of the f32 attention backward through the C ABI (rt_flash_backward_f32, rt_flash_backward_f32_dev)
against the CPU oracle's restatement of crates/rustorch-attention/src/cpu_backward.rs:46-185.

Bar: max-abs <= 2e-5 on every gradient for inputs in (-1, 1) (the kernels sum in f32 in another order than the
reference's scalar loops, and use exp2 on pre-scaled scores; the reference's own check of its backward is a finite
difference at 5e-3).  The reference's four tests run first, against the device."""
import ctypes as C

import numpy as np
import pytest

import rustorch_amd as ra
from rustorch_amd import _lib as L
from _gpu import dev, max_abs
from _util import lcg_buffer, seeded_normal

pytestmark = pytest.mark.gpu
TOL = 2e-5


def inputs(bhnd, seeds=(1, 2, 3, 4)):
    shape = ra.AttentionShape.new(*bhnd)
    return shape, [lcg_buffer(shape.buffer_len(), s) for s in seeds]


# ---- the reference's tests (cpu_backward.rs:230-299) ----------------------------------------------------------


def test_dq_matches_finite_difference():
    shape, (q, k, v, d_out) = inputs((1, 1, 4, 4))
    dq, dk, dv = ra.flash_backward(shape, q, k, v, d_out)
    for idx in (0, 5, 10):
        qp, qm = q.copy(), q.copy()
        qp[idx] += np.float32(1e-3)
        qm[idx] -= np.float32(1e-3)
        o_plus, o_minus = ra.flash_forward(shape, qp, k, v), ra.flash_forward(shape, qm, k, v)
        numeric = float(np.sum(d_out.astype(np.float64) * (o_plus.astype(np.float64) - o_minus) / 2e-3))
        assert abs(dq[idx] - numeric) < 5e-3, (idx, dq[idx], numeric)


def test_zero_grad_yields_zero_outputs():
    shape, (q, k, v, _) = inputs((1, 1, 3, 4))
    junk = [np.full(shape.buffer_len(), 7.0, dtype=np.float32) for _ in range(3)]
    grads = ra.flash_backward(shape, q, k, v, np.zeros(shape.buffer_len(), np.float32), *junk)
    for g in grads:
        assert np.array_equal(g, np.zeros_like(g))


def test_shape_mismatch_and_empty_seq():
    shape = ra.AttentionShape.new(1, 1, 4, 4)
    z = np.zeros(16, np.float32)
    with pytest.raises(ra.BufferShapeMismatch) as ei:
        ra.flash_backward(shape, np.zeros(10, np.float32), z, z, z)
    assert ei.value.which == "q"
    e = np.zeros(0, np.float32)
    assert ra.flash_backward(ra.AttentionShape.new(1, 1, 0, 4), e, e, e, e)[0].size == 0


# ---- parity with the oracle -----------------------------------------------------------------------------------

SHAPES = [(1, 1, 4, 4), (1, 1, 1, 16), (2, 3, 17, 8), (1, 2, 64, 32), (1, 1, 33, 5), (1, 1, 130, 64), (2, 2, 100, 128),
          (1, 2, 257, 96), (1, 1, 300, 100), (3, 1, 31, 33), (1, 4, 512, 64), (1, 1, 129, 1), (1, 1, 96, 127),
          # above the tiled kernels' registers: a workgroup per row (the reference has no limit, cpu_backward.rs:46-185)
          (1, 2, 70, 129), (2, 1, 33, 200), (1, 1, 130, 256), (1, 1, 65, 257), (1, 2, 40, 320), (1, 1, 17, 512)]


@pytest.mark.parametrize("bhnd", SHAPES)
def test_backward_matches_oracle(oracle, bhnd):
    shape, bufs = inputs(bhnd, seeds=(11, 12, 13, 14))
    got = ra.flash_backward(shape, *bufs)
    want = oracle.flash_backward(oracle.AttentionShape(*bhnd), *bufs)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert np.isfinite(g).all(), name
        assert max_abs(g, w) <= TOL, f"{bhnd} {name}: {max_abs(g, w):.3e}"


def test_backward_matches_oracle_on_normal_inputs(oracle):
    bhnd = (1, 2, 200, 64)
    shape = ra.AttentionShape.new(*bhnd)
    bufs = [seeded_normal(shape.buffer_len(), s) for s in (21, 22, 23, 24)]
    got = ra.flash_backward(shape, *bufs)
    want = oracle.flash_backward(oracle.AttentionShape(*bhnd), *bufs)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        # standard-normal scores reach +-10: gradients of a few units, errors scale with them
        assert max_abs(g, w) <= 1e-5 * max(1.0, float(np.abs(w).max())) * 4, name


def test_backward_head_dim_above_512_is_refused():
    shape = ra.AttentionShape.new(1, 1, 4, 513)
    z = np.zeros(shape.buffer_len(), np.float32)
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_backward(shape, z, z, z, z)
    assert ei.value.status == 21 and ei.value.expected == 512


def test_outputs_are_overwritten(oracle):
    shape, bufs = inputs((1, 2, 40, 16))
    clean = ra.flash_backward(shape, *bufs)
    junk = [np.full(shape.buffer_len(), np.nan, dtype=np.float32) for _ in range(3)]
    dirty = ra.flash_backward(shape, *bufs, *junk)
    for a, b in zip(clean, dirty):
        assert np.array_equal(a, b)  # also: the same launch twice gives the same bits (no atomics)


# ---- device-pointer entry -------------------------------------------------------------------------------------


def run_dev(shape, bufs, misalign=0):
    n = shape.buffer_len()
    d_in = [dev(np.concatenate([np.zeros(misalign, np.float32), b])) for b in bufs]
    d_out = [ra.HipStorage.zeros((n + misalign) * 4) for _ in range(3)]
    ws_bytes = ra.flash_backward_workspace_bytes(shape)
    ws = ra.HipStorage.zeros(ws_bytes)
    ra.flash_backward_f32_dev(shape, *[x.ptr + 4 * misalign for x in d_in], *[x.ptr + 4 * misalign for x in d_out], ws,
                              ws_bytes)
    ra.synchronize()
    return [x.download(np.float32)[misalign:] for x in d_out]


@pytest.mark.parametrize("bhnd,misalign", [((1, 2, 70, 64), 0), ((1, 2, 70, 64), 1), ((2, 1, 45, 20), 0), ((1, 1, 64, 128), 3)])
def test_device_entry_matches_host_entry(bhnd, misalign):
    shape, bufs = inputs(bhnd, seeds=(5, 6, 7, 8))
    want = ra.flash_backward(shape, *bufs)
    got = run_dev(shape, bufs, misalign)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        if misalign == 0:
            assert np.array_equal(g, w), name
        else:  # rows that are not 16-byte aligned take the element-wise loads and the other forward kernel
            assert max_abs(g, w) <= TOL, name


def test_device_entry_checks_workspace():
    shape = ra.AttentionShape.new(1, 1, 8, 8)
    s = shape._c()
    err = L.RtErr()
    buf = ra.HipStorage.zeros(4096)
    rc = L.lib().rt_flash_backward_f32_dev(None, C.byref(s), *([buf.ptr] * 7), buf.ptr, 16, C.byref(err))
    assert rc == L.RT_ERR_WORKSPACE_TOO_SMALL and err.expected == 8 * 10 * 4


# ---- full size: one head against the oracle, the whole tensor through identities ------------------------------


def test_full_size_single_head_matches_oracle(oracle):
    bhnd = (1, 1, 2048, 64)
    shape, bufs = inputs(bhnd, seeds=(31, 32, 33, 34))
    got = ra.flash_backward(shape, *bufs)
    want = oracle.flash_backward(oracle.AttentionShape(*bhnd), *bufs)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert max_abs(g, w) <= TOL, f"{name}: {max_abs(g, w):.3e}"


def test_full_size_identities():
    """B1 H8 N2048 D64.  Rows of P sum to 1, so sum_j dV_j = sum_i dO_i; sum_i Q_i.dQ_i = sum_j K_j.dK_j (both are
    scale * sum_ij dS_ij S_ij); and the gradients are linear in dO."""
    bhnd = (1, 8, 2048, 64)
    shape = ra.AttentionShape.new(*bhnd)
    q, k, v, d1, d2 = [seeded_normal(shape.buffer_len(), s) * np.float32(0.5) for s in (41, 42, 43, 44, 45)]
    dq, dk, dv = ra.flash_backward(shape, q, k, v, d1)
    r = lambda a: np.asarray(a, dtype=np.float64).reshape(bhnd)
    assert np.abs(r(dv).sum(axis=2) - r(d1).sum(axis=2)).max() < 2e-3  # sums of 2048 terms of size ~0.5
    lhs = (r(q) * r(dq)).sum(axis=(2, 3))
    rhs = (r(k) * r(dk)).sum(axis=(2, 3))
    assert np.abs(lhs - rhs).max() < 1e-3 * max(1.0, np.abs(lhs).max())
    g2 = ra.flash_backward(shape, q, k, v, d2)
    g3 = ra.flash_backward(shape, q, k, v, (2.0 * d1 - 0.5 * d2).astype(np.float32))
    for a, b, c in zip((dq, dk, dv), g2, g3):
        assert max_abs(2.0 * r(a) - 0.5 * r(b), r(c)) < 5e-5


def test_large_magnitude_scores(oracle):
    """Inputs in (-6, 6): scores reach +-70 and most rows are nearly one-hot.  Errors are relative to the size of the
    gradients (both sides round exp arguments of that size to about 4e-6)."""
    bhnd = (1, 2, 96, 32)
    shape = ra.AttentionShape.new(*bhnd)
    bufs = [lcg_buffer(shape.buffer_len(), s, span=12.0) for s in (51, 52, 53, 54)]
    got = ra.flash_backward(shape, *bufs)
    want = oracle.flash_backward(oracle.AttentionShape(*bhnd), *bufs)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert np.isfinite(g).all()
        assert max_abs(g, w) <= 1e-4 * float(np.abs(w).max()), f"{name}: {max_abs(g, w):.3e} of {np.abs(w).max():.3e}"


# ---- the saved-forward form -----------------------------------------------------------------------------------


@pytest.mark.parametrize("bhnd", [(1, 2, 70, 64), (2, 1, 45, 20), (1, 1, 200, 128), (1, 8, 256, 32)])
def test_saved_forward_form(bhnd):
    """rt_flash_forward_stats_f32_dev leaves the forward's output and lse = m + ln(l); the backward fed with them gives
    the bits of the recomputing backward (it runs the same kernels on the same values)."""
    b, h, n, d = bhnd
    shape, bufs = inputs(bhnd, seeds=(61, 62, 63, 64))
    q, k, v, d_out = bufs
    dq_, dk_, dv_, dg = [dev(x) for x in bufs]
    d_o, d_lse = ra.HipStorage.zeros(shape.buffer_len() * 4), ra.HipStorage.zeros(b * h * n * 4)
    ra.flash_forward_stats_f32_dev(shape, dq_, dk_, dv_, d_o, d_lse)
    ra.synchronize()
    out, lse = d_o.download(np.float32), d_lse.download(np.float32)
    assert np.array_equal(out, ra.flash_forward(shape, q, k, v))
    s = np.einsum("bhid,bhjd->bhij", *[x.astype(np.float64).reshape(bhnd) for x in (q, k)]) / np.sqrt(np.float64(np.float32(d)))
    m = s.max(axis=-1)
    want_lse = m + np.log(np.exp(s - m[..., None]).sum(axis=-1))
    assert max_abs(lse, want_lse.ravel()) <= 1e-5
    grads = [ra.HipStorage.zeros(shape.buffer_len() * 4) for _ in range(3)]
    ws = ra.HipStorage.zeros(b * h * n * 4)
    ra.flash_backward_saved_f32_dev(shape, dq_, dk_, dv_, d_o, d_lse, dg, *grads, ws, ws.byte_len)
    ra.synchronize()
    want = ra.flash_backward(shape, *bufs)
    for name, g, w in zip(("dq", "dk", "dv"), grads, want):
        assert np.array_equal(g.download(np.float32), w), name


def test_saved_forward_form_checks_workspace():
    shape = ra.AttentionShape.new(1, 2, 8, 8)
    buf = ra.HipStorage.zeros(4096)
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_backward_saved_f32_dev(shape, *([buf] * 9), buf, 63)
    assert ei.value.status == L.RT_ERR_WORKSPACE_TOO_SMALL
