"""Pins the oracle's attention backward (ro_flash_backward, restating crates/rustorch-attention/src/cpu_backward.rs:46-185).

Reference tests restated (cpu_backward.rs:230-299): finite-difference spot check of dQ at three indices, the
empty-sequence no-op, the length error naming "q", zero upstream gradient => zero gradients.
Independent anchors, each of which a dropped term, a wrong sign or a transposed operand fails:
torch autograd through a float64 softmax(QK^T/sqrt(d))V for all three gradients; central differences of the
oracle's own naive forward for dK and dV as well as dQ; the closed form for a single key (P == 1: dV = dO,
dQ = dK = 0); the identity sum_j dS_ij = 0 seen as "adding the same vector to every key leaves dQ unchanged"."""
import numpy as np
import pytest
import torch

from _util import lcg_buffer


def _inputs(oracle, b, h, n, d, seeds=(1, 2, 3, 4)):
    shape = oracle.AttentionShape(b, h, n, d)
    return shape, [lcg_buffer(shape.buffer_len(), s) for s in seeds]


def _torch_grads(q, k, v, d_out, b, h, n, d):
    t = [torch.tensor(np.asarray(a, dtype=np.float64).reshape(b, h, n, d), requires_grad=True) for a in (q, k, v)]
    s = (t[0] @ t[1].transpose(-1, -2)) / np.sqrt(np.float64(np.float32(d)))
    out = torch.softmax(s, -1) @ t[2]
    out.backward(torch.tensor(np.asarray(d_out, dtype=np.float64).reshape(b, h, n, d)))
    return [x.grad.numpy().ravel() for x in t]


# ---- reference tests ------------------------------------------------------------------------------------------


def _fd(oracle, shape, bufs, which, idx, eps):
    q, k, v, d_out = [a.copy() for a in bufs]
    tgt = (q, k, v)[which]
    saved = tgt[idx]
    tgt[idx] = saved + np.float32(eps)
    plus = oracle.naive_forward(shape, q, k, v)
    tgt[idx] = saved - np.float32(eps)
    minus = oracle.naive_forward(shape, q, k, v)
    return float(np.sum(d_out.astype(np.float64) * (plus.astype(np.float64) - minus) / (2.0 * eps)))


def test_dq_matches_finite_difference(oracle):
    shape, bufs = _inputs(oracle, 1, 1, 4, 4)
    dq, dk, dv = oracle.flash_backward(shape, *bufs)
    for idx in (0, 5, 10):
        assert abs(dq[idx] - _fd(oracle, shape, bufs, 0, idx, 1e-3)) < 5e-3


def test_empty_seq_is_no_op(oracle):
    shape = oracle.AttentionShape(1, 1, 0, 4)
    e = np.zeros(0, dtype=np.float32)
    dq, dk, dv = oracle.flash_backward(shape, e, e, e, e)
    assert dq.size == 0 and dk.size == 0 and dv.size == 0


def test_shape_mismatch_names_q(oracle):
    shape = oracle.AttentionShape(1, 1, 4, 4)
    z = np.zeros(16, dtype=np.float32)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_backward(shape, np.zeros(10, dtype=np.float32), z, z, z)
    assert ei.value.code == 2 and ei.value.which == "q" and (ei.value.expected, ei.value.got) == (16, 10)


def test_zero_grad_yields_zero_outputs(oracle):
    shape, bufs = _inputs(oracle, 1, 1, 3, 4)
    bufs[3] = np.zeros_like(bufs[3])
    for g in oracle.flash_backward(shape, *bufs):
        assert np.array_equal(g, np.zeros_like(g))


# ---- the order of the length checks (cpu_backward.rs:59-74) ---------------------------------------------------


def test_length_checks_in_order(oracle):
    shape = oracle.AttentionShape(1, 2, 3, 4)
    ok = np.zeros(24, dtype=np.float32)
    bad = np.zeros(5, dtype=np.float32)
    for pos, name in enumerate(("q", "k", "v", "do")):
        args = [ok] * 4
        for later in range(pos, 4):  # everything from `pos` on is wrong: the first wrong one is named
            args[later] = bad
        with pytest.raises(oracle.OracleError) as ei:
            oracle.flash_backward(shape, *args, out_lens=(1, 2, 3))
        assert ei.value.code == 2 and ei.value.which == name
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_backward(shape, ok, ok, ok, ok, out_lens=(24, 30, 7))
    assert ei.value.code == 3 and (ei.value.expected, ei.value.got) == (24, 30)  # got = the longest


def test_outputs_are_overwritten_not_accumulated(oracle):
    shape, bufs = _inputs(oracle, 1, 1, 5, 8)
    first = oracle.flash_backward(shape, *bufs)
    second = oracle.flash_backward(shape, *bufs)
    for a, b in zip(first, second):
        assert np.array_equal(a, b)


# ---- independent anchors --------------------------------------------------------------------------------------


@pytest.mark.parametrize("b,h,n,d", [(1, 1, 4, 4), (2, 3, 17, 8), (1, 2, 64, 32), (1, 1, 33, 5), (1, 1, 130, 64)])
def test_against_torch_autograd_f64(oracle, b, h, n, d):
    shape, bufs = _inputs(oracle, b, h, n, d, seeds=(11, 12, 13, 14))
    got = oracle.flash_backward(shape, *bufs)
    want = _torch_grads(*bufs, b, h, n, d)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert np.abs(g - w).max() < 2e-6 * max(1.0, np.sqrt(n)), name


def test_dk_dv_match_finite_difference(oracle):
    shape, bufs = _inputs(oracle, 1, 2, 6, 4, seeds=(5, 6, 7, 8))
    grads = oracle.flash_backward(shape, *bufs)
    for which in (0, 1, 2):
        for idx in (0, 7, 23, 47):
            assert abs(grads[which][idx] - _fd(oracle, shape, bufs, which, idx, 1e-2)) < 2e-3, (which, idx)


def test_single_key_closed_form(oracle):
    # one key: P == 1 whatever q and k are, so out = v, dV = dO, and nothing depends on q or k
    shape, bufs = _inputs(oracle, 2, 2, 1, 16)
    dq, dk, dv = oracle.flash_backward(shape, *bufs)
    assert np.array_equal(dv, bufs[3])
    assert np.array_equal(dq, np.zeros_like(dq)) and np.array_equal(dk, np.zeros_like(dk))


def test_dq_is_orthogonal_to_a_common_key_shift(oracle):
    # softmax is invariant to adding one vector c to every key, and then dQ_i = scale * sum_j dS_ij (K_j + c)
    # = the unshifted dQ_i because sum_j dS_ij = 0
    shape, bufs = _inputs(oracle, 1, 1, 9, 8)
    q, k, v, d_out = bufs
    c = lcg_buffer(8, 99)
    k2 = (k.reshape(9, 8) + c[None, :]).astype(np.float32).ravel()
    # q.c differs per row, which shifts every score of a row by the same amount: P is unchanged
    dq1, _, dv1 = oracle.flash_backward(shape, q, k, v, d_out)
    dq2, _, dv2 = oracle.flash_backward(shape, q, k2, v, d_out)
    assert np.abs(dq1 - dq2).max() < 2e-6 and np.abs(dv1 - dv2).max() < 2e-6
