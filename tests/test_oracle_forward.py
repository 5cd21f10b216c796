"""Pins the CPU oracle's forward functions.

The checks are the reference's own tests for this path, restated on the oracle
(crates/rustorch-attention/src/cpu_forward.rs:804-1087 and tests/equivalence.rs:34-143),
plus independent anchors a plausible mistake would trip: a float64 brute force, torch's
scaled_dot_product_attention (a library routine), closed forms, and the NaN rules.
"""
import numpy as np
import pytest
import torch

from _util import attention_f64, close_ref, hash_buffer, lcg_buffer, seeded_normal

FIXTURE_SHAPES = [  # tests/equivalence.rs:34-77
    (1, 1, 1, 4), (1, 1, 2, 4), (1, 1, 16, 8), (1, 2, 32, 16), (2, 2, 32, 16), (1, 4, 64, 32), (2, 4, 128, 32),
    (1, 8, 64, 64), (1, 8, 128, 64), (2, 8, 128, 64), (4, 8, 128, 64), (1, 1, 63, 32), (1, 1, 64, 32),
    (1, 1, 65, 32), (1, 1, 127, 32), (1, 1, 128, 32), (1, 1, 129, 32), (1, 1, 32, 4), (1, 1, 32, 128),
    (1, 1, 96, 48),
]


def shape_buffers(shape, span):
    n = shape.buffer_len()
    return lcg_buffer(n, 0xC0FFEE, span), lcg_buffer(n, 0xBADBEEF, span), lcg_buffer(n, 0xCAFE00, span)


@pytest.mark.parametrize("bhnd", FIXTURE_SHAPES)
def test_flash_matches_naive_on_20_fixed_shapes(oracle, bhnd):
    """tests/equivalence.rs:95-125: max-abs < 1e-4 and Frobenius < 1e-4*sqrt(n)."""
    shape = oracle.AttentionShape(*bhnd)
    q, k, v = shape_buffers(shape, 2.0)
    o_flash = oracle.flash_forward(shape, q, k, v)
    o_naive = oracle.naive_forward(shape, q, k, v)
    d = np.abs(o_flash - o_naive)
    assert d.max() < 1e-4
    assert np.sqrt((d.astype(np.float64) ** 2).sum()) < 1e-4 * np.sqrt(shape.buffer_len())
    # every output finite (equivalence.rs:128-143)
    assert np.isfinite(o_flash).all()
    # independent anchor: float64 brute force, far tighter than the reference's own bar
    ref = attention_f64(q.reshape(bhnd), k.reshape(bhnd), v.reshape(bhnd)).ravel()
    assert np.abs(o_flash - ref).max() < 5e-6
    assert np.abs(o_naive - ref).max() < 5e-6
    # the row-by-row statement of the recurrence (cpu_forward.rs:594-686) agrees as well
    assert np.abs(oracle.flash_forward_scalar(shape, q, k, v) - ref).max() < 5e-6


@pytest.mark.parametrize("bhnd,br,bc", [((2, 4, 32, 16), 64, 64), ((1, 2, 70, 24), 64, 64),
                                        ((2, 4, 128, 64), 64, 64), ((4, 8, 96, 32), 64, 64),
                                        ((1, 2, 70, 24), 16, 32), ((1, 2, 70, 24), 7, 5)])
def test_flash_matches_naive_unit_shapes(oracle, bhnd, br, bc):
    """cpu_forward.rs:804-840, :917-929 (span-3 LCG, atol 1e-4 + 1e-4 rel), plus odd tile sizes."""
    shape = oracle.AttentionShape(*bhnd, br=br, bc=bc)
    q, k, v = shape_buffers(shape, 3.0)
    assert close_ref(oracle.flash_forward(shape, q, k, v), oracle.naive_forward(shape, q, k, v), 1e-4)


def test_scaling_factor_is_one_over_sqrt_d(oracle):
    """cpu_forward.rs:843-856: N=1 => out == v."""
    shape = oracle.AttentionShape(1, 1, 1, 4)
    v = np.array([5.0, -2.0, 7.0, 1.0], dtype=np.float32)
    e0 = np.array([1.0, 0, 0, 0], dtype=np.float32)
    assert close_ref(oracle.flash_forward(shape, e0, e0, v), v, 1e-6)


def test_scale_value_two_keys_analytic(oracle):
    """A wrong scale (1/d, none, sqrt(d)) fails this: q=k0=4*e0, k1=0, D=16 => scores (4, 0)
    => weights softmax([4, 0]) exactly."""
    D = 16
    shape = oracle.AttentionShape(1, 1, 2, D)
    q = np.zeros((2, D), dtype=np.float32)
    k = np.zeros((2, D), dtype=np.float32)
    q[:, 0] = 4.0
    k[0, 0] = 4.0
    v = np.zeros((2, D), dtype=np.float32)
    v[0, :] = 1.0
    v[1, :] = -1.0
    w0 = 1.0 / (1.0 + np.exp(-4.0))
    expect = w0 * 1.0 + (1 - w0) * -1.0
    for fn in (oracle.flash_forward, oracle.naive_forward):
        out = fn(shape, q, k, v)
        assert np.allclose(out, expect, atol=1e-6)


def test_empty_seq_is_no_op(oracle):
    """cpu_forward.rs:861-869."""
    shape = oracle.AttentionShape(2, 4, 0, 16)
    e = np.zeros(0, dtype=np.float32)
    assert oracle.flash_forward(shape, e, e, e).size == 0


def test_zero_dim_returns_error(oracle):
    """cpu_forward.rs:872-882; ZeroDim is checked before any length."""
    shape = oracle.AttentionShape(1, 1, 4, 0)
    e = np.zeros(0, dtype=np.float32)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward(shape, e, e, e)
    assert ei.value.code == oracle.ERR_ZERO_DIM
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward(shape, np.zeros(3, np.float32), e, e)
    assert ei.value.code == oracle.ERR_ZERO_DIM


def test_buffer_size_mismatch_returns_error(oracle):
    """cpu_forward.rs:885-896 and the q,k,v,out check order of validate (:142-169)."""
    shape = oracle.AttentionShape(1, 1, 4, 8)
    good = np.zeros(32, dtype=np.float32)
    bad = np.zeros(16, dtype=np.float32)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward(shape, good, bad, good)
    assert (ei.value.code, ei.value.which, ei.value.expected, ei.value.got) == (
        oracle.ERR_BUFFER_SHAPE_MISMATCH, "k", 32, 16)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward(shape, bad, bad, bad)
    assert ei.value.which == "q"
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward(shape, good, good, bad)
    assert ei.value.which == "v"
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward(shape, good, good, good, out_len=31)
    assert (ei.value.code, ei.value.expected, ei.value.got) == (oracle.ERR_OUTPUT_SHAPE_MISMATCH, 32, 31)


def test_nan_input_propagates_to_output(oracle):
    """cpu_forward.rs:898-915 (br=bc=4): same NaN pattern in flash and naive; a NaN in Q row 0
    poisons row 0 only."""
    shape = oracle.AttentionShape(1, 1, 4, 8, br=4, bc=4)
    q = lcg_buffer(32, 1, 3.0)
    q[0] = np.nan
    k = lcg_buffer(32, 2, 3.0)
    v = lcg_buffer(32, 3, 3.0)
    f = oracle.flash_forward(shape, q, k, v).reshape(4, 8)
    n = oracle.naive_forward(shape, q, k, v).reshape(4, 8)
    assert np.array_equal(np.isnan(f), np.isnan(n))
    assert np.isnan(f[0]).all() and np.isfinite(f[1:]).all()


def test_causal_flash_matches_causal_naive(oracle):
    """cpu_forward.rs:934-941 + float64 anchor."""
    shape = oracle.AttentionShape(1, 2, 64, 32)
    q, k, v = shape_buffers(shape, 3.0)
    f = oracle.flash_forward_masked(shape, q, k, v, "causal")
    n = oracle.naive_forward_masked(shape, q, k, v, "causal")
    assert close_ref(f, n, 1e-4)
    ref = attention_f64(q.reshape(1, 2, 64, 32), k.reshape(1, 2, 64, 32), v.reshape(1, 2, 64, 32), "causal")
    assert np.abs(f - ref.ravel()).max() < 5e-6


def test_padding_flash_matches_padding_naive(oracle):
    """cpu_forward.rs:944-953 + float64 anchor."""
    shape = oracle.AttentionShape(1, 1, 8, 4)
    q, k, v = shape_buffers(shape, 3.0)
    keep = [True, False, True, True, False, True, False, True]
    f = oracle.flash_forward_masked(shape, q, k, v, ("padding", keep))
    n = oracle.naive_forward_masked(shape, q, k, v, ("padding", keep))
    assert close_ref(f, n, 1e-4)
    ref = attention_f64(q.reshape(1, 1, 8, 4), k.reshape(1, 1, 8, 4), v.reshape(1, 1, 8, 4), ("padding", keep))
    assert np.abs(f - ref.ravel()).max() < 5e-6


def test_causal_first_query_only_attends_to_self(oracle):
    """cpu_forward.rs:956-980: row 0 == V[0]."""
    shape = oracle.AttentionShape(1, 1, 4, 8)
    ones = np.ones(32, dtype=np.float32)
    v = np.zeros(32, dtype=np.float32)
    v[0:8] = 10.0 * np.arange(1, 9)
    v[8:16] = -99.0
    v[16:24] = 99.0
    out = oracle.flash_forward_masked(shape, ones, ones, v, "causal")
    assert close_ref(out[:8], v[:8], 1e-6)


def test_causal_constant_qk_gives_prefix_means(oracle):
    """Closed form: constant Q,K => row i is the mean of V[0..=i]; an off-by-one in the causal
    rule (kj >= qi) fails it."""
    N, D = 70, 8
    shape = oracle.AttentionShape(1, 1, N, D)
    ones = np.ones(N * D, dtype=np.float32)
    v = seeded_normal((N, D), 5)
    expect = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, N + 1)[:, None]
    for fn in (oracle.flash_forward_masked, oracle.naive_forward_masked):
        out = fn(shape, ones, ones, v, "causal").reshape(N, D)
        assert np.abs(out - expect).max() < 2e-6


def test_padding_mask_excludes_padded_positions_exactly(oracle):
    """cpu_forward.rs:983-998: keep=[T,F,F,T], q=k=1 => out[0] = (10+30)/2 = 20."""
    shape = oracle.AttentionShape(1, 1, 4, 4)
    ones = np.ones(16, dtype=np.float32)
    v = np.array([10, 0, 0, 0, 99, 0, 0, 0, -99, 0, 0, 0, 30, 0, 0, 0], dtype=np.float32)
    out = oracle.flash_forward_masked(shape, ones, ones, v, ("padding", [True, False, False, True]))
    assert abs(out[0] - 20.0) <= 1e-5


def test_padding_mask_length_mismatch_returns_error(oracle):
    """cpu_forward.rs:1001-1014."""
    shape = oracle.AttentionShape(1, 1, 4, 4)
    q, k, v = shape_buffers(shape, 3.0)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.flash_forward_masked(shape, q, k, v, ("padding", [True] * 3))
    assert (ei.value.code, ei.value.expected, ei.value.got) == (oracle.ERR_PADDING_LENGTH_MISMATCH, 4, 3)


def test_flash_stable_for_large_q_k_magnitudes(oracle):
    """cpu_forward.rs:1017-1037."""
    shape = oracle.AttentionShape(1, 1, 16, 8)
    i = np.arange(shape.buffer_len(), dtype=np.float32)
    q = (1e3 + np.sin(i * np.float32(0.01))).astype(np.float32)
    k = (1e3 + np.cos(i * np.float32(0.013))).astype(np.float32)
    v = np.sin(i * np.float32(0.07)).astype(np.float32)
    f = oracle.flash_forward(shape, q, k, v)
    n = oracle.naive_forward(shape, q, k, v)
    assert close_ref(f, n, 1e-3)
    assert np.isfinite(f).all()


def test_flash_matches_naive_random_shapes(oracle):
    """cpu_forward.rs:1045-1087: 200 random (B,H,N,D), br=bc=16, tol 1e-3 + 1e-3 rel; plus the
    committed regression seed B=H=N=1, D=4 (proptest-regressions/cpu_forward.txt:7)."""
    rng = np.random.default_rng(20260504)
    cases = [(1, 1, 1, 4)] + [(int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.integers(1, 40)),
                               int(rng.integers(4, 16))) for _ in range(200)]
    for bhnd in cases:
        shape = oracle.AttentionShape(*bhnd, br=16, bc=16)
        n = shape.buffer_len()
        q, k, v = hash_buffer(n, 1), hash_buffer(n, 13), hash_buffer(n, 29)
        assert close_ref(oracle.flash_forward(shape, q, k, v), oracle.naive_forward(shape, q, k, v), 1e-3, 1e-3), bhnd


@pytest.mark.parametrize("mask", [None, "causal"])
def test_oracle_matches_torch_sdpa(oracle, mask):
    """Library anchor: torch's CPU scaled_dot_product_attention on N(0,1) inputs."""
    bhnd = (2, 3, 150, 64)
    q, k, v = (seeded_normal(bhnd, s) for s in (11, 12, 13))
    shape = oracle.AttentionShape(*bhnd)
    out = oracle.flash_forward_masked(shape, q, k, v, mask).reshape(bhnd)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).double(), torch.from_numpy(k).double(), torch.from_numpy(v).double(),
        is_causal=(mask == "causal")).numpy()
    assert np.abs(out - ref).max() < 5e-6


def test_fully_masked_rows_are_nan(oracle):
    """cpu_forward.rs:411-420 / :754-758: no visible key => the whole row is NaN, in flash and naive."""
    shape = oracle.AttentionShape(1, 2, 5, 4)
    q, k, v = shape_buffers(shape, 2.0)
    keep = [False] * 5
    for fn in (oracle.flash_forward_masked, oracle.naive_forward_masked, oracle.flash_forward_scalar):
        assert np.isnan(fn(shape, q, k, v, ("padding", keep))).all()


def test_leading_fully_masked_kv_tile_poisons_tiled_forward(oracle):
    """A property of the reference's tiled recurrence worth pinning because the HIP path must
    reproduce it: when the FIRST kv tile [0, bc) has no visible key, p = exp(-inf - (-inf)) = NaN
    enters l (cpu_forward.rs:364-384) and, since alpha is forced to 0 rather than skipping the
    update, NaN*0 keeps it there: every row comes out NaN although later keys are visible.  The
    naive path (:702-763) gives the finite answer.  With a visible key anywhere in tile 0 the
    two agree."""
    shape = oracle.AttentionShape(1, 1, 12, 4, br=4, bc=4)
    q, k, v = shape_buffers(shape, 2.0)
    keep = [False] * 4 + [True] * 8
    assert np.isnan(oracle.flash_forward_masked(shape, q, k, v, ("padding", keep))).all()
    assert np.isnan(oracle.flash_forward_scalar(shape, q, k, v, ("padding", keep))).all()
    assert np.isfinite(oracle.naive_forward_masked(shape, q, k, v, ("padding", keep))).all()
    keep[3] = True
    f = oracle.flash_forward_masked(shape, q, k, v, ("padding", keep))
    assert close_ref(f, oracle.naive_forward_masked(shape, q, k, v, ("padding", keep)), 1e-5)
    # a fully masked tile AFTER a finite max contributes exactly zero
    keep = [True] * 4 + [False] * 4 + [True] * 4
    f = oracle.flash_forward_masked(shape, q, k, v, ("padding", keep))
    assert close_ref(f, oracle.naive_forward_masked(shape, q, k, v, ("padding", keep)), 1e-5)


def test_mask_is_masked(oracle):
    """mask.rs:96-157."""
    for qi in range(8):
        for kj in range(8):
            assert not oracle.mask_is_masked(None, qi, kj)
    assert not oracle.mask_is_masked("causal", 2, 0)
    assert not oracle.mask_is_masked("causal", 2, 2)
    assert oracle.mask_is_masked("causal", 2, 3)
    assert oracle.mask_is_masked("causal", 0, 1)
    keep = [True, False, True, True, False]
    assert [oracle.mask_is_masked(("padding", keep), 0, j) for j in range(5)] == [False, True, False, False, True]
    assert not oracle.mask_is_masked(("padding", []), 0, 0)
    assert not oracle.mask_is_masked(("padding", keep), 0, 7)  # out of range => not masked
    for i in range(16):
        assert not oracle.mask_is_masked("causal", i, i)


def test_threads_do_not_change_result(oracle):
    shape = oracle.AttentionShape(3, 4, 96, 32)
    q, k, v = shape_buffers(shape, 2.0)
    a = oracle.flash_forward_masked(shape, q, k, v, "causal", threads=1)
    b = oracle.flash_forward_masked(shape, q, k, v, "causal", threads=8)
    assert np.array_equal(a, b)


def test_varlen_causal_matches_f64_on_valid_rows(oracle):
    """Padded-batch convention: valid rows equal causal attention over the sequence's own
    prefix; padded rows are exactly 0.0 (or NaN when zero fill is off)."""
    B, H, N, D = 3, 2, 40, 16
    lens = [40, 17, 1]
    q, k, v = (seeded_normal((B, H, N, D), s) for s in (1, 2, 3))
    out = oracle.varlen_causal_forward(q, k, v, lens, B, H, N, D).reshape(B, H, N, D)
    nan_out = oracle.varlen_causal_forward(q, k, v, lens, B, H, N, D, zero_padded_rows=False).reshape(B, H, N, D)
    for b, n in enumerate(lens):
        ref = attention_f64(q[b:b + 1, :, :n], k[b:b + 1, :, :n], v[b:b + 1, :, :n], "causal")[0]
        assert np.abs(out[b, :, :n] - ref).max() < 5e-6
        assert (out[b, :, n:] == 0.0).all()
        assert np.isnan(nan_out[b, :, n:]).all()


def test_non_finite_v_row_poisons_every_row_even_where_hidden(oracle):
    """cpu_forward.rs:268-425 multiplies P (exact zeros where masked) into every V tile: 0 * NaN = NaN reaches every
    query row in that column, hidden or not, in the tiled form; the scalar and naive forms agree."""
    b, h, n, d, j = 1, 1, 130, 8, 100
    q, k, v = (lcg_buffer(b * h * n * d, s, 2.0) for s in (5, 6, 7))
    v = v.copy()
    v[j * d + 2] = np.nan
    sh = oracle.AttentionShape(b, h, n, d)
    out = oracle.flash_forward_masked(sh, q, k, v, "causal").reshape(n, d)
    assert np.isnan(out[:, 2]).all() and np.isfinite(np.delete(out, 2, axis=1)).all()
    naive = oracle.naive_forward_masked(sh, q, k, v, "causal").reshape(n, d)
    assert np.array_equal(np.isnan(naive), np.isnan(out))
