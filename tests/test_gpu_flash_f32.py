"""GPU parity of the f32 prefill path through the C ABI (rt_flash_forward[_masked]_f32,
rt_gqa_forward_f32) against the CPU oracle.  Bar: max-abs <= 1e-5, NaN patterns exact.  The cases
are the reference's own (cpu_forward.rs:804-1087, tests/equivalence.rs, gqa.rs:278-388)."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_close_nan, max_abs
from _util import hash_buffer, lcg_buffer, seeded_normal
from test_oracle_forward import FIXTURE_SHAPES

pytestmark = pytest.mark.gpu
TOL = 1e-5


def buffers(n, span):
    return lcg_buffer(n, 0xC0FFEE, span), lcg_buffer(n, 0xBADBEEF, span), lcg_buffer(n, 0xCAFE00, span)


def omask(mask):
    if mask.kind == 0:
        return None
    if mask.kind == 1:
        return "causal"
    return ("padding", mask.keep)


@pytest.mark.parametrize("bhnd", FIXTURE_SHAPES)
def test_flash_matches_oracle_on_20_fixed_shapes(oracle, bhnd):
    shape = ra.AttentionShape.new(*bhnd)
    q, k, v = buffers(shape.buffer_len(), 2.0)
    rng = np.random.default_rng(bhnd[2])
    keep = rng.random(bhnd[2]) < 0.7
    keep[0] = True
    for mask in (ra.Mask.none(), ra.Mask.causal(), ra.Mask.padding(keep)):
        got = ra.flash_forward_masked(shape, q, k, v, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(*bhnd), q, k, v, omask(mask))
        assert_close_nan(got, want, TOL, f"{bhnd} mask={mask.kind}")
        assert np.isfinite(got).all()


@pytest.mark.parametrize("bhnd", [(2, 4, 32, 16), (1, 2, 70, 24), (2, 4, 128, 64), (4, 8, 96, 32), (1, 3, 300, 128),
                                  (1, 2, 33, 100), (2, 1, 257, 5)])
def test_flash_matches_oracle_unit_shapes(oracle, bhnd):
    shape = ra.AttentionShape.new(*bhnd)
    q, k, v = buffers(shape.buffer_len(), 3.0)
    for mask in (ra.Mask.none(), ra.Mask.causal()):
        got = ra.flash_forward_masked(shape, q, k, v, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(*bhnd), q, k, v, omask(mask))
        assert_close_nan(got, want, TOL, str(bhnd))


@pytest.mark.parametrize("bhnd", [(1, 2, 70, 129), (1, 1, 100, 192), (2, 1, 65, 256), (1, 1, 33, 200)])
def test_flash_head_dims_above_128(oracle, bhnd):
    shape = ra.AttentionShape.new(*bhnd)
    q, k, v = buffers(shape.buffer_len(), 2.0)
    keep = np.arange(bhnd[2]) % 3 != 1
    for mask in (ra.Mask.none(), ra.Mask.causal(), ra.Mask.padding(keep)):
        got = ra.flash_forward_masked(shape, q, k, v, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(*bhnd), q, k, v, omask(mask))
        assert_close_nan(got, want, TOL, f"{bhnd} mask={mask.kind}")


@pytest.mark.parametrize("bhnd", [(1, 2, 70, 257), (2, 1, 33, 320), (1, 1, 130, 512), (1, 2, 5, 300)])
def test_flash_head_dims_above_256(oracle, bhnd):
    """The reference takes any dim != 0 (cpu_forward.rs:142-169): above the tiled kernels a workgroup per query row
    serves the same masks and row rules, fully masked rows and the leading-masked-tile rule included."""
    shape = ra.AttentionShape.new(*bhnd)
    q, k, v = buffers(shape.buffer_len(), 2.0)
    n = bhnd[2]
    keep = np.arange(n) % 3 != 1
    lead = np.r_[np.zeros(min(64, n), bool), np.ones(max(n - 64, 0), bool)]
    for mask in (ra.Mask.none(), ra.Mask.causal(), ra.Mask.padding(keep), ra.Mask.padding(lead), ra.Mask.padding(np.zeros(n, bool))):
        got = ra.flash_forward_masked(shape, q, k, v, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(*bhnd), q, k, v, omask(mask))
        assert_close_nan(got, want, TOL, f"{bhnd} mask={mask.kind}")


def test_flash_head_dim_above_512_is_refused():
    shape = ra.AttentionShape.new(1, 1, 4, 513)
    z = np.zeros(shape.buffer_len(), np.float32)
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_forward(shape, z, z, z)
    assert ei.value.status == 21 and ei.value.expected == 512


def test_scaling_factor_is_one_over_sqrt_d():
    shape = ra.AttentionShape.new(1, 1, 1, 4)
    e0 = np.array([1.0, 0, 0, 0], dtype=np.float32)
    v = np.array([5.0, -2.0, 7.0, 1.0], dtype=np.float32)
    assert max_abs(ra.flash_forward(shape, e0, e0, v), v) <= 1e-6


def test_scale_value_two_keys_analytic():
    D = 16
    shape = ra.AttentionShape.new(1, 1, 2, D)
    q = np.zeros((2, D), dtype=np.float32)
    k = np.zeros((2, D), dtype=np.float32)
    q[:, 0] = 4.0
    k[0, 0] = 4.0
    v = np.zeros((2, D), dtype=np.float32)
    v[0], v[1] = 1.0, -1.0
    w0 = 1.0 / (1.0 + np.exp(-4.0))
    assert np.allclose(ra.flash_forward(shape, q, k, v), 2 * w0 - 1, atol=1e-6)


def test_empty_seq_is_no_op():
    shape = ra.AttentionShape.new(2, 4, 0, 16)
    assert ra.flash_forward(shape, [], [], []).size == 0


def test_errors_in_reference_order():
    e = np.zeros(0, dtype=np.float32)
    with pytest.raises(ra.ZeroDim):
        ra.flash_forward(ra.AttentionShape.new(1, 1, 4, 0), e, e, e)
    shape = ra.AttentionShape.new(1, 1, 4, 8)
    good, bad = np.zeros(32, np.float32), np.zeros(16, np.float32)
    with pytest.raises(ra.BufferShapeMismatch) as ei:
        ra.flash_forward(shape, good, bad, good)
    assert (ei.value.which, ei.value.expected, ei.value.got) == ("k", 32, 16)
    with pytest.raises(ra.OutputShapeMismatch):
        ra.flash_forward(shape, good, good, good, out=np.zeros(31, np.float32))
    with pytest.raises(ra.PaddingLengthMismatch) as ei:
        ra.flash_forward_masked(ra.AttentionShape.new(1, 1, 4, 4), bad, bad, bad, ra.Mask.padding([True] * 3))
    assert (ei.value.expected, ei.value.got) == (4, 3)


def test_nan_input_propagates_to_output(oracle):
    shape = ra.AttentionShape(1, 1, 4, 8, 4, 4)
    q = lcg_buffer(32, 1, 3.0)
    q[0] = np.nan
    k, v = lcg_buffer(32, 2, 3.0), lcg_buffer(32, 3, 3.0)
    got = ra.flash_forward(shape, q, k, v)
    want = oracle.flash_forward(oracle.AttentionShape(1, 1, 4, 8, 4, 4), q, k, v)
    assert_close_nan(got, want, TOL)
    assert np.isnan(got[:8]).all() and np.isfinite(got[8:]).all()
    # a NaN key poisons exactly the rows that can see it
    q = lcg_buffer(32, 1, 3.0)
    k[2 * 8 + 3] = np.nan
    for mask, om in ((ra.Mask.causal(), "causal"), (ra.Mask.none(), None)):
        got = ra.flash_forward_masked(shape, q, k, v, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(1, 1, 4, 8, 4, 4), q, k, v, om)
        assert_close_nan(got, want, TOL)


def test_causal_first_query_only_attends_to_self():
    shape = ra.AttentionShape.new(1, 1, 4, 8)
    ones = np.ones(32, dtype=np.float32)
    v = np.zeros(32, dtype=np.float32)
    v[0:8] = 10.0 * np.arange(1, 9)
    v[8:16], v[16:24] = -99.0, 99.0
    out = ra.flash_forward_masked(shape, ones, ones, v, ra.Mask.causal())
    assert max_abs(out[:8], v[:8]) <= 1e-6


def test_causal_constant_qk_gives_prefix_means():
    N, D = 70, 8
    shape = ra.AttentionShape.new(1, 1, N, D)
    ones = np.ones(N * D, dtype=np.float32)
    v = seeded_normal((N, D), 5)
    expect = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, N + 1)[:, None]
    out = ra.flash_forward_masked(shape, ones, ones, v, ra.Mask.causal()).reshape(N, D)
    assert max_abs(out, expect) < 2e-6


def test_padding_mask_excludes_padded_positions_exactly():
    shape = ra.AttentionShape.new(1, 1, 4, 4)
    ones = np.ones(16, dtype=np.float32)
    v = np.array([10, 0, 0, 0, 99, 0, 0, 0, -99, 0, 0, 0, 30, 0, 0, 0], dtype=np.float32)
    out = ra.flash_forward_masked(shape, ones, ones, v, ra.Mask.padding([True, False, False, True]))
    assert abs(out[0] - 20.0) <= 1e-5


def test_fully_masked_rows_and_leading_masked_tile(oracle):
    """Rows without a visible key are NaN; a padding mask hiding the reference's whole first key
    tile [0, bc) makes every row NaN (what the reference's recurrence produces)."""
    shape = ra.AttentionShape(1, 2, 5, 4)
    q, k, v = buffers(shape.buffer_len(), 2.0)
    assert np.isnan(ra.flash_forward_masked(shape, q, k, v, ra.Mask.padding([False] * 5))).all()
    for bc, keep in ((4, [False] * 4 + [True] * 8), (4, [False] * 3 + [True] * 9), (8, [False] * 7 + [True] * 5),
                     (8, [False] * 8 + [True] * 4), (64, [False] * 11 + [True]), (4, [True] * 4 + [False] * 4 + [True] * 4)):
        shape = ra.AttentionShape(1, 1, 12, 4, 4, bc)
        q, k, v = buffers(shape.buffer_len(), 2.0)
        got = ra.flash_forward_masked(shape, q, k, v, ra.Mask.padding(keep))
        want = oracle.flash_forward_masked(oracle.AttentionShape(1, 1, 12, 4, 4, bc), q, k, v, ("padding", keep))
        assert_close_nan(got, want, TOL, f"bc={bc} keep={keep}")


def test_flash_stable_for_large_q_k_magnitudes(oracle):
    shape = ra.AttentionShape.new(1, 1, 16, 8)
    i = np.arange(shape.buffer_len(), dtype=np.float32)
    q = (1e3 + np.sin(i * np.float32(0.01))).astype(np.float32)
    k = (1e3 + np.cos(i * np.float32(0.013))).astype(np.float32)
    v = np.sin(i * np.float32(0.07)).astype(np.float32)
    got = ra.flash_forward(shape, q, k, v)
    want = oracle.naive_forward(oracle.AttentionShape(1, 1, 16, 8), q, k, v)
    assert np.isfinite(got).all()
    # scores ~1e6/sqrt(8): one f32 ulp of a score is ~0.03, so the reference's own bar (1e-3 rel) applies here
    assert np.all(np.abs(got - want) <= 1e-3 + 1e-3 * np.maximum(np.abs(got), np.abs(want)))


def test_flash_matches_oracle_random_shapes(oracle):
    rng = np.random.default_rng(20260504)
    cases = [(1, 1, 1, 4)] + [(int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.integers(1, 40)),
                               int(rng.integers(4, 16))) for _ in range(100)]
    for bhnd in cases:
        shape = ra.AttentionShape(*bhnd, 16, 16)
        n = shape.buffer_len()
        q, k, v = hash_buffer(n, 1), hash_buffer(n, 13), hash_buffer(n, 29)
        got = ra.flash_forward(shape, q, k, v)
        want = oracle.flash_forward(oracle.AttentionShape(*bhnd, 16, 16), q, k, v)
        assert_close_nan(got, want, TOL, str(bhnd))


def test_config_f32_causal_b1_h8_n2048_d64(oracle):
    """Workload 0 of the benchmark set: the reference's own CPU-runnable case, N(0,1) inputs, causal."""
    bhnd = (1, 8, 2048, 64)
    q, k, v = (seeded_normal(bhnd, s) for s in (101, 102, 103))
    shape = ra.AttentionShape.new(*bhnd)
    got = ra.flash_forward_masked(shape, q, k, v, ra.Mask.causal())
    want = oracle.flash_forward_masked(oracle.AttentionShape(*bhnd), q, k, v, "causal")
    assert_close_nan(got, want, TOL, "cfg f32")
    assert max_abs(got.reshape(bhnd)[0, :, 0], v[0, :, 0]) <= 1e-6  # causal row 0 == V[0]


# ---- gqa_forward_f32 ------------------------------------------------------------------------------------


@pytest.mark.parametrize("b,hq,hkv,sq,skv,d", [(1, 4, 4, 3, 3, 4), (1, 8, 2, 4, 4, 8), (2, 6, 3, 1, 37, 16),
                                              (2, 6, 3, 5, 37, 16), (1, 32, 8, 1, 700, 128), (1, 4, 2, 1, 1, 8),
                                              (2, 8, 2, 130, 130, 64), (1, 3, 1, 2, 9, 200), (1, 8, 2, 100, 333, 64),
                                              (2, 4, 1, 33, 1000, 128), (1, 6, 2, 65, 31, 20), (1, 2, 1, 7, 70, 5)])
def test_gqa_forward_matches_oracle(oracle, b, hq, hkv, sq, skv, d):
    q = seeded_normal((b, hq, sq, d), 1)
    k = seeded_normal((b, hkv, skv, d), 2)
    v = seeded_normal((b, hkv, skv, d), 3)
    out = np.full(b * hq * sq * d, 7.0, dtype=np.float32)
    ra.gqa_forward_f32(q, k, v, out, b, hq, hkv, sq, skv, d)
    want = oracle.gqa_forward_f32(q, k, v, b, hq, hkv, sq, skv, d)
    assert_close_nan(out, want, TOL)
    vv = v.reshape(b, hkv, skv * d)
    o = out.reshape(b, hq, sq * d)
    g = hq // hkv
    for h in range(hq):  # outputs inside [min V, max V] of the mapped kv head (gqa.rs:303-317)
        assert (o[:, h].min(axis=1) >= vv[:, h // g].min(axis=1) - 1e-5).all()
        assert (o[:, h].max(axis=1) <= vv[:, h // g].max(axis=1) + 1e-5).all()


@pytest.mark.parametrize("b,hq,hkv,sq,skv,d", [(2, 8, 2, 130, 130, 64), (1, 8, 2, 100, 333, 64), (1, 6, 2, 65, 31, 20),
                                              (1, 2, 1, 7, 70, 5), (1, 32, 8, 1, 700, 128)])
def test_gqa_device_entry_matches_host_entry(b, hq, hkv, sq, skv, d):
    from _gpu import dev

    q = seeded_normal((b, hq, sq, d), 4)
    k = seeded_normal((b, hkv, skv, d), 5)
    v = seeded_normal((b, hkv, skv, d), 6)
    want = np.zeros(b * hq * sq * d, dtype=np.float32)
    ra.gqa_forward_f32(q, k, v, want, b, hq, hkv, sq, skv, d)
    st = ra.Stream()
    dout = ra.HipStorage.zeros(want.nbytes)
    ra.gqa_forward_f32_dev(dev(q), dev(k), dev(v), dout, b, hq, hkv, sq, skv, d, stream=st)
    st.synchronize()
    assert np.array_equal(dout.download(np.float32), want)
    with pytest.raises(ra.HeadCountMismatch):
        ra.gqa_forward_f32_dev(dout, dout, dout, dout, 1, 5, 2, 1, 1, 4)


def test_gqa_errors():
    z = lambda n: np.zeros(n, dtype=np.float32)
    with pytest.raises(ra.HeadCountMismatch):
        ra.gqa_forward_f32(z(20), z(8), z(8), z(20), 1, 5, 2, 1, 1, 4)
    with pytest.raises(ra.HeadCountMismatch):
        ra.gqa_forward_f32(z(20), z(8), z(8), z(20), 1, 4, 0, 1, 1, 4)
    with pytest.raises(ra.WrongInputLen) as ei:
        ra.gqa_forward_f32(z(7), z(8), z(8), z(16), 1, 4, 2, 1, 1, 4)
    assert (ei.value.which, ei.value.expected, ei.value.got) == ("q", 16, 7)
    with pytest.raises(ra.WrongInputLen) as ei:
        ra.gqa_forward_f32(z(16), z(8), z(8), z(15), 1, 4, 2, 1, 1, 4)
    assert ei.value.which == "out"


def test_host_slice_calls_from_several_threads(oracle):
    """flash_forward is re-entrant in the reference (rayon's global pool, no state of its own).  Here small calls share
    one pinned staging buffer: one call at a time holds it, a concurrent one copies buffer by buffer.  Four threads
    call at once (ctypes releases the interpreter lock during the call) and every result must be its own."""
    import threading

    shapes = [(1, 2, 40, 16), (2, 1, 65, 32), (1, 1, 130, 64), (1, 3, 33, 8)]
    work = []
    for t, bhnd in enumerate(shapes):
        shape = ra.AttentionShape.new(*bhnd)
        bufs = [lcg_buffer(shape.buffer_len(), 100 * t + i, 2.0) for i in range(3)]
        want = oracle.flash_forward_masked(oracle.AttentionShape(*bhnd), *bufs, "causal")
        work.append((shape, bufs, want))
    errors = []

    def run(idx):
        shape, bufs, want = work[idx]
        for _ in range(25):
            got = ra.flash_forward_masked(shape, *bufs, ra.Mask.causal())
            d = max_abs(got, want)
            if not d <= TOL:
                errors.append((idx, d))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(work))]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors[:3]


@pytest.mark.parametrize("n,d,j", [(600, 64, 400), (300, 128, 290), (200, 320, 150)])
@pytest.mark.parametrize("bad", [np.nan, -np.inf])
def test_strict_mode_gives_the_reference_outcome_for_non_finite_v(oracle, n, d, j, bad):
    """rt_set_strict_non_finite_v: the column of a non-finite V element is NaN in every row that does not see its
    key, as in the reference (cpu_forward.rs:268-425); finite elements agree with the oracle as ever."""
    b, h = 2, 2
    q, k, v = (seeded_normal(b * h * n * d, s) for s in (61, 62, 63))
    vbad = v.copy().reshape(b, h, n, d)
    vbad[1, 0, j, 3] = bad
    vbad[0, 1, n - 1, 0] = bad
    shape, osh = ra.AttentionShape.new(b, h, n, d), oracle.AttentionShape(b, h, n, d)
    want = oracle.flash_forward_masked(osh, q, k, vbad.ravel(), "causal").reshape(b, h, n, d)
    assert ra.set_strict_non_finite_v(True) is False
    try:
        got = ra.flash_forward_masked(shape, q, k, vbad.ravel(), ra.Mask.causal()).reshape(b, h, n, d)
    finally:
        assert ra.set_strict_non_finite_v(False) is True
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    assert np.isnan(got[1, 0, :j, 3]).all() and np.isnan(got[0, 1, :n - 1, 0]).all()
    fin = np.isfinite(want)
    assert np.abs(got[fin] - want[fin]).max() <= TOL


@pytest.mark.parametrize("bad", [np.nan, -np.inf])
def test_non_finite_v_row_at_a_causally_hidden_position(oracle, bad):
    """A non-finite V row j under the causal mask.  The reference multiplies the hidden probabilities (exact zeros)
    into V on every key tile, so 0 * NaN poisons every query row; the kernels skip key tiles that lie wholly past a
    query tile.  Rows that see key j are NaN as in the reference; rows at least 256 positions before j are finite
    and equal the result with that V row zeroed; rows in between are NaN or that finite value."""
    b, h, n, d, j = 1, 2, 600, 64, 400
    q, k, v = (seeded_normal(b * h * n * d, s) for s in (61, 62, 63))
    vbad = v.copy().reshape(b, h, n, d)
    vbad[:, :, j, 3] = bad
    vzero = v.copy().reshape(b, h, n, d)
    vzero[:, :, j, :] = 0.0
    shape, osh = ra.AttentionShape.new(b, h, n, d), oracle.AttentionShape(b, h, n, d)
    want_ref = oracle.flash_forward_masked(osh, q, k, vbad.ravel(), "causal").reshape(b, h, n, d)
    assert (~np.isfinite(want_ref[..., 3])).all()
    got = ra.flash_forward_masked(shape, q, k, vbad.ravel(), ra.Mask.causal()).reshape(b, h, n, d)
    clean = oracle.flash_forward_masked(osh, q, k, vzero.ravel(), "causal").reshape(b, h, n, d)
    assert (~np.isfinite(got[:, :, j:, 3])).all()  # NaN, or +-Inf where the row's weight on key j is positive
    early = got[:, :, :j - 255]
    assert np.isfinite(early).all() and max_abs(early, clean[:, :, :j - 255]) <= TOL
    mid = got[:, :, j - 255:j]
    with np.errstate(invalid="ignore"):
        assert (~np.isfinite(mid) | (np.abs(mid - clean[:, :, j - 255:j]) <= TOL)).all()
