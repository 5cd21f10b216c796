"""GPU parity of the bf16 prefill kernels through the C ABI (rt_flash_forward_bf16_dev,
rt_flash_forward_varlen_bf16_dev) against the CPU oracle run in f32 on the same bf16-rounded
inputs.  Bar: max-abs <= 2e-2 and, per block of 256 query rows of a (b,h) slab, relative Frobenius error <= 1e-2;
NaN and zero-row patterns exact."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_bf16_parity, bf16_round, dev, flash_bf16, max_abs
from _util import seeded_normal

pytestmark = pytest.mark.gpu
TOL = 2e-2


def inputs(shape_q, shape_kv, seeds=(1, 2, 3), q_mul=1.0):
    q = seeded_normal(shape_q, seeds[0]) * np.float32(q_mul)
    k = seeded_normal(shape_kv, seeds[1])
    v = seeded_normal(shape_kv, seeds[2])
    return bf16_round(q), bf16_round(k), bf16_round(v)


# (kernel forced through rt_debug_force_bf16_prefill_kernel, head dim): the persistent 8-wave kernel covers 64 and 128, the
# 4-wave tile kernel every multiple of 8 up to 256 (zero-padded to 32 / 64 / 96 / 128 / 256 in LDS)
KERNEL_DIMS = [("persistent", 64), ("persistent", 128), ("tile", 32), ("tile", 64), ("tile", 80), ("tile", 96),
               ("tile", 128), ("tile", 8), ("tile", 200), ("tile", 256), ("wide", 64)]


@pytest.fixture
def force_kernel():
    yield ra.debug_force_bf16_prefill_kernel
    ra.debug_force_bf16_prefill_kernel("auto")


@pytest.mark.parametrize("kernel,d", KERNEL_DIMS)
@pytest.mark.parametrize("n", [1, 2, 31, 63, 64, 65, 127, 128, 129, 200, 513])
def test_flash_bf16_matches_oracle(oracle, force_kernel, n, kernel, d):
    force_kernel(kernel)
    b, h = 2, 3
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (n, n + 1, n + 2))
    shape = ra.AttentionShape.new(b, h, n, d)
    rng = np.random.default_rng(n)
    keep = rng.random(n) < 0.7
    keep[0] = True
    for mask, om in ((ra.Mask.none(), None), (ra.Mask.causal(), "causal"), (ra.Mask.padding(keep), ("padding", keep))):
        got = flash_bf16(shape, qb, kb, vb, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), qf, kf, vf, om)
        assert_bf16_parity(got, want, d, n, f"n={n} d={d} mask={mask.kind} kernel={kernel}")


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("n", [300, 2048 + 77])
def test_both_prefill_kernels_agree(oracle, force_kernel, n, d):
    """The two kernels behind rt_flash_forward_bf16_dev on one input: each within the bar of the oracle, and of
    each other (they round P to bf16 at the same point, so they differ by accumulation order only)."""
    b, h = 1, 8
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (71, 72, 73))
    shape = ra.AttentionShape.new(b, h, n, d)
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), qf, kf, vf, "causal")
    outs = {}
    for kernel in ("persistent", "tile"):
        force_kernel(kernel)
        outs[kernel] = flash_bf16(shape, qb, kb, vb, ra.Mask.causal())
        assert_bf16_parity(outs[kernel], want, d, n, kernel)
    assert max_abs(outs["persistent"], outs["tile"]) <= TOL


@pytest.mark.parametrize("kernel,d", [("persistent", 64), ("persistent", 128), ("tile", 64), ("tile", 128), ("wide", 64)])
def test_row_max_that_keeps_rising_along_the_keys(oracle, force_kernel, kernel, d):
    """Scores that grow with the key index: a ramp that lifts the row max by tens of units from one 32-key item to
    the next, one key hundreds of units above everything before it (an exponential taken against the old max
    overflows f32), then keys far below the max.  Whatever rule a kernel uses to decide when to raise its running
    max, the result is the plain softmax of the oracle."""
    force_kernel(kernel)
    b, h, n = 1, 2, 700
    rng = np.random.default_rng(5)
    u = np.full(d, 1.0 / np.sqrt(d), dtype=np.float32) * np.float32(d ** 0.25)  # (a u).(b u) / sqrt(d) = a b
    a_row = rng.uniform(1.0, 3.0, size=(b, h, n, 1)).astype(np.float32)
    prof = np.concatenate([np.linspace(-50.0, 50.0, 400), np.full(50, 20.0), [400.0], np.full(149, 100.0),
                           np.full(100, -300.0)]).astype(np.float32)
    assert prof.size == n
    q = a_row * u + 0.3 * rng.standard_normal((b, h, n, d), dtype=np.float32)
    k = prof[None, None, :, None] * u + 0.3 * rng.standard_normal((b, h, n, d), dtype=np.float32)
    v = rng.standard_normal((b, h, n, d), dtype=np.float32)
    (qb, qf), (kb, kf), (vb, vf) = bf16_round(q), bf16_round(k), bf16_round(v)
    shape = ra.AttentionShape.new(b, h, n, d)
    for mask, om in ((ra.Mask.causal(), "causal"), (ra.Mask.none(), None)):
        got = flash_bf16(shape, qb, kb, vb, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), qf, kf, vf, om)
        assert np.isfinite(want).all()
        assert_bf16_parity(got, want, d, n, f"kernel={kernel} d={d} mask={mask.kind}")


def test_flash_bf16_closed_forms():
    """N=1 => out == v exactly; causal row 0 == V[0] exactly; constant V => constant output."""
    d = 128
    (qb, qf), (kb, kf), (vb, vf) = inputs((1, 2, 1, d), (1, 2, 1, d))
    assert np.array_equal(flash_bf16(ra.AttentionShape.new(1, 2, 1, d), qb, kb, vb), vf)
    n = 300
    (qb, qf), (kb, kf), (vb, vf) = inputs((1, 2, n, d), (1, 2, n, d))
    out = flash_bf16(ra.AttentionShape.new(1, 2, n, d), qb, kb, vb, ra.Mask.causal()).reshape(1, 2, n, d)
    assert np.array_equal(out[0, :, 0], vf.reshape(1, 2, n, d)[0, :, 0])
    const = np.tile(np.linspace(-2, 2, d, dtype=np.float32), (1, 2, n, 1))
    cb, cf = bf16_round(const)
    out = flash_bf16(ra.AttentionShape.new(1, 2, n, d), qb, kb, cb, ra.Mask.causal())
    assert max_abs(out, cf) <= 2 ** -7 * 2.0  # weights sum to 1 up to P's bf16 rounding


@pytest.mark.parametrize("mask", ["causal", "none"])
def test_long_head_dim_64_is_served_by_the_tile_kernel_and_the_64_rows_per_wave_kernel_agrees(oracle, mask):
    """B=4, H=32, N=2048, D=64: with nothing forced the library takes the tile kernel here (the same bits as the
    forced tile kernel); the kernel with 64 query rows per wave, which runs when asked for, rounds the same f32 sums.
    Every row of eight (batch, head) slabs of either against the oracle."""
    b, h, n, d = 4, 32, 2048, 64
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (91, 92, 93))
    shape = ra.AttentionShape.new(b, h, n, d)
    m = ra.Mask.causal() if mask == "causal" else ra.Mask.none()
    ra.debug_force_bf16_prefill_kernel("auto")
    got = flash_bf16(shape, qb, kb, vb, m).reshape(b * h, n, d)
    try:
        ra.debug_force_bf16_prefill_kernel("tile")
        tile = flash_bf16(shape, qb, kb, vb, m).reshape(b * h, n, d)
        ra.debug_force_bf16_prefill_kernel("wide")
        wide = flash_bf16(shape, qb, kb, vb, m).reshape(b * h, n, d)
    finally:
        ra.debug_force_bf16_prefill_kernel("auto")
    assert np.array_equal(got, tile, equal_nan=True)
    assert max_abs(wide, tile) <= 2 ** -7 * 4.0  # a bf16 ulp or two of values below 4
    q3, k3, v3 = (x.reshape(b * h, n * d) for x in (qf, kf, vf))
    for slab in (0, 1, 31, 64, 77, 100, 126, 127):
        want = oracle.flash_forward_masked(oracle.AttentionShape(1, 1, n, d), q3[slab], k3[slab], v3[slab],
                                           "causal" if mask == "causal" else None).reshape(n, d)
        assert_bf16_parity(got[slab], want, d, n, f"slab {slab}")
        assert_bf16_parity(wide[slab], want, d, n, f"slab {slab}, 64 rows per wave")


@pytest.mark.parametrize("kernel", ["persistent", "tile", "wide"])
def test_flash_bf16_masks_nan_rules(oracle, force_kernel, kernel):
    force_kernel(kernel)
    b, h, n, d = 1, 2, 150, 64
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d))
    shape = ra.AttentionShape.new(b, h, n, d)
    osh = oracle.AttentionShape(b, h, n, d)
    for keep in (np.zeros(n, bool), np.r_[np.zeros(64, bool), np.ones(n - 64, bool)],
                 np.r_[np.zeros(63, bool), np.ones(n - 63, bool)], np.r_[np.ones(64, bool), np.zeros(n - 64, bool)]):
        got = flash_bf16(shape, qb, kb, vb, ra.Mask.padding(keep))
        want = oracle.flash_forward_masked(osh, qf, kf, vf, ("padding", keep))
        assert_bf16_parity(got, want, d, n)
    # NaN in a query row poisons that row only; NaN in a key row poisons the rows that see it
    qn = qf.copy()
    qn[5 * d + 3] = np.nan
    kn = kf.copy()
    kn[100 * d + 7] = np.nan
    for mask, om in ((ra.Mask.causal(), "causal"), (ra.Mask.none(), None)):
        got = flash_bf16(shape, oracle.f32_to_bf16(qn), oracle.f32_to_bf16(kn), vb, mask)
        want = oracle.flash_forward_masked(osh, qn, kn, vf, om)
        assert_bf16_parity(got, want, d, n)


@pytest.mark.parametrize("kernel,d", [("persistent", 128), ("tile", 128), ("wide", 64)])
@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 1), (6, 6)])
def test_flash_bf16_gqa_head_mapping(oracle, force_kernel, kernel, d, hq, hkv):
    """kv head = h / (Hq/Hkv): equals the oracle on explicitly replicated K/V (gqa.rs:151-177)."""
    force_kernel(kernel)
    b, n = 2, 130
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, hq, n, d), (b, hkv, n, d))
    got = flash_bf16(ra.AttentionShape.new(b, hq, n, d), qb, kb, vb, ra.Mask.causal(), n_kv_heads=hkv)
    g = hq // hkv
    kr = np.repeat(kf.reshape(b, hkv, n, d), g, axis=1)
    vr = np.repeat(vf.reshape(b, hkv, n, d), g, axis=1)
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, hq, n, d), qf, kr, vr, "causal")
    assert_bf16_parity(got, want, d, n)


def run_varlen(shape, qb, kb, vb, lens, zero=True):
    dq, dk, dv = dev(qb), dev(kb), dev(vb)
    dl = dev(np.asarray(lens, dtype=np.int32))
    n_out = shape.buffer_len()
    dout = ra.HipStorage(n_out * 2)
    dout.upload(np.full(n_out, 0x7B7B, dtype=np.uint16))
    ra.flash_forward_varlen_bf16_dev(shape, dq, dk, dv, dl, dout, zero_padded_rows=zero)
    ra.synchronize()
    from oracle import attn_oracle
    return attn_oracle.bf16_to_f32(dout.download(np.uint16, n_out))


@pytest.mark.parametrize("kernel,d", [("persistent", 64), ("tile", 64), ("tile", 96), ("persistent", 128), ("wide", 64)])
def test_varlen_small(oracle, force_kernel, kernel, d):
    force_kernel(kernel)
    b, h, n = 4, 2, 200
    lens = [200, 1, 129, 0]
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d))
    shape = ra.AttentionShape.new(b, h, n, d)
    for zero in (True, False):
        got = run_varlen(shape, qb, kb, vb, lens, zero)
        want = oracle.varlen_causal_forward(qf, kf, vf, lens, b, h, n, d, zero_padded_rows=zero)
        assert_bf16_parity(got, want, d, n)
        if zero:
            g = got.reshape(b, h, n, d)
            for i, L in enumerate(lens):
                assert (g[i, :, L:] == 0.0).all() and not np.signbit(g[i, :, L:]).any()


@pytest.mark.parametrize("d", [32, 64, 128])
def test_rows_behind_a_short_sequence_may_hold_anything(oracle, force_kernel, d):
    """Sequences shorter than one key tile in a padded batch whose K and V rows behind each sequence's last key hold NaN
    and infinities: the first key tile is requested before the lengths are known, so those rows do arrive in the
    workgroup; nothing of them may reach a valid row (V rows behind the last key count as zeros, their scores are
    masked), and the padded rows are zeros."""
    force_kernel("tile")
    b, h, n = 5, 2, 100
    lens = [1, 5, 63, 64, 65]
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (81, 82, 83))
    k4, v4 = kf.copy().reshape(b, h, n, d), vf.copy().reshape(b, h, n, d)
    for i, L in enumerate(lens):
        k4[i, :, L:] = np.nan
        v4[i, :, L:] = np.inf
        v4[i, :, L:, ::3] = np.nan
    shape = ra.AttentionShape.new(b, h, n, d)
    got = run_varlen(shape, qb, oracle.f32_to_bf16(k4.ravel()), oracle.f32_to_bf16(v4.ravel()), lens, True)
    want = oracle.varlen_causal_forward(qf, kf, vf, lens, b, h, n, d, zero_padded_rows=True)
    assert np.isfinite(got).all()
    assert_bf16_parity(got, want, d, n)
    g = got.reshape(b, h, n, d)
    for i, L in enumerate(lens):
        assert (g[i, :, L:] == 0.0).all()


def test_strict_mode_on_a_padded_batch(oracle, strict_v):
    """The strict pass takes each sequence's own length: a non-finite V element inside a sequence reaches the rows
    before its key, one in the padding behind a sequence reaches nothing."""
    b, h, n, d = 3, 2, 400, 64
    lens = [400, 130, 257]
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (71, 72, 73))
    v4 = vf.copy().reshape(b, h, n, d)
    v4[0, 1, 399, 7] = np.inf
    v4[1, 0, 129, 0] = np.nan
    v4[1, 1, 131, 3] = np.nan   # behind the 130 keys of sequence 1
    v4[2, 0, 5, 9] = -np.inf
    shape = ra.AttentionShape.new(b, h, n, d)
    strict_v(True)
    got = run_varlen(shape, qb, kb, oracle.f32_to_bf16(v4.ravel()), lens, True).reshape(b, h, n, d)
    want = oracle.varlen_causal_forward(qf, kf, v4.ravel(), lens, b, h, n, d, zero_padded_rows=True).reshape(b, h, n, d)
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    assert np.isnan(got[0, 1, :399, 7]).all() and np.isnan(got[1, 0, :129, 0]).all() and np.isnan(got[2, 0, :5, 9]).all()
    assert np.isfinite(got[1, 1]).all() and (got[1, :, 130:] == 0.0).all()
    fin = np.isfinite(want)
    assert np.abs(got[fin] - want[fin]).max() <= TOL


@pytest.mark.parametrize("kernel", ["auto", "persistent", "tile", "wide"])
def test_config_padded_batch_b16_h16_n1024_d64(oracle, force_kernel, kernel):
    """The variable-length workload of the benchmark set: lengths uniform in [128, 1024] from a seed, key padding + causal,
    padded query rows exactly 0."""
    force_kernel(kernel)
    b, h, n, d = 16, 16, 1024, 64
    lens = np.random.default_rng(2026).integers(128, 1025, size=b).astype(np.int32)
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (21, 22, 23))
    got = run_varlen(ra.AttentionShape.new(b, h, n, d), qb, kb, vb, lens)
    want = oracle.varlen_causal_forward(qf, kf, vf, lens, b, h, n, d)
    assert_bf16_parity(got, want, d, n, f"lens={lens.tolist()}")
    g = got.reshape(b, h, n, d)
    for i, L in enumerate(lens):
        assert (g[i, :, L:] == 0.0).all()


def test_config_prefill_b4_h32_n4096_d128(oracle):
    """The headline prefill workload at full size.  The oracle (which computes every tile, as the reference
    does) checks a sample of (b,h) slabs in full; size-independent properties cover all slabs:
    causal row 0 == V[0] exactly, and a second run with V := const gives const."""
    b, h, n, d = 4, 32, 4096, 128
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (31, 32, 33))
    shape = ra.AttentionShape.new(b, h, n, d)
    got = flash_bf16(shape, qb, kb, vb, ra.Mask.causal()).reshape(b, h, n, d)
    assert np.isfinite(got).all()
    v4 = vf.reshape(b, h, n, d)
    assert np.array_equal(got[:, :, 0], v4[:, :, 0])
    q4, k4 = qf.reshape(b, h, n, d), kf.reshape(b, h, n, d)
    worst = 0.0
    for (bi, hi) in ((0, 0), (1, 13), (3, 31)):
        want = oracle.flash_forward_masked(oracle.AttentionShape(1, 1, n, d), q4[bi, hi], k4[bi, hi], v4[bi, hi],
                                           "causal").reshape(n, d)
        worst = max(worst, max_abs(got[bi, hi], want))
        assert_bf16_parity(got[bi, hi], want, d, n, f"slab ({bi},{hi})")
    assert worst <= TOL, worst
    # rows are convex combinations of V rows
    assert (got.max(axis=2) <= v4.max(axis=2) + 1e-2).all() and (got.min(axis=2) >= v4.min(axis=2) - 1e-2).all()


def test_config_long_context_b1_h32_n16384_d128(oracle):
    """The large-logit workload of the benchmark set: Q scaled by 2.0 before rounding.  Checked against the oracle on the
    first 2048 rows of two heads (causal rows depend only on their prefix, so the truncated problem
    is the same computation) and on sampled late rows through the reference's single-row decode
    function (row i of causal attention == unmasked attention of q_i over keys [0, i])."""
    b, h, n, d = 1, 32, 16384, 128
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (41, 42, 43), q_mul=2.0)
    shape = ra.AttentionShape.new(b, h, n, d)
    got = flash_bf16(shape, qb, kb, vb, ra.Mask.causal()).reshape(h, n, d)
    assert np.isfinite(got).all()
    q4, k4, v4 = qf.reshape(h, n, d), kf.reshape(h, n, d), vf.reshape(h, n, d)
    assert np.array_equal(got[:, 0], v4[:, 0])
    for hi in (0, 17):
        m = 2048
        want = oracle.flash_forward_masked(oracle.AttentionShape(1, 1, m, d), q4[hi, :m], k4[hi, :m], v4[hi, :m],
                                           "causal").reshape(m, d)
        assert_bf16_parity(got[hi, :m], want, d, m, f"head {hi}, first {m} rows")
    rng = np.random.default_rng(5)
    for hi in (3, 31):
        # whole 256-row blocks late in the sequence, each row through the single-row function (a key item lost
        # there moves the block's relative error to ~0.1 and its max-abs by less than the absolute bar)
        for r0 in (n - 256, 9 * 1024 + 512):
            want = np.stack([oracle.gqa_forward_f32(q4[hi, i], k4[hi, :i + 1], v4[hi, :i + 1], 1, 1, 1, 1, i + 1, d)
                             for i in range(r0, r0 + 256)])
            assert_bf16_parity(got[hi, r0:r0 + 256], want, d, 256, f"head {hi}, rows {r0}..{r0 + 255}")
        for i in rng.integers(2048, n, size=5).tolist():
            want = oracle.gqa_forward_f32(q4[hi, i], k4[hi, :i + 1], v4[hi, :i + 1], 1, 1, 1, 1, i + 1, d)
            assert_bf16_parity(got[hi, i], want, d, 1, f"head {hi}, row {i}")


@pytest.mark.parametrize("d", [4, 100, 257, 264, 320, 12])
@pytest.mark.parametrize("n", [1, 33, 130])
def test_head_dims_outside_the_matrix_core_kernels(oracle, n, d):
    """Head dims above 256, or not a multiple of 8 (rows are then not 16-byte aligned): a workgroup per query row, the
    same masks and row rules (the reference takes any dim != 0, cpu_forward.rs:142-169)."""
    b, h = 2, 3
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (n, n + 1, n + 2))
    shape = ra.AttentionShape.new(b, h, n, d)
    keep = np.random.default_rng(n).random(n) < 0.7
    keep[0] = True
    for mask, om in ((ra.Mask.none(), None), (ra.Mask.causal(), "causal"), (ra.Mask.padding(keep), ("padding", keep)),
                     (ra.Mask.padding(np.zeros(n, bool)), ("padding", np.zeros(n, bool)))):
        got = flash_bf16(shape, qb, kb, vb, mask)
        want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), qf, kf, vf, om)
        assert_bf16_parity(got, want, d, n, f"n={n} d={d} mask={mask.kind}")
    lens = [n, n // 2]
    for zero in (True, False):
        got = run_varlen(shape, qb, kb, vb, lens, zero)
        want = oracle.varlen_causal_forward(qf, kf, vf, lens, b, h, n, d, zero_padded_rows=zero)
        assert_bf16_parity(got, want, d, n, f"varlen n={n} d={d}")


def test_head_dim_above_512_is_an_error():
    shape = ra.AttentionShape.new(1, 1, 8, 520)
    z = dev(np.zeros(8 * 520, dtype=np.uint16))
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_forward_bf16_dev(shape, z, z, z, z)
    assert ei.value.status == 21 and ei.value.expected == 512


@pytest.fixture
def strict_v():
    yield ra.set_strict_non_finite_v
    ra.set_strict_non_finite_v(False)


@pytest.mark.parametrize("kernel,n,d,j", [("persistent", 1024, 128, 700), ("tile", 1024, 128, 700), ("tile", 777, 64, 500),
                                          ("tile", 300, 100, 299), ("wide", 777, 64, 500)])
@pytest.mark.parametrize("bad", [np.nan, -np.inf])
def test_strict_mode_gives_the_reference_outcome_for_non_finite_v(oracle, force_kernel, strict_v, kernel, n, d, j, bad):
    """With rt_set_strict_non_finite_v on, a non-finite V element at key j makes that column NaN in every row that
    does not see key j, as the reference's walk over every key tile does (cpu_forward.rs:268-425); rows that see it
    are non-finite as before, and every other column equals the oracle's."""
    force_kernel(kernel)
    assert strict_v(True) is False
    b, hq, hkv = 2, 4, 2
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, hq, n, d), (b, hkv, n, d), (51, 52, 53))
    vbad = vf.copy().reshape(b, hkv, n, d)
    vbad[1, 0, j, 5] = bad
    vbad[0, 1, j // 2, 2] = bad
    vbad = vbad.ravel()
    shape = ra.AttentionShape.new(b, hq, n, d)
    got = flash_bf16(shape, qb, kb, oracle.f32_to_bf16(vbad), ra.Mask.causal(), n_kv_heads=hkv).reshape(b, hq, n, d)
    g = hq // hkv
    k4, v4 = kf.reshape(b, hkv, n, d), vbad.reshape(b, hkv, n, d)
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, hq, n, d), qf, np.repeat(k4, g, axis=1).ravel(),
                                       np.repeat(v4, g, axis=1).ravel(), "causal").reshape(b, hq, n, d)
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    assert np.isnan(got[1, 0:g, :j, 5]).all() and np.isnan(got[0, g:2 * g, :j // 2, 2]).all()
    fin = np.isfinite(want)
    assert np.abs(got[fin] - want[fin]).max() <= TOL
    assert strict_v(False) is True


@pytest.mark.parametrize("kernel", ["persistent", "tile"])
@pytest.mark.parametrize("bad", [np.nan, np.inf])
def test_non_finite_v_row_at_a_causally_hidden_position(oracle, force_kernel, kernel, bad):
    """A non-finite V row j under the causal mask.  The reference walks every key tile and multiplies the hidden
    probabilities (exact zeros) into V, so 0 * NaN (or 0 * Inf) makes EVERY query row non-finite in that column (cpu_forward.rs:268-425: no tile is
    skipped).  The kernels skip key tiles that lie wholly past a query tile and never read those V rows: rows that
    see key j (i >= j) are NaN as in the reference; rows at least 256 positions before j are finite and equal the
    result with that V row replaced by zeros; rows in between are NaN or that finite value."""
    force_kernel(kernel)
    b, h, n, d, j = 1, 2, 1024, 128, 700
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (51, 52, 53))
    vbad = vf.copy().reshape(b, h, n, d)
    vbad[:, :, j, 5] = bad
    vbad = vbad.ravel()
    vzero = vf.copy().reshape(b, h, n, d)
    vzero[:, :, j, :] = 0.0
    vzero = vzero.ravel()
    shape, osh = ra.AttentionShape.new(b, h, n, d), oracle.AttentionShape(b, h, n, d)
    want_ref = oracle.flash_forward_masked(osh, qf, kf, vbad, "causal").reshape(b, h, n, d)
    assert (~np.isfinite(want_ref[..., 5])).all()  # the reference: every row, hidden or not
    got = flash_bf16(shape, qb, kb, oracle.f32_to_bf16(vbad), ra.Mask.causal()).reshape(b, h, n, d)
    clean = oracle.flash_forward_masked(osh, qf, kf, vzero, "causal").reshape(b, h, n, d)
    assert (~np.isfinite(got[:, :, j:, 5])).all()  # NaN, or +-Inf where the row's weight on key j is positive
    early = got[:, :, :j - 255]
    assert np.isfinite(early).all() and max_abs(early, clean[:, :, :j - 255]) <= TOL
    mid = got[:, :, j - 255:j]
    with np.errstate(invalid="ignore"):
        ok = ~np.isfinite(mid) | (np.abs(mid - clean[:, :, j - 255:j]) <= TOL)
    assert ok.all()
    # the other columns of the poisoned rows stay finite in both (only column 5 of V is bad)
    assert np.isfinite(got[..., :5]).all() and np.isfinite(want_ref[..., :5]).all()


@pytest.mark.parametrize("kernel", ["persistent", "tile", "wide"])
@pytest.mark.parametrize("mask", ["none", "padding"])
@pytest.mark.parametrize("n,d", [(200, 128), (100, 128), (200, 64), (40, 64), (330, 96)])
def test_infinite_last_v_row_with_a_ragged_last_key_tile(oracle, force_kernel, kernel, mask, n, d):
    """+Inf in the last key's V row, sequence lengths that end inside a key tile.  Every row that weighs that key
    gets +Inf in that column, as in the reference (cpu_forward.rs:268-425); the key slots behind the last key carry
    weight zero and must not turn the column into NaN (0 * Inf), whichever tile the last key falls in."""
    force_kernel(kernel)
    b, h = 2, 2
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (61, 62, 63))
    vbad = vf.copy().reshape(b, h, n, d)
    vbad[:, :, n - 1, 5] = np.inf
    vbad = vbad.ravel()
    shape, osh = ra.AttentionShape.new(b, h, n, d), oracle.AttentionShape(b, h, n, d)
    if mask == "padding":
        keep = np.ones(n, dtype=bool)
        keep[3] = keep[n // 2] = False
        want = oracle.flash_forward_masked(osh, qf, kf, vbad, ("padding", keep)).reshape(b, h, n, d)
        got = flash_bf16(shape, qb, kb, oracle.f32_to_bf16(vbad), ra.Mask.padding(keep)).reshape(b, h, n, d)
    else:
        want = oracle.flash_forward_masked(osh, qf, kf, vbad, None).reshape(b, h, n, d)
        got = flash_bf16(shape, qb, kb, oracle.f32_to_bf16(vbad)).reshape(b, h, n, d)
    assert np.isposinf(want[..., 5]).all()
    assert np.isposinf(got[..., 5]).all()
    rest = np.ones(d, dtype=bool)
    rest[5] = False
    assert np.isfinite(got[..., rest]).all() and max_abs(got[..., rest], want[..., rest]) <= TOL


@pytest.mark.parametrize("kernel,d", [("persistent", 64), ("persistent", 128), ("tile", 64), ("tile", 128), ("tile", 96),
                                      ("wide", 64)])
def test_two_launches_give_the_same_bits(force_kernel, kernel, d):
    """No atomics, no order that depends on timing: the same inputs give the same output bits on every launch.
    (A vector instruction that reads a matrix result too early, for one, shows up here as last-bit differences.)"""
    force_kernel(kernel)
    b, h, n = 1, 2, 300
    (qb, _), (kb, _), (vb, _) = inputs((b, h, n, d), (b, h, n, d), (81, 82, 83))
    shape = ra.AttentionShape.new(b, h, n, d)
    dq, dk, dv = dev(qb), dev(kb), dev(vb)
    for mask in (ra.Mask.none(), ra.Mask.causal()):
        outs = []
        for _ in range(4):
            dout = ra.HipStorage(qb.size * 2)
            ra.flash_forward_bf16_dev(shape, dq, dk, dv, dout, mask)
            ra.synchronize()
            outs.append(dout.download(np.uint16))
        assert all(np.array_equal(outs[0], o) for o in outs[1:])


def test_padding_mask_longer_than_the_persistent_kernel_holds(oracle):
    """A key-padding vector of more than 65536 keys: the persistent kernel keeps the mask as bits in LDS and stops
    there, so the call goes to the tile kernel whatever the head dim.  Sampled rows are checked through the reference's
    single-row attention over the kept keys (a padding mask hides the same keys from every query)."""
    b, h, n, d = 1, 1, 66000, 64
    (qb, qf), (kb, kf), (vb, vf) = inputs((b, h, n, d), (b, h, n, d), (91, 92, 93))
    keep = np.ones(n, bool)
    keep[500:40000] = False
    keep[65990:] = False
    got = flash_bf16(ra.AttentionShape.new(b, h, n, d), qb, kb, vb, ra.Mask.padding(keep)).reshape(n, d)
    assert np.isfinite(got).all()
    k2, v2 = kf.reshape(n, d)[keep], vf.reshape(n, d)[keep]
    q2 = qf.reshape(n, d)
    for i in (0, 1, 499, 500, 39999, 40000, 65535, 65536, 65999):
        want = oracle.gqa_forward_f32(q2[i], k2, v2, 1, 1, 1, 1, k2.shape[0], d)
        assert_bf16_parity(got[i], want, d, 1, f"row {i}")
