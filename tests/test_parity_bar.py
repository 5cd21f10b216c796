"""The comparison rule of the bf16 parity checks (oracle.rel_fro_blocks beside max-abs <= 2e-2), exercised on the
CPU: a kernel that is correct up to bf16 rounding passes both bars at a long sequence, one that loses a 32-key
item for the last 256 query rows passes the absolute bar alone and fails the relative one."""
import numpy as np


def _round(oracle, x):
    return oracle.bf16_to_f32(oracle.f32_to_bf16(np.asarray(x, dtype=np.float32).ravel())).reshape(np.shape(x))


def test_relative_bar_sees_a_dropped_key_item_the_absolute_bar_misses(oracle):
    n, d = 4096, 128
    rng = np.random.default_rng(0)
    q, k, v = (_round(oracle, rng.standard_normal(n * d, dtype=np.float32)) for _ in range(3))
    want = oracle.flash_forward_masked(oracle.AttentionShape(1, 1, n, d), q, k, v, "causal").reshape(n, d)
    good = _round(oracle, want)
    assert np.abs(good - want).max() <= oracle.BF16_MAX_ABS
    assert oracle.rel_fro_blocks(good, want, d, n) <= oracle.BF16_REL_FRO / 3
    # the last 256 rows without keys 1000..1031
    q64 = q.reshape(n, d)[-256:].astype(np.float64)
    s = q64 @ k.reshape(n, d).astype(np.float64).T / np.sqrt(d)
    s = np.where(np.arange(n)[None] > np.arange(n - 256, n)[:, None], -np.inf, s)
    s[:, 1000:1032] = -np.inf
    p = np.exp(s - s.max(axis=1, keepdims=True))
    bad = want.copy()
    bad[-256:] = (p / p.sum(axis=1, keepdims=True)) @ v.reshape(n, d).astype(np.float64)
    assert np.abs(bad - want).max() <= oracle.BF16_MAX_ABS          # the absolute bar does not see it
    assert oracle.rel_fro_blocks(bad, want, d, n) > 5 * oracle.BF16_REL_FRO


def test_relative_bar_edge_cases(oracle):
    f = oracle.rel_fro_blocks
    z = np.zeros((4, 300, 8), dtype=np.float32)
    assert f(z, z, 8, 300) == 0.0                                   # all-zero blocks reproduced exactly
    w = z.copy()
    w[1, 299, 3] = 1e-6
    assert f(w, z, 8, 300) == np.inf                                # a zero block that is not reproduced
    a = np.ones((2, 256, 8), dtype=np.float32)
    b = a.copy()
    b[1] *= 1.5
    assert abs(f(b, a, 8, 256) - 0.5) < 1e-12                       # the worst block, not the average
    n1 = a.copy()
    n1[0, 0, :] = np.nan
    assert f(n1, n1, 8, 256) == 0.0                                 # NaN in want is left out
    assert f(a, n1, 8, 256) == 0.0
    i1, i2 = a.copy(), a.copy()
    i1[0, 0, 0] = i2[0, 0, 0] = np.inf
    assert f(i1, i2, 8, 256) == 0.0                                 # equal infinities agree
    assert f(a, i2, 8, 256) == np.inf
    assert f(np.zeros(0), np.zeros(0), 8) == 0.0
    # fewer than min_elems per block: one block for the array; decode rows: one block per row
    small = np.ones((3, 2, 8), dtype=np.float32)
    off = small.copy()
    off[0, 0, 0] = 2.0
    assert abs(f(off, small, 8, 2) - np.sqrt(1.0 / 48.0)) < 1e-12
    rows = np.ones((5, 64), dtype=np.float32)
    r2 = rows.copy()
    r2[3] *= 1.25
    assert abs(f(r2, rows, 64, block_rows=1, min_elems=64) - 0.25) < 1e-12
