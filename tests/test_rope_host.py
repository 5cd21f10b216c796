"""The host mirror of RoPE (rustorch_amd/rope.py) against the oracle: tables, both conventions, the reference's
error values (crates/rustorch-nn/src/rope.rs:245-329)."""
import numpy as np
import pytest

import rustorch_amd as ra


@pytest.mark.parametrize("d,n,base", [(4, 8, 10000.0), (64, 512, 10000.0), (128, 1024, 500000.0)])
def test_tables_match_oracle_to_an_ulp(oracle, d, n, base):
    a, b = ra.RoPE(d, n, base), oracle.RoPE(d, n, base)
    assert np.abs(a.cos - b.cos).max() <= 2 ** -23 and np.abs(a.sin - b.sin).max() <= 2 ** -23
    assert (a.cos != b.cos).mean() < 0.05 and (a.sin != b.sin).mean() < 0.05


@pytest.mark.parametrize("name,oname", [("apply_inplace_half_split", "apply_half_split"),
                                        ("apply_inplace", "apply_interleaved")])
def test_apply_matches_oracle(oracle, name, oname):
    rng = np.random.default_rng(2)
    b, h, s, d, off = 2, 3, 5, 16, 7
    host, ref = ra.RoPE(d, 32), oracle.RoPE(d, 32)
    host.cos, host.sin = ref.cos.copy(), ref.sin.copy()  # same tables: the arithmetic itself must agree exactly
    x = rng.standard_normal(b * h * s * d).astype(np.float32)
    y = x.copy()
    getattr(host, name)(y, b, h, s, off)
    assert np.array_equal(y, getattr(ref, oname)(x, b, h, s, off))


def test_errors_follow_the_reference():
    rope = ra.RoPE(4, 4)
    with pytest.raises(ra.PositionOverflow) as e:
        rope.apply_inplace(np.zeros(8, dtype=np.float32), 1, 1, 2, 3)
    assert (e.value.max_seq, e.value.requested) == (4, 5)
    with pytest.raises(ra.RopeWrongInputLen) as e:
        rope.apply_inplace_half_split(np.zeros(7, dtype=np.float32), 1, 1, 2, 0)
    assert (e.value.expected, e.value.got) == (8, 7)
    with pytest.raises(ValueError):
        ra.RoPE(5, 4)
    x = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    y = x.copy()
    ra.RoPE(4, 8).apply_inplace(y, 1, 1, 1, 0)
    assert np.abs(y - x).max() < 1e-6  # position 0 is the identity (rope.rs:247-256)


def test_multi_head_attention_routing_rule():
    """The branch MultiHeadAttention::forward takes (crates/rustorch-nn/src/attention.rs:325-333, :347-356)."""
    import rustorch_amd as ra
    assert ra.mha_attention_route(1, 1, False) == "identity"
    assert ra.mha_attention_route(1, 1, True) == "composed"
    assert ra.mha_attention_route(128, 128, False) == "flash"
    assert ra.mha_attention_route(128, 128, True) == "composed"
    assert ra.mha_attention_route(1, 64, False) == "composed"
    v = np.arange(2 * 3 * 4, dtype=np.float32)
    out = ra.mha_attention_f32(v, v, v, 2, 1, 1, 3, 4)  # the identity route needs no device
    assert np.array_equal(out, v) and out is not v
