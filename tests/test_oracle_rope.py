"""Pins the oracle's RoPE tables, the two rotation conventions, the per-head RMSNorm and the decode
preparation step.  Reference tests restated: rope.rs:245-329.  Independent anchors: float64 closed forms of a
plane rotation, the `rotate_half` formulation of the half-split rule written with torch, torch's rms_norm,
norm preservation, and the permutation that maps one convention onto the other."""
import numpy as np
import pytest
import torch


# ---- reference tests (crates/rustorch-nn/src/rope.rs:245-329) ----------------------------------------------


def test_position_0_is_identity(oracle):
    rope = oracle.RoPE(4, 8, 10000.0)
    x = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    for fn in (rope.apply_interleaved, rope.apply_half_split):
        assert np.abs(fn(x, 1, 1, 1, 0) - x).max() < 1e-6


def test_preserves_pair_norms(oracle):
    rope = oracle.RoPE(8, 16, 10000.0)
    x = (np.arange(8, dtype=np.float32) + 1) * np.float32(0.1)
    y = rope.apply_interleaved(x, 1, 1, 1, 5)
    for k in range(4):
        assert abs((x[2 * k] ** 2 + x[2 * k + 1] ** 2) - (y[2 * k] ** 2 + y[2 * k + 1] ** 2)) < 1e-5
    z = rope.apply_half_split(x, 1, 1, 1, 5)
    for k in range(4):
        assert abs((x[k] ** 2 + x[k + 4] ** 2) - (z[k] ** 2 + z[k + 4] ** 2)) < 1e-5


def test_overflow_returns_err(oracle):
    rope = oracle.RoPE(4, 4, 10000.0)
    for fn in (rope.apply_interleaved, rope.apply_half_split):
        with pytest.raises(oracle.OracleError) as e:
            fn(np.zeros(8, dtype=np.float32), 1, 1, 2, 3)
        assert e.value.code == oracle.ERR_ROPE_POSITION_OVERFLOW
        assert (e.value.expected, e.value.got) == (4, 5)  # max_seq, requested (rope.rs:179-184)


def test_wrong_input_length(oracle):
    rope = oracle.RoPE(4, 4, 10000.0)
    for fn in (rope.apply_interleaved, rope.apply_half_split):
        with pytest.raises(oracle.OracleError) as e:
            fn(np.zeros(7, dtype=np.float32), 1, 1, 2, 0)
        assert e.value.code == oracle.ERR_ROPE_WRONG_INPUT_LEN
        assert (e.value.expected, e.value.got) == (8, 7)


def test_length_is_checked_before_position(oracle):
    rope = oracle.RoPE(4, 4, 10000.0)
    with pytest.raises(oracle.OracleError) as e:
        rope.apply_half_split(np.zeros(7, dtype=np.float32), 1, 1, 2, 3)
    assert e.value.code == oracle.ERR_ROPE_WRONG_INPUT_LEN


def test_batched_matches_row_by_row(oracle):
    rope = oracle.RoPE(4, 16, 10000.0)
    seq = 5
    x = (np.arange(seq * 4, dtype=np.float32) + 1) * np.float32(0.1)
    for name in ("apply_interleaved", "apply_half_split"):
        batched = getattr(rope, name)(x, 1, 1, seq, 0)
        rows = np.concatenate([getattr(rope, name)(x[4 * s:4 * s + 4], 1, 1, 1, s) for s in range(seq)])
        assert np.abs(batched - rows).max() < 1e-5


def test_odd_head_dim_is_rejected(oracle):
    with pytest.raises(ValueError):
        oracle.RoPE(5, 4)


# ---- independent anchors ------------------------------------------------------------------------------------


def test_tables_against_float64(oracle):
    d, n, base = 64, 300, 10000.0
    rope = oracle.RoPE(d, n, base)
    k = np.arange(d // 2, dtype=np.float64)
    ang = np.arange(n, dtype=np.float64)[:, None] / base ** (2 * k / d)[None, :]
    # f32 angle = p * theta carries a rounding of up to 2^-24 relative: 300 * 6e-8 = 2e-5 absolute in the angle
    assert np.abs(rope.cos.reshape(n, d // 2) - np.cos(ang)).max() < 5e-5
    assert np.abs(rope.sin.reshape(n, d // 2) - np.sin(ang)).max() < 5e-5
    # theta_0 = 1 exactly: column 0 is cos(p), sin(p) of the integer position
    assert np.abs(rope.cos.reshape(n, d // 2)[:, 0] - np.cos(np.arange(n))).max() < 1e-6
    assert rope.cos.shape == (n * d // 2,) and rope.sin[: d // 2].max() == 0.0


def test_unit_vector_rotates_to_cos_sin(oracle):
    """x = e_k: the half-split rule sends it to cos at k and sin at k + D/2 (a wrong sign or a swapped pair fails)."""
    d, p = 8, 3
    rope = oracle.RoPE(d, 8, 10000.0)
    for k in range(d // 2):
        x = np.zeros(d, dtype=np.float32)
        x[k] = 1.0
        y = rope.apply_half_split(x, 1, 1, 1, p)
        theta = p / 10000.0 ** (2 * k / d)
        want = np.zeros(d)
        want[k], want[k + d // 2] = np.cos(theta), np.sin(theta)
        assert np.abs(y - want).max() < 1e-6
        x = np.zeros(d, dtype=np.float32)
        x[k + d // 2] = 1.0
        y = rope.apply_half_split(x, 1, 1, 1, p)
        want = np.zeros(d)
        want[k], want[k + d // 2] = -np.sin(theta), np.cos(theta)
        assert np.abs(y - want).max() < 1e-6


def test_half_split_is_rotate_half_formulation(oracle):
    """HF's apply_rotary_pos_emb: x * cos + rotate_half(x) * sin with rotate_half(x) = cat(-x2, x1)."""
    g = torch.Generator().manual_seed(3)
    b, h, s, d, off = 2, 3, 7, 16, 4
    rope = oracle.RoPE(d, 32, 10000.0)
    x = torch.randn(b, h, s, d, generator=g, dtype=torch.float32)
    cos = torch.from_numpy(rope.cos.reshape(32, d // 2))[off:off + s]
    sin = torch.from_numpy(rope.sin.reshape(32, d // 2))[off:off + s]
    cos2, sin2 = torch.cat([cos, cos], -1).double(), torch.cat([sin, sin], -1).double()
    xd = x.double()
    rot = torch.cat([-xd[..., d // 2:], xd[..., : d // 2]], -1)
    want = (xd * cos2 + rot * sin2).numpy().ravel()
    got = rope.apply_half_split(x.numpy(), b, h, s, off)
    assert np.abs(got - want).max() < 1e-6


def test_conventions_differ_by_a_permutation(oracle):
    """interleaved(x)[2k], [2k+1] == half_split(perm x)[k], [k + D/2] where perm gathers even then odd dims."""
    rng = np.random.default_rng(5)
    d = 12
    rope = oracle.RoPE(d, 16, 500.0)
    x = rng.standard_normal(d).astype(np.float32)
    perm = np.concatenate([np.arange(0, d, 2), np.arange(1, d, 2)])
    a = rope.apply_interleaved(x, 1, 1, 1, 9)
    bb = rope.apply_half_split(x[perm], 1, 1, 1, 9)
    assert np.array_equal(a[perm], bb)


def test_rms_norm_against_torch_and_closed_form(oracle):
    rng = np.random.default_rng(11)
    n_heads, d, eps = 5, 32, 1e-6
    x = rng.standard_normal(n_heads * d).astype(np.float32)
    gamma = rng.standard_normal(d).astype(np.float32)
    got = oracle.rms_norm_per_head(x, gamma, n_heads, d, eps)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x).double().reshape(n_heads, d), (d,),
                                        torch.from_numpy(gamma).double(), eps).numpy().ravel()
    assert np.abs(got - want).max() < 2e-6
    # constant head c, gamma 1: c / sqrt(c^2 + eps)
    c = np.float32(0.75)
    got = oracle.rms_norm_per_head(np.full(2 * d, c), np.ones(d), 2, d, 0.25)
    assert np.abs(got - c / np.sqrt(c * c + 0.25)).max() < 1e-6
    # heads are independent: scaling one head leaves the others alone and leaves itself unchanged when eps -> 0
    y = x.copy()
    y[:d] *= 7.0
    got2 = oracle.rms_norm_per_head(y, gamma, n_heads, d, 0.0)
    got0 = oracle.rms_norm_per_head(x, gamma, n_heads, d, 0.0)
    assert np.array_equal(got2[d:], got0[d:]) and np.abs(got2[:d] - got0[:d]).max() < 1e-5


def _prepare_reference(oracle, q, k, v, kc, vc, pos, qg, kg, eps, rope, b_, hq, hkv, d, lmax):
    """The same step composed from the pinned pieces above, one head at a time."""
    qf = oracle.bf16_to_f32(q).reshape(b_, hq, d)
    kf = oracle.bf16_to_f32(k).reshape(b_, hkv, d)
    q_out = np.zeros((b_, hq, d), dtype=np.uint16)
    kc, vc = kc.copy().reshape(b_, hkv, lmax, d), vc.copy().reshape(b_, hkv, lmax, d)
    for b in range(b_):
        for h in range(hq):
            row = qf[b, h]
            if qg is not None:
                row = oracle.rms_norm_per_head(row, qg, 1, d, eps)
            q_out[b, h] = oracle.f32_to_bf16(rope.apply_half_split(row, 1, 1, 1, int(pos[b])))
        for h in range(hkv):
            row = kf[b, h]
            if kg is not None:
                row = oracle.rms_norm_per_head(row, kg, 1, d, eps)
            kc[b, h, pos[b]] = oracle.f32_to_bf16(rope.apply_half_split(row, 1, 1, 1, int(pos[b])))
            vc[b, h, pos[b]] = v.reshape(b_, hkv, d)[b, h]
    return q_out.ravel(), kc.ravel(), vc.ravel()


@pytest.mark.parametrize("norms", [(True, True), (False, False), (True, False)])
def test_decode_prepare_is_norm_then_rope_then_append(oracle, norms):
    rng = np.random.default_rng(21)
    b_, hq, hkv, d, lmax = 3, 4, 2, 16, 12
    rope = oracle.RoPE(d, lmax, 10000.0)
    q = oracle.f32_to_bf16(rng.standard_normal(b_ * hq * d).astype(np.float32))
    k = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * d).astype(np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * d).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * lmax * d).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * lmax * d).astype(np.float32))
    pos = np.array([0, 11, 5], dtype=np.int32)
    qg = rng.standard_normal(d).astype(np.float32) if norms[0] else None
    kg = rng.standard_normal(d).astype(np.float32) if norms[1] else None
    want_q, want_kc, want_vc = _prepare_reference(oracle, q, k, v, kc, vc, pos, qg, kg, 1e-6, rope, b_, hq, hkv, d, lmax)
    kc2, vc2 = kc.copy(), vc.copy()
    got_q = oracle.decode_prepare_bf16(q, k, v, kc2, vc2, pos, qg, kg, 1e-6, rope, b_, hq, hkv, d, lmax)
    assert np.array_equal(got_q, want_q) and np.array_equal(kc2, want_kc) and np.array_equal(vc2, want_vc)
    # position 0, no norm: q unchanged, k row 0 = k_in (identity rotation), v row = v_in
    if not any(norms):
        assert np.array_equal(got_q.reshape(b_, hq, d)[0], q.reshape(b_, hq, d)[0])
        assert np.array_equal(kc2.reshape(b_, hkv, lmax, d)[0, :, 0], k.reshape(b_, hkv, d)[0])
    # batch 1 with the cache's append rule (llm_kernels.rs:353-372) for v
    kc3, vc3 = kc[: hkv * lmax * d].copy(), vc[: hkv * lmax * d].copy()
    kc4, vc4 = kc3.copy(), vc3.copy()
    oracle.decode_prepare_bf16(q[: hq * d], k[: hkv * d], v[: hkv * d], kc3, vc3, [7], None, None, 0.0, rope, 1, hq, hkv,
                               d, lmax)
    oracle.kv_append_bf16(kc4, vc4, k[: hkv * d], v[: hkv * d], 7, hkv, d, lmax)
    assert np.array_equal(vc3, vc4)
    touched = np.nonzero(kc3 != kc4)[0]
    assert touched.size > 0 and set((touched // d) % lmax) == {7}  # only row 7 of each head differs (rotated k)


def test_decode_prepare_position_errors(oracle):
    d, lmax = 8, 4
    rope = oracle.RoPE(d, 16, 10000.0)
    z = np.zeros(1 * 1 * d, dtype=np.uint16)
    kc, vc = np.zeros(lmax * d, dtype=np.uint16), np.zeros(lmax * d, dtype=np.uint16)
    with pytest.raises(oracle.OracleError) as e:
        oracle.decode_prepare_bf16(z, z, z, kc, vc, [4], None, None, 0.0, rope, 1, 1, 1, d, lmax)
    assert e.value.code == oracle.ERR_KV_OVERFLOW and (e.value.expected, e.value.got) == (4, 5)
    with pytest.raises(oracle.OracleError) as e:
        oracle.decode_prepare_bf16(z, z, z, kc, vc, [16], None, None, 0.0, rope, 1, 1, 1, d, lmax)
    assert e.value.code == oracle.ERR_ROPE_POSITION_OVERFLOW
    assert not kc.any() and not vc.any()


def test_decode_prepare_with_several_new_tokens(oracle):
    """seq > 1 (a prompt): token s of a sequence is rotated at position p + s (rope.rs:192-193) and lands in cache
    row p + s (kv_cache.rs:97-110); assembled here from the batched RoPE call and the f32 cache append."""
    rng = np.random.default_rng(31)
    b_, hq, hkv, d, lmax, seq = 2, 3, 2, 8, 16, 5
    rope = oracle.RoPE(d, lmax, 10000.0)
    q = oracle.f32_to_bf16(rng.standard_normal(b_ * hq * seq * d).astype(np.float32))
    k = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * seq * d).astype(np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * seq * d).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * lmax * d).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * lmax * d).astype(np.float32))
    kg = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    pos = np.array([3, 11], dtype=np.int32)
    kc2, vc2 = kc.copy(), vc.copy()
    got_q = oracle.decode_prepare_bf16(q, k, v, kc2, vc2, pos, None, kg, 1e-6, rope, b_, hq, hkv, d, lmax, seq=seq)
    want_kc = oracle.bf16_to_f32(kc).reshape(b_, hkv * lmax * d).copy()
    want_vc = oracle.bf16_to_f32(vc).reshape(b_, hkv * lmax * d).copy()
    for b in range(b_):
        qb = oracle.bf16_to_f32(q).reshape(b_, hq * seq * d)[b]
        want_q = oracle.f32_to_bf16(rope.apply_half_split(qb, 1, hq, seq, int(pos[b])))
        assert np.array_equal(got_q.reshape(b_, -1)[b], want_q)
        kb = oracle.bf16_to_f32(k).reshape(b_, hkv * seq, d)[b]
        kb = oracle.rms_norm_per_head(kb, kg, hkv * seq, d, 1e-6)
        kb = oracle.bf16_to_f32(oracle.f32_to_bf16(rope.apply_half_split(kb, 1, hkv, seq, int(pos[b]))))
        vb = oracle.bf16_to_f32(v).reshape(b_, hkv * seq * d)[b]
        oracle.kv_cache_append(want_kc[b], want_vc[b], 1, hkv, lmax, d, int(pos[b]), seq, kb, vb)
    assert np.array_equal(oracle.bf16_to_f32(kc2), want_kc.ravel())
    assert np.array_equal(oracle.bf16_to_f32(vc2), want_vc.ravel())
    with pytest.raises(oracle.OracleError) as e:  # the last token would sit at row 16 of a 16-row cache
        oracle.decode_prepare_bf16(q, k, v, kc2, vc2, [3, 12], None, kg, 1e-6, rope, b_, hq, hkv, d, lmax, seq=seq)
    assert e.value.code == oracle.ERR_ROPE_POSITION_OVERFLOW and (e.value.expected, e.value.got) == (16, 17)
