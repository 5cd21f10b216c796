"""Pins the oracle's online-softmax monoid, GQA forward, KV-cache indexing, bf16 rounding and the
decode restatements.  Reference tests restated: online_softmax.rs:177-384, gqa.rs:278-388,
kv_cache.rs:289-359; independent anchors: float64 brute force, torch's bf16 cast, algebraic laws."""
import numpy as np
import pytest
import torch

from _util import attention_f64, seeded_normal


def close(a, b, tol):
    if np.isnan(a) and np.isnan(b):
        return True
    if np.isinf(a) and np.isinf(b) and np.sign(a) == np.sign(b):
        return True
    return abs(a - b) <= tol * (1.0 + max(abs(a), abs(b)))


def naive_ml(xs):
    xs = np.asarray(xs, dtype=np.float64)
    if xs.size == 0:
        return -np.inf, 0.0
    m = xs.max()
    with np.errstate(invalid="ignore"):
        return m, np.exp(xs - m).sum()


# ---- online softmax (online_softmax.rs:177-306) ---------------------------------------------


def test_single_tile_matches_naive(oracle):
    xs = [0.5, -1.0, 2.5, 0.1, -3.0, 4.0]
    st = oracle.online_softmax_full(xs)
    m, l = naive_ml(xs)
    assert close(st.m, m, 1e-6) and close(st.l, l, 1e-6)


def test_four_tiles_combine_match_naive(oracle):
    xs = np.sin(np.arange(32, dtype=np.float32) * np.float32(0.1))
    comb = oracle.OnlineSoftmaxState()
    for i in range(0, 32, 8):
        comb = oracle.combine_tiles(comb, oracle.online_softmax_full(xs[i:i + 8]))
    m, l = naive_ml(xs)
    assert close(comb.m, m, 1e-7) and close(comb.l, l, 1e-6)


def test_associativity_and_commutativity(oracle):
    S = oracle.OnlineSoftmaxState
    a, b, c, d = S(1.5, 3.0), S(0.7, 5.0), S(2.1, 1.0), S(-0.3, 7.0)
    ct = oracle.combine_tiles
    s1 = ct(ct(a, b), ct(c, d))
    s2 = ct(ct(ct(a, b), c), d)
    s3 = ct(a, ct(b, ct(c, d)))
    for s in (s2, s3):
        assert close(s1.m, s.m, 1e-6) and close(s1.l, s.l, 1e-6)
    ab, ba = ct(a, b), ct(b, a)
    assert close(ab.m, ba.m, 1e-7) and close(ab.l, ba.l, 1e-7)
    # closed form: l = 3 + 5*exp(0.7-1.5)
    assert close(ab.l, 3.0 + 5.0 * np.exp(0.7 - 1.5), 1e-6) and ab.m == 1.5


def test_empty_and_identity(oracle):
    st = oracle.online_softmax_full([])
    assert st.m == -np.inf and st.l == 0.0 and st.is_empty()
    s = oracle.OnlineSoftmaxState(1.5, 3.0)
    for r in (oracle.combine_tiles(oracle.OnlineSoftmaxState(), s), oracle.combine_tiles(s, oracle.OnlineSoftmaxState())):
        assert (r.m, r.l) == (1.5, 3.0)
    one = oracle.online_softmax_full([2.5])
    two = oracle.OnlineSoftmaxState.from_scalar(2.5)
    assert (one.m, one.l) == (two.m, two.l) == (2.5, 1.0)


def test_all_neg_inf_and_pos_inf(oracle):
    st = oracle.online_softmax_full([-np.inf] * 4)
    assert st.m == -np.inf and (np.isnan(st.l) or st.l == 0.0)
    st = oracle.online_softmax_full([1.0, np.inf, -2.0, 0.0])
    assert st.m == np.inf and st.l == 1.0


def test_large_magnitudes(oracle):
    st = oracle.online_softmax_full(np.array([1e10, 1e10 + 1e-5, 1e10 - 1e-5], dtype=np.float32))
    assert st.m == np.float32(1e10) and abs(st.l - 3.0) < 0.1
    st = oracle.online_softmax_full(np.array([1e30] * 4, dtype=np.float32))
    assert st.m == np.float32(1e30) and st.l == 4.0


def test_online_softmax_properties(oracle):
    """online_softmax.rs:333-384 (1000 cases each in the reference; 300 here for time)."""
    rng = np.random.default_rng(7)
    for _ in range(300):
        xs = rng.uniform(-100, 100, size=int(rng.integers(1, 200))).astype(np.float32)
        full = oracle.online_softmax_full(xs)
        m, l = naive_ml(xs)
        assert close(full.m, m, 1e-6) and close(full.l, l, 1e-5)
        tile = int(rng.integers(1, max(xs.size, 2)))
        comb = oracle.OnlineSoftmaxState()
        for i in range(0, xs.size, tile):
            comb = oracle.combine_tiles(comb, oracle.online_softmax_full(xs[i:i + tile]))
        assert close(full.m, comb.m, 1e-6) and close(full.l, comb.l, 1e-5)
        a = oracle.OnlineSoftmaxState(float(rng.uniform(-100, 100)), float(rng.uniform(0.001, 1000)))
        b = oracle.OnlineSoftmaxState(float(rng.uniform(-100, 100)), float(rng.uniform(0.001, 1000)))
        ab, ba = oracle.combine_tiles(a, b), oracle.combine_tiles(b, a)
        assert close(ab.m, ba.m, 1e-7) and close(ab.l, ba.l, 1e-6)


# ---- GQA (gqa.rs:278-388) ------------------------------------------------------------------


def test_gqa_with_n_kv_heads_eq_n_heads_matches_mha(oracle):
    b, hq, hkv, sq, skv, d = 1, 4, 4, 3, 3, 4
    q = (np.arange(b * hq * sq * d, dtype=np.float32) + 1) * np.float32(0.01)
    k = (np.arange(b * hkv * skv * d, dtype=np.float32) + 1) * np.float32(0.02)
    v = (np.arange(b * hkv * skv * d, dtype=np.float32) + 1) * np.float32(0.03)
    out = oracle.gqa_forward_f32(q, k, v, b, hq, hkv, sq, skv, d).reshape(hq, sq, d)
    vv = v.reshape(hkv, skv * d)
    for h in range(hq):
        assert out[h].min() >= vv[h].min() - 1e-5 and out[h].max() <= vv[h].max() + 1e-5
    ref = attention_f64(q.reshape(1, hq, sq, d), k.reshape(1, hkv, skv, d), v.reshape(1, hkv, skv, d))
    assert np.abs(out - ref[0]).max() < 1e-6


def test_gqa_4_to_1_group_ratio(oracle):
    b, hq, hkv, sq, skv, d = 1, 8, 2, 4, 4, 8
    q = np.sin(np.arange(b * hq * sq * d, dtype=np.float32) * np.float32(0.001))
    k = np.cos(np.arange(b * hkv * skv * d, dtype=np.float32) * np.float32(0.001))
    v = np.tan((np.arange(b * hkv * skv * d, dtype=np.float32) + 1) * np.float32(0.0005))
    out = oracle.gqa_forward_f32(q, k, v, b, hq, hkv, sq, skv, d).reshape(hq, sq, d)
    assert np.isfinite(out).all()
    g = hq // hkv
    for kvh in range(hkv):
        assert np.abs(out[kvh * g, 0] - out[kvh * g + g - 1, 0]).sum() > 1e-6
    # equality with explicit replication of K/V to Hq heads (float64)
    kr = np.repeat(k.reshape(1, hkv, skv, d), g, axis=1)
    vr = np.repeat(v.reshape(1, hkv, skv, d), g, axis=1)
    ref = attention_f64(q.reshape(1, hq, sq, d), kr, vr)
    assert np.abs(out - ref[0]).max() < 1e-6


@pytest.mark.parametrize("sq,skv", [(1, 37), (5, 37), (1, 1), (3, 300)])
def test_gqa_decode_branch_matches_f64(oracle, sq, skv):
    """seq_q != seq_kv takes decode_attn_row (gqa.rs:216-270): unmasked cross attention.
    head mapping kv_h = h / group: a wrong mapping (h % n_kv) fails the float64 comparison."""
    b, hq, hkv, d = 2, 6, 3, 16
    q = seeded_normal((b, hq, sq, d), 1)
    k = seeded_normal((b, hkv, skv, d), 2)
    v = seeded_normal((b, hkv, skv, d), 3)
    out = oracle.gqa_forward_f32(q, k, v, b, hq, hkv, sq, skv, d).reshape(b, hq, sq, d)
    g = hq // hkv
    ref = attention_f64(q, np.repeat(k, g, axis=1), np.repeat(v, g, axis=1))
    assert np.abs(out - ref).max() < 5e-6
    out1 = oracle.gqa_forward_f32(q, k, v, b, hq, hkv, sq, skv, d, threads=1).reshape(b, hq, sq, d)
    assert np.array_equal(out, out1)


def test_gqa_errors(oracle):
    """gqa.rs:370-388 and the head-count, q, k, v, out order of :106-141."""
    z = lambda n: np.zeros(n, dtype=np.float32)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.gqa_forward_f32(z(20), z(8), z(8), 1, 5, 2, 1, 1, 4)
    assert ei.value.code == oracle.ERR_HEAD_COUNT_MISMATCH
    with pytest.raises(oracle.OracleError) as ei:
        oracle.gqa_forward_f32(z(20), z(8), z(8), 1, 4, 0, 1, 1, 4)
    assert ei.value.code == oracle.ERR_HEAD_COUNT_MISMATCH
    with pytest.raises(oracle.OracleError) as ei:
        oracle.gqa_forward_f32(z(7), z(8), z(8), 1, 4, 2, 1, 1, 4)
    assert (ei.value.code, ei.value.which, ei.value.expected, ei.value.got) == (oracle.ERR_WRONG_INPUT_LEN, "q", 16, 7)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.gqa_forward_f32(z(16), z(9), z(8), 1, 4, 2, 1, 1, 4)
    assert ei.value.which == "k"
    with pytest.raises(oracle.OracleError) as ei:
        oracle.gqa_forward_f32(z(16), z(8), z(9), 1, 4, 2, 1, 1, 4)
    assert ei.value.which == "v"
    with pytest.raises(oracle.OracleError) as ei:
        oracle.gqa_forward_f32(z(16), z(8), z(8), 1, 4, 2, 1, 1, 4, out_len=15)
    assert ei.value.which == "out"


# ---- KV cache (kv_cache.rs:289-359) ---------------------------------------------------------


def test_kv_cache_append_index_table(oracle):
    b, h, d, max_seq = 1, 2, 4, 8
    kc = np.zeros(b * h * max_seq * d, dtype=np.float32)
    vc = np.zeros_like(kc)
    bhsd = 2 * 3 * 4
    nk = np.arange(bhsd, dtype=np.float32) * np.float32(0.1)
    nv = np.arange(bhsd, dtype=np.float32) * np.float32(0.01)
    oracle.kv_cache_append(kc, vc, b, h, max_seq, d, 0, 3, nk, nv)
    # h=0 rows land at [0..12), h=1 rows at [32..44) (kv_cache.rs:306-322)
    assert np.array_equal(kc[0:12], nk[0:12]) and np.array_equal(kc[32:44], nk[12:24])
    assert np.array_equal(vc[32:44], nv[12:24]) and (kc[12:32] == 0).all()
    # a second append goes behind the first
    oracle.kv_cache_append(kc, vc, b, h, max_seq, d, 3, 1, np.full(8, 7, np.float32), np.full(8, 9, np.float32))
    assert (kc[12:16] == 7).all() and (kc[44:48] == 7).all() and (vc[44:48] == 9).all()
    # trim of the valid prefix (model.rs:638-650)
    t = oracle.kv_trim(kc, h, max_seq, 4, d).reshape(h, 4, d)
    assert np.array_equal(t[0].ravel(), kc[0:16]) and np.array_equal(t[1].ravel(), kc[32:48])


def test_kv_cache_errors(oracle):
    kc = np.zeros(16, dtype=np.float32)
    vc = np.zeros(16, dtype=np.float32)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.kv_cache_append(kc, vc, 1, 1, 4, 4, 0, 5, np.zeros(20, np.float32), np.zeros(20, np.float32))
    assert ei.value.code == oracle.ERR_KV_OVERFLOW and (ei.value.got, ei.value.expected) == (5, 4)
    with pytest.raises(oracle.OracleError) as ei:
        oracle.kv_cache_append(kc, vc, 1, 1, 4, 4, 0, 1, np.zeros(3, np.float32), np.zeros(3, np.float32))
    assert ei.value.code == oracle.ERR_KV_WRONG_INPUT_LEN and ei.value.expected == 4


# ---- bf16 rounding ---------------------------------------------------------------------------


def test_bf16_round_to_nearest_even_matches_torch(oracle):
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2 ** 32, size=200000, dtype=np.uint64).astype(np.uint32)
    ties = np.array([0x3F808000, 0x3F818000, 0x3F7F8000, 0x00008000, 0x00018000, 0x7F7F8000, 0x7F7FFFFF,
                     0x80008000, 0x00000001, 0x7F800000, 0xFF800000, 0x3F800001, 0x3F80FFFF], dtype=np.uint32)
    x = np.concatenate([bits, ties]).view(np.float32)
    got = oracle.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(oracle.bf16_to_f32(got[nan])).all()
    # round trip is exact on bf16 values
    assert np.array_equal(oracle.f32_to_bf16(oracle.bf16_to_f32(got[~nan])), got[~nan])


# ---- device-convention decode (llm_kernels.rs:353-457) -----------------------------------------


def _bf16(oracle, x):
    bits = oracle.f32_to_bf16(x)
    return bits, oracle.bf16_to_f32(bits)


def test_kv_append_bf16_indexing(oracle):
    n_kv, d, max_seq = 3, 8, 5
    kc = np.zeros(n_kv * max_seq * d, dtype=np.uint16)
    vc = np.zeros_like(kc)
    k_in = np.arange(1, n_kv * d + 1, dtype=np.uint16)
    v_in = k_in + 100
    oracle.kv_append_bf16(kc, vc, k_in, v_in, 2, n_kv, d, max_seq)
    kc3 = kc.reshape(n_kv, max_seq, d)
    assert np.array_equal(kc3[:, 2, :].ravel(), k_in) and kc3[:, [0, 1, 3, 4], :].sum() == 0
    assert np.array_equal(vc.reshape(n_kv, max_seq, d)[:, 2, :].ravel(), v_in)


@pytest.mark.parametrize("kv_len", [1, 2, 77, 300])
def test_gqa_decode_online_bf16_matches_f64(oracle, kv_len):
    """One-pass device-convention decode vs float64 attention over the valid prefix; kv_len = 1
    => out == v_0 exactly (bf16 in, bf16 out)."""
    hq, hkv, d, max_seq = 8, 2, 32, 320
    qb, qf = _bf16(oracle, seeded_normal((hq, d), 1))
    kb, kf = _bf16(oracle, seeded_normal((hkv, max_seq, d), 2))
    vb, vf = _bf16(oracle, seeded_normal((hkv, max_seq, d), 3))
    out = oracle.bf16_to_f32(oracle.gqa_decode_online_bf16(qb, kb, vb, hq, hkv, kv_len, d, max_seq)).reshape(hq, d)
    g = hq // hkv
    kk = np.repeat(kf.reshape(hkv, max_seq, d)[:, :kv_len], g, axis=0)[None]
    vv = np.repeat(vf.reshape(hkv, max_seq, d)[:, :kv_len], g, axis=0)[None]
    ref = attention_f64(qf.reshape(1, hq, 1, d), kk, vv)[0, :, 0, :]
    assert np.abs(out - ref).max() <= 2e-2
    assert np.abs(out - ref).max() <= np.abs(ref).max() * 2 ** -8 + 1e-6  # one bf16 rounding of the result
    if kv_len == 1:
        assert np.array_equal(out, vv[0, :, 0, :].astype(np.float32))


def test_gqa_decode_batched_matches_per_sequence_reference_call(oracle):
    """The ragged-batch oracle equals, sequence by sequence, the reference's own B=1 call chain
    (trim the cache, then gqa_forward_f32 with seq_q = 1), and float64 attention."""
    B, hq, hkv, d, max_seq = 3, 8, 2, 16, 50
    lens = np.array([50, 1, 23], dtype=np.int32)
    qb, qf = _bf16(oracle, seeded_normal((B, hq, d), 1))
    kb, kf = _bf16(oracle, seeded_normal((B, hkv, max_seq, d), 2))
    vb, vf = _bf16(oracle, seeded_normal((B, hkv, max_seq, d), 3))
    out = oracle.gqa_decode_batched_bf16(qb, kb, vb, lens, B, hq, hkv, d, max_seq).reshape(B, hq, d)
    kf = kf.reshape(B, hkv, max_seq, d)
    vf = vf.reshape(B, hkv, max_seq, d)
    qf = qf.reshape(B, hq, d)
    for b in range(B):
        n = int(lens[b])
        kt = oracle.kv_trim(kf[b], hkv, max_seq, n, d)
        vt = oracle.kv_trim(vf[b], hkv, max_seq, n, d)
        one = oracle.gqa_forward_f32(qf[b], kt, vt, 1, hq, hkv, 1, n, d).reshape(hq, d)
        if n == 1:
            # seq_q == seq_kv == 1 takes the flash branch (gqa.rs:151): out = v, as decode gives
            assert np.allclose(out[b], one, atol=1e-6)
        else:
            assert np.array_equal(out[b], one)
        g = hq // hkv
        ref = attention_f64(qf[b].reshape(1, hq, 1, d), np.repeat(kf[b, :, :n], g, axis=0)[None],
                            np.repeat(vf[b, :, :n], g, axis=0)[None])[0, :, 0]
        assert np.abs(out[b] - ref).max() < 5e-6


# ---- ro_gqa_decode_chunk_bf16: gqa_decode_batched_f32 (crates/rustorch-metal/src/kernels.rs:14432-14516) ------


def _chunk_inputs(oracle, b, s, hq, hkv, d, max_seq, seed):
    rng = np.random.default_rng(seed)
    q = oracle.f32_to_bf16(rng.standard_normal((b, s, hq, d), dtype=np.float32))
    k = oracle.f32_to_bf16(rng.standard_normal((b, hkv, max_seq, d), dtype=np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal((b, hkv, max_seq, d), dtype=np.float32))
    return q, k, v


def test_chunk_decode_against_float64_brute_force(oracle):
    """Every (sequence, position, head) row against softmax(q.K^T / sqrt(d)) V in float64 over the keys
    [0, kv_len - seq_new + s]: a wrong causal offset, head map or layout fails here."""
    b, s, hq, hkv, d, max_seq = 2, 5, 6, 2, 16, 40
    lens = [40, 9]
    q, k, v = _chunk_inputs(oracle, b, s, hq, hkv, d, max_seq, 3)
    got = oracle.gqa_decode_chunk_bf16(q, k, v, lens, b, s, hq, hkv, d, max_seq).reshape(b, s, hq, d)
    qf = oracle.bf16_to_f32(q).astype(np.float64).reshape(b, s, hq, d)
    kf = oracle.bf16_to_f32(k).astype(np.float64).reshape(b, hkv, max_seq, d)
    vf = oracle.bf16_to_f32(v).astype(np.float64).reshape(b, hkv, max_seq, d)
    for bi in range(b):
        for si in range(s):
            n = lens[bi] - s + si + 1
            for h in range(hq):
                kv = h // (hq // hkv)
                sc = kf[bi, kv, :n] @ qf[bi, si, h] / np.sqrt(np.float64(np.float32(d)))
                w = np.exp(sc - sc.max())
                want = (w / w.sum()) @ vf[bi, kv, :n]
                assert np.abs(got[bi, si, h] - want).max() <= 5e-6, (bi, si, h)


def test_chunk_of_one_position_is_the_single_row_decode(oracle):
    """seq_new = 1 reduces to decode_attn_row on the prefix (gqa.rs:216-270), the function the batched decode oracle
    applies: same phases in the same order."""
    b, hq, hkv, d, max_seq = 3, 8, 2, 32, 70
    lens = [70, 1, 33]
    q, k, v = _chunk_inputs(oracle, b, 1, hq, hkv, d, max_seq, 5)
    a = oracle.gqa_decode_chunk_bf16(q, k, v, lens, b, 1, hq, hkv, d, max_seq)
    w = oracle.gqa_decode_batched_bf16(q, k, v, lens, b, hq, hkv, d, max_seq)
    assert np.abs(a - w).max() <= 1e-6


def test_chunk_from_position_zero_is_causal_attention(oracle):
    """kv_len = seq_new (pos_base 0): row s sees keys [0, s], which is the causal forward of
    cpu_forward.rs:193-425 on the same tensors (closed form: row 0 equals V[0])."""
    b, s, hq, hkv, d = 1, 37, 4, 2, 16
    q, k, v = _chunk_inputs(oracle, b, s, hq, hkv, d, s, 8)
    got = oracle.gqa_decode_chunk_bf16(q, k, v, [s], b, s, hq, hkv, d, s).reshape(b, s, hq, d)
    vf = oracle.bf16_to_f32(v).reshape(b, hkv, s, d)
    kf = oracle.bf16_to_f32(k).reshape(b, hkv, s, d)
    qf = oracle.bf16_to_f32(q).reshape(b, s, hq, d).transpose(0, 2, 1, 3)
    g = hq // hkv
    assert np.array_equal(got[0, 0], np.repeat(vf[0, :, 0], g, axis=0))
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, hq, s, d), np.ascontiguousarray(qf),
                                       np.repeat(kf, g, axis=1), np.repeat(vf, g, axis=1), "causal")
    assert np.abs(got - want.reshape(b, hq, s, d).transpose(0, 2, 1, 3)).max() <= 1e-5


def test_chunk_position_without_keys_is_a_row_of_zeros(oracle):
    """The shader's loops over an empty key range leave acc = 0.0 (kernels.rs:14504-14514); the same rule as the
    single-position decode with kv_len == 0."""
    q, k, v = _chunk_inputs(oracle, 1, 3, 2, 1, 8, 10, 1)
    got = oracle.gqa_decode_chunk_bf16(q, k, v, [1], 1, 3, 2, 1, 8, 10).reshape(3, 2, 8)
    assert (got[:2] == 0.0).all() and np.isfinite(got[2]).all() and got[2].any()
    # seq_new = 1 with an empty cache: what gqa_decode_batched_bf16 gives for kv_len == 0
    q, k, v = _chunk_inputs(oracle, 2, 1, 4, 2, 8, 10, 2)
    got = oracle.gqa_decode_chunk_bf16(q, k, v, [0, 7], 2, 1, 4, 2, 8, 10)
    want = oracle.gqa_decode_batched_bf16(q, k, v, [0, 7], 2, 4, 2, 8, 10)
    assert np.abs(got - want).max() <= 1e-6 and not got.reshape(2, -1)[0].any()
