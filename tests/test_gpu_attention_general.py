"""GPU parity of the general bf16 attention entries through the C ABI -- rt_mha_forward_masked_bf16_dev (the masked /
cross-attention core of MultiHeadAttention::forward, crates/rustorch-nn/src/attention.rs:371-399, on bf16 tensors)
and rt_gqa_decode_chunk_bf16 (gqa_decode_batched_f32, crates/rustorch-metal/src/kernels.rs:14432-14516, in bf16 over
a batch) -- against the CPU oracle run in f32 on the same bf16-rounded inputs.  Bar: max-abs <= 2e-2 and relative Frobenius
error <= 1e-2 per block of 256 rows, NaN patterns exact."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_bf16_parity, bf16_round, dev, max_abs
from _util import seeded_normal

pytestmark = pytest.mark.gpu
K = ra.LlmKernels()


def run_masked(oracle, b, tq, tkv, h, d, mask, seed=0):
    qb, qf = bf16_round(seeded_normal(b * tq * h * d, seed))
    kb, kf = bf16_round(seeded_normal(b * tkv * h * d, seed + 1))
    vb, vf = bf16_round(seeded_normal(b * tkv * h * d, seed + 2))
    dout = ra.HipStorage(max(qb.size, 8) * 2)
    dout.upload(np.full(max(qb.size, 8), 0x7B7B, dtype=np.uint16))
    m = None if mask is None else np.ascontiguousarray(mask, dtype=np.float32).ravel()
    dm = None if m is None else dev(m)
    dq, dk, dv = (dev(x) if x.size else None for x in (qb, kb, vb))  # held until the launch has run
    ra.mha_forward_masked_bf16_dev(dq, dk, dv, dout, b, tq, tkv, h, d, dm, 0 if m is None else m.size)
    ra.synchronize()
    got = oracle.bf16_to_f32(dout.download(np.uint16, qb.size))
    want = oracle.mha_forward_masked(qf, kf, vf, b, tq, tkv, h, d, mask)
    assert_bf16_parity(got, want, d, None, f"b={b} tq={tq} tkv={tkv} h={h} d={d}")
    return got


@pytest.mark.parametrize("b,t,h,d", [(1, 1, 1, 8), (2, 5, 3, 8), (2, 128, 4, 64), (1, 70, 2, 96), (1, 33, 1, 136),
                                     (2, 257, 2, 32), (1, 130, 2, 256), (1, 200, 3, 80), (2, 40, 2, 20), (1, 65, 2, 300)])
@pytest.mark.parametrize("kind", ["none", "causal", "window", "bool", "per_head"])
def test_self_attention_with_masks(oracle, b, t, h, d, kind):
    rng = np.random.default_rng(7)
    mask = {"none": None, "causal": ra.causal_mask(t), "window": ra.sliding_window_mask(t, 3),
            "bool": ra.bool_to_additive((rng.random((t, t)) > 0.4).astype(np.float32)),
            "per_head": (rng.standard_normal((b * h, t, t)) * 2).astype(np.float32)}[kind]
    run_masked(oracle, b, t, t, h, d, mask)


@pytest.mark.parametrize("b,tq,tkv,h,d", [(2, 4, 9, 2, 8), (1, 100, 7, 3, 64), (2, 1, 300, 2, 128), (1, 6, 1, 1, 16),
                                          (2, 70, 333, 3, 80), (1, 257, 64, 2, 24), (1, 33, 1000, 1, 128),
                                          (1, 31, 97, 2, 136), (8, 16, 512, 8, 64), (2, 129, 130, 2, 256)])
def test_cross_attention(oracle, b, tq, tkv, h, d):
    rng = np.random.default_rng(9)
    run_masked(oracle, b, tq, tkv, h, d, None)
    run_masked(oracle, b, tq, tkv, h, d, np.where(rng.random((tq, tkv)) > 0.3, 0.0, -1.0e4).astype(np.float32))
    run_masked(oracle, b, tq, tkv, h, d, (rng.standard_normal((b * h, tq, tkv))).astype(np.float32))


def test_masked_rows_and_edge_cases(oracle):
    b, t, h, d = 1, 6, 2, 8
    m = np.zeros((t, t), dtype=np.float32)
    m[2, :] = -1.0e4  # masked everywhere with the reference's value: uniform weights, finite
    got = run_masked(oracle, b, t, t, h, d, m)
    assert np.isfinite(got).all()
    m[3, :] = -np.inf  # masked everywhere with -inf: that row is NaN, as in the reference's softmax
    got = run_masked(oracle, b, t, t, h, d, m).reshape(b, t, h * d)
    assert np.isnan(got[0, 3]).all() and np.isfinite(np.delete(got[0], 3, axis=0)).all()
    # no keys: rows of zeros
    assert not run_masked(oracle, b, t, 0, h, d, None).any()
    # the routing rule's unmasked self-attention equals the flash entry on the [B,T,H,hd] layout
    t, d = 300, 64
    qb, _ = bf16_round(seeded_normal(b * t * h * d, 1))
    kb, _ = bf16_round(seeded_normal(b * t * h * d, 2))
    vb, _ = bf16_round(seeded_normal(b * t * h * d, 3))
    o1, o2 = ra.HipStorage(qb.size * 2), ra.HipStorage(qb.size * 2)
    dq, dk, dv = dev(qb), dev(kb), dev(vb)  # held until both launches have run
    ra.mha_forward_masked_bf16_dev(dq, dk, dv, o1, b, t, t, h, d)
    ra.flash_forward_bnhd_bf16_dev(ra.AttentionShape.new(b, h, t, d), dq, dk, dv, o2)
    ra.synchronize()
    a1, a2 = o1.download(np.uint16), o2.download(np.uint16)
    assert np.array_equal(a1, a2), f"{int((a1 != a2).sum())} of {a1.size} elements differ"


def test_masked_bf16_errors():
    z = ra.HipStorage(1 << 16)
    with pytest.raises(ra.DeviceError) as ei:  # head dim above 512
        ra.mha_forward_masked_bf16_dev(z, z, z, z, 1, 4, 4, 2, 520)
    assert ei.value.status == 21
    with pytest.raises(ra.WrongInputLen):  # mask of the wrong size
        ra.mha_forward_masked_bf16_dev(z, z, z, z, 1, 4, 4, 2, 16, z, 15)


# ---- chunked causal decode over the cache -------------------------------------------------------------------

def run_chunk(oracle, b, s, hq, hkv, d, max_seq, lens, seed=0, scalar_len=False):
    qb, _ = bf16_round(seeded_normal((b, s, hq, d), seed))
    kb, _ = bf16_round(seeded_normal((b, hkv, max_seq, d), seed + 1))
    vb, _ = bf16_round(seeded_normal((b, hkv, max_seq, d), seed + 2))
    dout = ra.HipStorage(qb.size * 2)
    dout.upload(np.full(qb.size, 0x7B7B, dtype=np.uint16))
    arg = int(lens[0]) if scalar_len else dev(np.asarray(lens, dtype=np.int32))
    dq, dk, dv = dev(qb), dev(kb), dev(vb)  # held until the launch has run
    K.gqa_decode_chunk_bf16(None, dq, dk, dv, dout, arg, b, s, hq, hkv, d, max_seq)
    ra.synchronize()
    got = oracle.bf16_to_f32(dout.download(np.uint16))
    want = oracle.gqa_decode_chunk_bf16(qb, kb, vb, lens, b, s, hq, hkv, d, max_seq)
    assert_bf16_parity(got, want, d, None, f"b={b} s={s} hq={hq} hkv={hkv} d={d} lens={list(lens)}")
    return got, (qb, kb, vb)


@pytest.mark.parametrize("b,s,hq,hkv,d,max_seq,lens", [
    (1, 4, 8, 2, 128, 300, [260]),
    (3, 7, 32, 8, 128, 1100, [1100, 7, 513]),
    (2, 16, 8, 8, 64, 200, [200, 16]),
    (2, 5, 6, 2, 96, 150, [150, 77]),        # a group of 3
    (1, 33, 16, 2, 256, 400, [400]),
    (2, 130, 4, 1, 64, 500, [500, 131]),      # more rows than one tile holds
    (2, 3, 4, 4, 80, 64, [64, 3]),
    (1, 1, 32, 8, 128, 2100, [2100]),
    # one long cache and few new positions (the reference's own call shape): the keys are cut into spans whose
    # partials a second kernel folds
    (1, 16, 32, 8, 128, 8192, [8192]),
    (1, 4, 32, 8, 128, 8192, [8191]),
    (2, 7, 8, 2, 64, 3000, [3000, 700]),      # spans of a sequence much shorter than the cache: most of them empty
    (1, 33, 16, 2, 256, 2000, [1999]),
    (1, 40, 4, 1, 96, 1000, [1000]),          # two query tiles, each with its spans
    (3, 5, 8, 2, 128, 1500, [1500, 3, 0]),    # a sequence shorter than the chunk, and an empty one
    # one head per kv head (rows are not packed) and a cache too short for spans: positions without keys are rows of
    # zeros here as well, not the NaN rows of flash_forward
    (1, 8, 1, 1, 64, 64, [5]),
    (1, 8, 1, 1, 128, 64, [0]),
    (2, 8, 4, 4, 64, 64, [5, 64]),
    (2, 6, 2, 2, 96, 100, [2, 100]),
])
def test_chunk_decode_matches_oracle(oracle, b, s, hq, hkv, d, max_seq, lens):
    run_chunk(oracle, b, s, hq, hkv, d, max_seq, lens)


@pytest.mark.parametrize("s", [4, 16])
def test_chunk_decode_of_one_long_sequence_with_a_host_length(oracle, s):
    """batch 1, kv_lens = NULL and kv_len = pos_base + B: the reference call (kernels.rs:14522-14570) at 8192 keys."""
    run_chunk(oracle, 1, s, 32, 8, 128, 8192, [8192], seed=s, scalar_len=True)
    run_chunk(oracle, 1, s, 32, 8, 128, 8192, [5000], seed=s + 1, scalar_len=True)


def test_chunk_of_one_is_the_batched_decode(oracle):
    """seq_new = 1: the same numbers as rt_gqa_decode_batched_bf16 (within the bar; the kernels differ), a sequence
    without keys included: both leave a row of zeros for it."""
    b, hq, hkv, d, max_seq = 4, 32, 8, 128, 700
    lens = [700, 1, 513, 0]
    got, (qb, kb, vb) = run_chunk(oracle, b, 1, hq, hkv, d, max_seq, lens)
    want = oracle.gqa_decode_batched_bf16(qb, kb, vb, lens, b, hq, hkv, d, max_seq)
    assert_bf16_parity(got, want, d, None)
    ws = ra.HipStorage(max(K.gqa_decode_workspace_bytes(b, hq, hkv, d, max_seq), 256))
    dout = ra.HipStorage(qb.size * 2)
    dq, dk, dv, dl = dev(qb), dev(kb), dev(vb), dev(np.asarray(lens, np.int32))
    K.gqa_decode_batched_bf16(None, dq, dk, dv, dout, dl, b, hq, hkv, d, max_seq, ws, ws.byte_len)
    ra.synchronize()
    batched = oracle.bf16_to_f32(dout.download(np.uint16))
    assert_bf16_parity(got, batched, d, None)
    assert not got.reshape(b, -1)[3].any() and not batched.reshape(b, -1)[3].any()


def test_chunk_from_position_zero_is_causal_prefill(oracle):
    """pos_base = 0 (the cache holds exactly the new positions): causal self-attention of the chunk, equal to the
    prefill entry on the [B,T,H,hd] layout with the keys taken from the cache."""
    b, s, hq, hkv, d = 2, 150, 8, 2, 128
    got, (qb, kb, vb) = run_chunk(oracle, b, s, hq, hkv, d, s, [s, s], scalar_len=True)
    k4 = oracle.bf16_to_f32(kb).reshape(b, hkv, s, d)
    v4 = oracle.bf16_to_f32(vb).reshape(b, hkv, s, d)
    q4 = oracle.bf16_to_f32(qb).reshape(b, s, hq, d).transpose(0, 2, 1, 3)
    g = hq // hkv
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, hq, s, d), np.ascontiguousarray(q4),
                                       np.repeat(k4, g, axis=1), np.repeat(v4, g, axis=1), "causal")
    want = want.reshape(b, hq, s, d).transpose(0, 2, 1, 3)
    assert_bf16_parity(got.reshape(b, s, hq, d), want, d, None)


def test_chunk_decode_errors_and_rows_without_keys(oracle):
    z = ra.HipStorage(1 << 16)
    with pytest.raises(ra.Overflow):  # scalar kv_len shorter than the chunk
        K.gqa_decode_chunk_bf16(None, z, z, z, z, 3, 1, 4, 8, 2, 64, 16)
    with pytest.raises(ra.DeviceError) as ei:
        K.gqa_decode_chunk_bf16(None, z, z, z, z, 8, 1, 4, 8, 2, 20, 16)
    assert ei.value.status == 21
    # a sequence whose cache is shorter than the chunk: its first positions see no key and come out as rows of zeros
    got, _ = run_chunk(oracle, 2, 4, 4, 2, 64, 32, [2, 32])
    g = got.reshape(2, 4, 4, 64)
    assert not g[0, :2].any() and g[0, 2:].any(axis=-1).all() and np.isfinite(g).all()
    with pytest.raises(TypeError):
        K.gqa_decode_chunk_bf16(None, z, z, z, z, 3.5, 1, 4, 8, 2, 64, 16)
    K.gqa_decode_chunk_bf16(None, z, z, z, z, np.int32(16), 1, 4, 8, 2, 64, 16)  # a numpy integer is a length, not an address
    ra.synchronize()
