"""rt_qk_norm_rope_kv_append_bf16 against the oracle's restatement of steps 2a, 2b, 3 of decode_step
(crates/rustorch-llm/src/model.rs:575-636): bit-exact on bf16 storage (the kernel runs the reference's f32
arithmetic in the reference's order and rounds once)."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_decode_parity

pytestmark = pytest.mark.gpu


def _case(oracle, rng, b_, hq, hkv, d, lmax, positions, norms, eps=1e-6, base=10000.0, table_rows=None, seq=1):
    rope = ra.RoPE(d, table_rows or lmax, base)
    oro = oracle.RoPE(d, table_rows or lmax, base)
    oro.cos, oro.sin = rope.cos.copy(), rope.sin.copy()  # the caller's tables are an input of the kernel
    q = oracle.f32_to_bf16(rng.standard_normal(b_ * hq * seq * d).astype(np.float32))
    k = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * seq * d).astype(np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * seq * d).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * lmax * d).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal(b_ * hkv * lmax * d).astype(np.float32))
    qg = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32) if norms[0] else None
    kg = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32) if norms[1] else None
    return rope, oro, q, k, v, kc, vc, qg, kg


def _run(oracle, rope, oro, q, k, v, kc, vc, qg, kg, positions, b_, hq, hkv, d, lmax, eps, scalar_pos=False, seq=1):
    K = ra.LlmKernels()
    dq, dk, dv, dkc, dvc = (ra.HipStorage.from_numpy(x) for x in (q, k, v, kc, vc))
    dqg = ra.HipStorage.from_numpy(qg) if qg is not None else None
    dkg = ra.HipStorage.from_numpy(kg) if kg is not None else None
    pos_arg = int(positions[0]) if scalar_pos else ra.HipStorage.from_numpy(np.asarray(positions, dtype=np.int32))
    K.qk_norm_rope_kv_append_bf16(None, dq, dk, dv, dkc, dvc, pos_arg, rope, b_, hq, hkv, d, lmax, q_gamma=dqg,
                                  k_gamma=dkg, eps=eps, seq=seq)
    ra.synchronize()
    want_kc, want_vc = kc.copy(), vc.copy()
    want_q = oracle.decode_prepare_bf16(q, k, v, want_kc, want_vc, positions, qg, kg, eps, oro, b_, hq, hkv, d, lmax,
                                        seq=seq)
    got_q, got_kc, got_vc = dq.download(np.uint16), dkc.download(np.uint16), dvc.download(np.uint16)
    assert np.array_equal(got_q, want_q)
    assert np.array_equal(got_kc, want_kc)
    assert np.array_equal(got_vc, want_vc)


@pytest.mark.parametrize("norms", [(True, True), (False, False), (True, False), (False, True)])
@pytest.mark.parametrize("b_,hq,hkv,d,lmax", [(3, 4, 2, 16, 12), (2, 8, 8, 64, 40), (64, 32, 8, 128, 256), (1, 2, 1, 258, 9)])
def test_matches_oracle_bit_for_bit(oracle, norms, b_, hq, hkv, d, lmax):
    rng = np.random.default_rng(100 + d + b_)
    positions = rng.integers(0, lmax, size=b_).astype(np.int32)
    positions[0] = 0
    positions[-1] = lmax - 1
    rope, oro, q, k, v, kc, vc, qg, kg = _case(oracle, rng, b_, hq, hkv, d, lmax, positions, norms)
    _run(oracle, rope, oro, q, k, v, kc, vc, qg, kg, positions, b_, hq, hkv, d, lmax, 1e-6)


@pytest.mark.parametrize("norms", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("b_,hq,hkv,d,lmax,seq", [(2, 3, 1, 16, 24, 5), (2, 8, 2, 128, 700, 300), (1, 4, 4, 64, 64, 64),
                                                  (2, 4, 2, 256, 400, 257), (1, 2, 1, 96, 1100, 1024), (2, 2, 2, 72, 80, 40),
                                                  (1, 6, 2, 32, 40, 33), (3, 2, 1, 128, 31, 31)])
def test_several_new_tokens_match_oracle_bit_for_bit(oracle, b_, hq, hkv, d, lmax, seq, norms):
    """A prompt: [batch, heads, seq, head_dim] inputs, token s at position p + s and cache row p + s.  From 32 tokens
    on, head dims that are a multiple of 16 up to 256 take the kernel that moves 64 consecutive tokens of a head
    through LDS; the others (and head dim 72 here) the one-wave-per-row kernel: the same
    bits either way."""
    rng = np.random.default_rng(300 + seq)
    positions = rng.integers(0, lmax - seq + 1, size=b_).astype(np.int32)
    positions[-1] = lmax - seq
    rope, oro, q, k, v, kc, vc, qg, kg = _case(oracle, rng, b_, hq, hkv, d, lmax, positions, norms, seq=seq)
    _run(oracle, rope, oro, q, k, v, kc, vc, qg, kg, positions, b_, hq, hkv, d, lmax, 1e-6, seq=seq)


def test_prompt_overflow_is_reported_for_the_last_token():
    rope = ra.RoPE(8, 16)
    K = ra.LlmKernels()
    buf = ra.HipStorage(4096)
    with pytest.raises(ra.Overflow) as e:
        K.qk_norm_rope_kv_append_bf16(None, buf, buf, buf, buf, buf, 3, rope, 1, 1, 1, 8, 7, seq=5)
    assert (e.value.requested, e.value.max) == (8, 7)
    with pytest.raises(ra.PositionOverflow) as e:
        K.qk_norm_rope_kv_append_bf16(None, buf, buf, buf, buf, buf, 12, rope, 1, 1, 1, 8, 32, seq=5)
    assert (e.value.max_seq, e.value.requested) == (16, 17)


def test_scalar_position_is_the_reference_call(oracle):
    """batch 1, one host position: rope_half_split x2 + kv_append_bf16 of cuda_backend.rs:486-540 in one call."""
    rng = np.random.default_rng(7)
    b_, hq, hkv, d, lmax = 1, 32, 8, 128, 64
    rope, oro, q, k, v, kc, vc, qg, kg = _case(oracle, rng, b_, hq, hkv, d, lmax, [17], (True, True), table_rows=128)
    _run(oracle, rope, oro, q, k, v, kc, vc, qg, kg, np.array([17], dtype=np.int32), b_, hq, hkv, d, lmax, 1e-5,
         scalar_pos=True)


def test_large_rope_base_and_long_position(oracle):
    rng = np.random.default_rng(9)
    b_, hq, hkv, d, lmax = 2, 4, 4, 128, 8192
    rope, oro, q, k, v, kc, vc, qg, kg = _case(oracle, rng, b_, hq, hkv, d, lmax, None, (True, True), base=500000.0)
    _run(oracle, rope, oro, q, k, v, kc, vc, qg, kg, np.array([8191, 4097], dtype=np.int32), b_, hq, hkv, d, lmax, 1e-6)


def test_position_errors_and_untouched_buffers(oracle):
    rng = np.random.default_rng(3)
    b_, hq, hkv, d, lmax = 2, 2, 1, 8, 4
    rope, oro, q, k, v, kc, vc, qg, kg = _case(oracle, rng, b_, hq, hkv, d, lmax, None, (False, False), table_rows=16)
    K = ra.LlmKernels()
    dq, dk, dv, dkc, dvc = (ra.HipStorage.from_numpy(x) for x in (q, k, v, kc, vc))
    with pytest.raises(ra.Overflow) as e:  # inside the tables, outside the cache
        K.qk_norm_rope_kv_append_bf16(None, dq, dk, dv, dkc, dvc, 4, rope, b_, hq, hkv, d, lmax)
    assert (e.value.requested, e.value.max) == (5, 4)
    with pytest.raises(ra.PositionOverflow) as e:  # the RoPE check comes first (model.rs:620-636: rope, then append)
        K.qk_norm_rope_kv_append_bf16(None, dq, dk, dv, dkc, dvc, 16, rope, b_, hq, hkv, d, lmax)
    assert (e.value.max_seq, e.value.requested) == (16, 17)
    with pytest.raises(ra.DeviceError):
        K.qk_norm_rope_kv_append_bf16(None, dq, dk, dv, dkc, dvc, 0, ra.RoPE(6, 16), b_, hq, hkv, 7, lmax)
    # device positions out of range: that sequence is left alone, the other one is processed
    pos = ra.HipStorage.from_numpy(np.array([9, 2], dtype=np.int32))
    K.qk_norm_rope_kv_append_bf16(None, dq, dk, dv, dkc, dvc, pos, rope, b_, hq, hkv, d, lmax)
    ra.synchronize()
    got_q, got_kc = dq.download(np.uint16).reshape(b_, hq, d), dkc.download(np.uint16).reshape(b_, hkv, lmax, d)
    assert np.array_equal(got_q[0], q.reshape(b_, hq, d)[0]) and np.array_equal(got_kc[0], kc.reshape(b_, hkv, lmax, d)[0])
    want_kc, want_vc = kc.copy(), vc.copy()
    want_q = oracle.decode_prepare_bf16(q[hq * d:], k[hkv * d:], v[hkv * d:], want_kc[hkv * lmax * d:],
                                        want_vc[hkv * lmax * d:], [2], None, None, 1e-6, oro, 1, hq, hkv, d, lmax)
    assert np.array_equal(got_q[1].ravel(), want_q)
    assert np.array_equal(got_kc[1].ravel(), want_kc[hkv * lmax * d:])


def test_prepare_then_decode_matches_cpu_decode_step(oracle):
    """The device inner loop of one decode step -- prepare, then batched GQA decode over [..pos+1] -- against
    the CPU path on the same bf16 inputs."""
    rng = np.random.default_rng(12)
    b_, hq, hkv, d, lmax = 4, 8, 2, 128, 96
    positions = np.array([0, 95, 33, 64], dtype=np.int32)
    rope, oro, q, k, v, kc, vc, qg, kg = _case(oracle, rng, b_, hq, hkv, d, lmax, positions, (True, True))
    K = ra.LlmKernels()
    dq, dk, dv, dkc, dvc = (ra.HipStorage.from_numpy(x) for x in (q, k, v, kc, vc))
    dqg, dkg = ra.HipStorage.from_numpy(qg), ra.HipStorage.from_numpy(kg)
    dpos = ra.HipStorage.from_numpy(positions)
    dlens = ra.HipStorage.from_numpy(positions + 1)
    dout = ra.HipStorage(b_ * hq * d * 2)
    ws_bytes = K.gqa_decode_workspace_bytes(b_, hq, hkv, d, lmax)
    ws = ra.HipStorage(max(ws_bytes, 256))
    K.qk_norm_rope_kv_append_bf16(None, dq, dk, dv, dkc, dvc, dpos, rope, b_, hq, hkv, d, lmax, q_gamma=dqg,
                                  k_gamma=dkg)
    K.gqa_decode_batched_bf16(None, dq, dkc, dvc, dout, dlens, b_, hq, hkv, d, lmax, ws, ws.byte_len)
    ra.synchronize()
    want_kc, want_vc = kc.copy(), vc.copy()
    want_q = oracle.decode_prepare_bf16(q, k, v, want_kc, want_vc, positions, qg, kg, 1e-6, oro, b_, hq, hkv, d, lmax)
    want = oracle.gqa_decode_batched_bf16(want_q, want_kc, want_vc, positions + 1, b_, hq, hkv, d, lmax)
    got = oracle.bf16_to_f32(dout.download(np.uint16))
    assert_decode_parity(got, want, d)
