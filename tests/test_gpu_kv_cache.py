"""Device KVCache mirror against the oracle's KVLayerCache::append (crates/rustorch-nn/src/kv_cache.rs:77-112)
and the reference's own tests (kv_cache.rs:289-359): same protocol, same errors, same index table."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_decode_parity

pytestmark = pytest.mark.gpu


def test_new_cache_has_zero_len_and_zeroed_buffers():
    c = ra.KVCache(12, 1, 8, 64, 128)
    assert (c.num_layers(), c.max_seq(), c.current_len()) == (12, 128, 0)
    assert c.dims() == (1, 8, 128, 64)
    ra.synchronize()
    assert not c.k_buffer(0).download(np.uint16).any() and not c.v_buffer(11).download(np.uint16).any()
    assert c.k_buffer(12) is None and ra.KVCache(0, 1, 1, 4, 4).dims() is None


@pytest.mark.parametrize("dtype,np_dtype", [("f32", np.float32), ("bf16", np.uint16)])
@pytest.mark.parametrize("b,h,lmax,d", [(1, 1, 5, 2), (2, 3, 16, 8), (1, 2, 9, 3), (2, 2, 40, 128)])
def test_append_advance_matches_oracle(oracle, dtype, np_dtype, b, h, lmax, d):
    """Prefill-sized append, then token by token; every step compared with the oracle on float32 values."""
    rng = np.random.default_rng(5)
    c = ra.KVCache(2, b, h, d, lmax, dtype=dtype)
    want_k = np.zeros(b * h * lmax * d, dtype=np.float32)
    want_v = np.zeros_like(want_k)
    cur = 0
    for seq_added in (min(3, lmax - 1), 1, 1):
        nk = rng.standard_normal(b * h * seq_added * d).astype(np.float32)
        nv = rng.standard_normal(b * h * seq_added * d).astype(np.float32)
        if dtype == "bf16":
            nk, nv = oracle.bf16_to_f32(oracle.f32_to_bf16(nk)), oracle.bf16_to_f32(oracle.f32_to_bf16(nv))
            dk, dv = ra.HipStorage.from_numpy(oracle.f32_to_bf16(nk)), ra.HipStorage.from_numpy(oracle.f32_to_bf16(nv))
        else:
            dk, dv = ra.HipStorage.from_numpy(nk), ra.HipStorage.from_numpy(nv)
        c.append(1, seq_added, dk, dv)
        c.advance(seq_added)
        oracle.kv_cache_append(want_k, want_v, b, h, lmax, d, cur, seq_added, nk, nv)
        cur += seq_added
        assert c.current_len() == cur
        ra.synchronize()
        got_k, got_v = c.k_buffer(1).download(np_dtype), c.v_buffer(1).download(np_dtype)
        if dtype == "bf16":
            got_k, got_v = oracle.bf16_to_f32(got_k), oracle.bf16_to_f32(got_v)
        assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)
    assert not c.k_buffer(0).download(np_dtype).any()  # the other layer is untouched


def test_index_table_of_the_reference():
    """kv_cache.rs:306-322: batch 1, 1 head, max_seq 4, head_dim 2; two appends land at rows 0 and 1."""
    c = ra.KVCache(1, 1, 1, 2, 4, dtype="f32")
    for step, (kk, vv) in enumerate((([1.0, 2.0], [10.0, 20.0]), ([3.0, 4.0], [30.0, 40.0]))):
        c.append(0, 1, ra.HipStorage.from_numpy(np.array(kk, dtype=np.float32)),
                 ra.HipStorage.from_numpy(np.array(vv, dtype=np.float32)))
        c.advance(1)
    ra.synchronize()
    assert c.k_buffer(0).download(np.float32)[:4].tolist() == [1.0, 2.0, 3.0, 4.0]
    assert c.v_buffer(0).download(np.float32)[:4].tolist() == [10.0, 20.0, 30.0, 40.0]
    c.clear()
    assert c.current_len() == 0
    assert c.k_buffer(0).download(np.float32)[:2].tolist() == [1.0, 2.0]  # contents stay, only the length resets


def test_errors_of_the_reference():
    c = ra.KVCache(1, 1, 1, 2, 2, dtype="f32")
    two = ra.HipStorage.from_numpy(np.zeros(2, dtype=np.float32))
    three = ra.HipStorage.from_numpy(np.zeros(3, dtype=np.float32))
    six = ra.HipStorage.from_numpy(np.zeros(6, dtype=np.float32))
    with pytest.raises(ra.Overflow) as e:  # kv_cache.rs:326-336
        c.append(0, 3, six, six)
    assert (e.value.requested, e.value.max) == (3, 2)
    with pytest.raises(ra.KVWrongInputLen) as e:  # kv_cache.rs:338-348
        c.append(0, 1, three, two)
    assert (e.value.expected, e.value.got_k, e.value.got_v) == (2, 3, 2)
    with pytest.raises(ra.LayerOutOfRange) as e:
        c.append(5, 1, two, two)
    assert (e.value.layer, e.value.num_layers) == (5, 1)
    c.advance(2)
    with pytest.raises(ra.Overflow) as e:
        c.advance(1)
    assert (e.value.requested, e.value.max) == (3, 2) and c.current_len() == 2
    with pytest.raises(ra.Overflow):  # overflow is checked before the lengths (kv_cache.rs:84-97)
        c.append(0, 1, three, three)


def test_cache_feeds_decode_without_a_trim(oracle):
    """Prefill 5 tokens, append one more, decode over [..6] straight from the cache buffers."""
    rng = np.random.default_rng(8)
    b, hq, hkv, d, lmax = 2, 4, 2, 64, 32
    c = ra.KVCache(1, b, hkv, d, lmax)
    K = ra.LlmKernels()
    kc = np.zeros(b * hkv * lmax * d, dtype=np.float32)
    vc = np.zeros_like(kc)
    cur = 0
    for seq_added in (5, 1):
        nk = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal(b * hkv * seq_added * d).astype(np.float32)))
        nv = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal(b * hkv * seq_added * d).astype(np.float32)))
        c.append(0, seq_added, ra.HipStorage.from_numpy(oracle.f32_to_bf16(nk)), ra.HipStorage.from_numpy(oracle.f32_to_bf16(nv)))
        c.advance(seq_added)
        oracle.kv_cache_append(kc, vc, b, hkv, lmax, d, cur, seq_added, nk, nv)
        cur += seq_added
    q = oracle.f32_to_bf16(rng.standard_normal(b * hq * d).astype(np.float32))
    dq, dout = ra.HipStorage.from_numpy(q), ra.HipStorage(b * hq * d * 2)
    lens = np.full(b, c.current_len(), dtype=np.int32)
    dl = ra.HipStorage.from_numpy(lens)
    ws = ra.HipStorage(max(K.gqa_decode_workspace_bytes(b, hq, hkv, d, lmax), 256))
    K.gqa_decode_batched_bf16(None, dq, c.k_buffer(0), c.v_buffer(0), dout, dl, b, hq, hkv, d, lmax, ws, ws.byte_len)
    ra.synchronize()
    want = oracle.gqa_decode_batched_bf16(q, oracle.f32_to_bf16(kc), oracle.f32_to_bf16(vc), lens, b, hq, hkv, d, lmax)
    assert_decode_parity(oracle.bf16_to_f32(dout.download(np.uint16)), want, d)
