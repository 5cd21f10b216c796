"""GPU parity of the decode path through the C ABI (rt_kv_append_bf16, rt_gqa_decode_online_bf16,
rt_gqa_decode_batched_bf16) against the CPU oracle.  Bar: max-abs <= 2e-2 and, per (sequence, head) row, relative Frobenius error
<= 1e-2, vs the f32 CPU path on the same bf16-rounded inputs."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_decode_parity, bf16_round, dev, max_abs
from _util import seeded_normal

pytestmark = pytest.mark.gpu
K = ra.LlmKernels()


def test_kv_append_bf16_matches_oracle(oracle):
    n_kv, d, max_seq = 8, 128, 33
    kc = np.random.default_rng(1).integers(0, 2 ** 16, n_kv * max_seq * d).astype(np.uint16)
    vc = np.random.default_rng(2).integers(0, 2 ** 16, n_kv * max_seq * d).astype(np.uint16)
    dk, dv = dev(kc), dev(vc)
    for pos in (0, 17, 32):
        k_in = np.random.default_rng(pos).integers(0, 2 ** 16, n_kv * d).astype(np.uint16)
        v_in = np.random.default_rng(pos + 100).integers(0, 2 ** 16, n_kv * d).astype(np.uint16)
        K.kv_append_bf16(None, dk, dv, dev(k_in), dev(v_in), pos, n_kv, d, max_seq)
        oracle.kv_append_bf16(kc, vc, k_in, v_in, pos, n_kv, d, max_seq)
    ra.synchronize()
    assert np.array_equal(dk.download(np.uint16), kc) and np.array_equal(dv.download(np.uint16), vc)
    with pytest.raises(ra.Overflow):
        K.kv_append_bf16(None, dk, dv, dk, dv, max_seq, n_kv, d, max_seq)


@pytest.mark.parametrize("hq,hkv,d,max_seq,kv_len", [(8, 2, 32, 320, 77), (32, 8, 128, 600, 600), (8, 2, 64, 10, 0)])
def test_gqa_decode_naive_bf16_is_the_same_function(oracle, hq, hkv, d, max_seq, kv_len):
    """llm_kernels.rs:461-545, :990-1042: the reference's three-pass decode kernel computes what the online one does
    (max, then exp and sum, then the weighted sum of V).  Checked against a float64 three-pass softmax written out
    here, and bit for bit against the online entry, whose kernels it runs."""
    qb, qf = bf16_round(seeded_normal((hq, d), 11))
    kb, kf = bf16_round(seeded_normal((hkv, max_seq, d), 12))
    vb, vf = bf16_round(seeded_normal((hkv, max_seq, d), 13))
    outs = []
    for call in (K.gqa_decode_naive_bf16, K.gqa_decode_online_bf16):
        dout = ra.HipStorage(hq * d * 2)
        dout.upload(np.full(hq * d, 0x7B7B, dtype=np.uint16))
        call(None, dev(qb), dev(kb), dev(vb), dout, hq, hkv, kv_len, d, max_seq)
        ra.synchronize()
        outs.append(dout.download(np.uint16))
    assert np.array_equal(outs[0], outs[1])
    got = oracle.bf16_to_f32(outs[0]).reshape(hq, d)
    q64 = qf.reshape(hq, d).astype(np.float64)
    k64 = kf.reshape(hkv, max_seq, d).astype(np.float64)
    v64 = vf.reshape(hkv, max_seq, d).astype(np.float64)
    for h in range(hq):
        kvh = h * hkv // hq
        if kv_len == 0:
            assert np.all(got[h] == 0.0)
            continue
        sc = k64[kvh, :kv_len] @ q64[h] / np.sqrt(np.float64(np.float32(d)))  # pass 1
        w = np.exp(sc - sc.max())                                               # pass 2
        want = (w / w.sum()) @ v64[kvh, :kv_len]                                # pass 3
        assert_decode_parity(got[h], want, d, f"head {h}")


@pytest.mark.parametrize("hq,hkv,d,max_seq,kv_len", [(8, 2, 32, 320, 1), (8, 2, 32, 320, 77), (32, 8, 128, 600, 600),
                                                     (6, 3, 96, 50, 49), (4, 4, 256, 40, 40), (8, 2, 64, 10, 0),
                                                     (16, 2, 256, 4096, 4096), (16, 2, 256, 100, 64), (8, 8, 256, 300, 257)])
def test_gqa_decode_online_bf16_matches_oracle(oracle, hq, hkv, d, max_seq, kv_len):
    """The reference call (batch 1): compared with the restated device kernel (bf16 out) and with
    the CPU path in f32."""
    qb, qf = bf16_round(seeded_normal((hq, d), 1))
    kb, kf = bf16_round(seeded_normal((hkv, max_seq, d), 2))
    vb, vf = bf16_round(seeded_normal((hkv, max_seq, d), 3))
    dout = ra.HipStorage(hq * d * 2)
    dout.upload(np.full(hq * d, 0x7B7B, dtype=np.uint16))
    K.gqa_decode_online_bf16(None, dev(qb), dev(kb), dev(vb), dout, hq, hkv, kv_len, d, max_seq)
    ra.synchronize()
    got = oracle.bf16_to_f32(dout.download(np.uint16))
    want_dev = oracle.bf16_to_f32(oracle.gqa_decode_online_bf16(qb, kb, vb, hq, hkv, kv_len, d, max_seq))
    assert_decode_parity(got, want_dev, d, "restated device kernel")
    want_cpu = oracle.gqa_decode_batched_bf16(qb, kb, vb, [kv_len], 1, hq, hkv, d, max_seq)
    assert_decode_parity(got, want_cpu, d, "cpu path")
    if kv_len == 1:
        g = hq // hkv
        assert np.array_equal(got.reshape(hq, d), np.repeat(vf.reshape(hkv, max_seq, d)[:, 0], g, axis=0))
    if kv_len == 0:
        assert (got == 0).all()


def run_batched(oracle, qb, kb, vb, lens, b, hq, hkv, d, max_seq):
    ws_bytes = K.gqa_decode_workspace_bytes(b, hq, hkv, d, max_seq)
    ws = ra.HipStorage(max(ws_bytes, 256))
    dout = ra.HipStorage(b * hq * d * 2)
    dout.upload(np.full(b * hq * d, 0x7B7B, dtype=np.uint16))
    K.gqa_decode_batched_bf16(None, dev(qb), dev(kb), dev(vb), dout, dev(np.asarray(lens, dtype=np.int32)), b, hq,
                              hkv, d, max_seq, ws, ws.byte_len)
    ra.synchronize()
    return oracle.bf16_to_f32(dout.download(np.uint16))


@pytest.mark.parametrize("b,hq,hkv,d,max_seq,lens", [
    (5, 32, 8, 128, 1100, [1, 511, 512, 513, 1100]),
    (3, 8, 8, 64, 700, [700, 0, 33]),
    (2, 8, 1, 128, 1500, [1500, 1023]),
    (2, 16, 8, 64, 300, [300, 17]),
    (2, 6, 2, 128, 100, [100, 50]),   # group of 3: outside the split-K kernel, generic path
    (2, 4, 2, 96, 100, [100, 50]),    # head dim 96: generic path
    (3, 16, 2, 256, 600, [600, 1, 333]),
    (2, 8, 8, 256, 130, [0, 130]),
])
def test_gqa_decode_batched_matches_oracle(oracle, b, hq, hkv, d, max_seq, lens):
    qb, qf = bf16_round(seeded_normal((b, hq, d), 1))
    kb, kf = bf16_round(seeded_normal((b, hkv, max_seq, d), 2))
    vb, vf = bf16_round(seeded_normal((b, hkv, max_seq, d), 3))
    got = run_batched(oracle, qb, kb, vb, lens, b, hq, hkv, d, max_seq)
    want = oracle.gqa_decode_batched_bf16(qb, kb, vb, lens, b, hq, hkv, d, max_seq)
    assert np.isfinite(got).all()
    assert_decode_parity(got, want, d)
    g4 = got.reshape(b, hq, d)
    v4 = vf.reshape(b, hkv, max_seq, d)
    for i, L in enumerate(lens):
        if L == 1:  # one key: out == v_0 exactly
            assert np.array_equal(g4[i], np.repeat(v4[i, :, 0], hq // hkv, axis=0))
        if L == 0:
            assert (g4[i] == 0).all()


def test_decode_split_equals_unsplit(oracle):
    """Split-K invariance: the batched (chunked) path and the single-pass reference call agree for
    lengths on both sides of every chunk boundary."""
    hq, hkv, d, max_seq = 8, 2, 128, 2100
    qb, _ = bf16_round(seeded_normal((1, hq, d), 1))
    kb, _ = bf16_round(seeded_normal((1, hkv, max_seq, d), 2))
    vb, _ = bf16_round(seeded_normal((1, hkv, max_seq, d), 3))
    dq, dk, dv = dev(qb), dev(kb), dev(vb)
    for L in (511, 512, 513, 1024, 1025, 2047, 2100):
        split = run_batched(oracle, qb, kb, vb, [L], 1, hq, hkv, d, max_seq)
        dout = ra.HipStorage(hq * d * 2)
        K.gqa_decode_online_bf16(None, dq, dk, dv, dout, hq, hkv, L, d, max_seq)
        ra.synchronize()
        one = oracle.bf16_to_f32(dout.download(np.uint16))
        assert max_abs(split, one) <= 2 ** -7 * np.abs(one).max() + 1e-6, L


def test_decode_workspace_too_small_is_an_error():
    b, hq, hkv, d, max_seq = 2, 8, 2, 128, 1024
    z = ra.HipStorage(b * hkv * max_seq * d * 2)
    lens = dev(np.array([5, 5], dtype=np.int32))
    with pytest.raises(ra.DeviceError) as ei:
        K.gqa_decode_batched_bf16(None, z, z, z, z, lens, b, hq, hkv, d, max_seq, z, 16)
    assert ei.value.status == 22 and ei.value.expected == K.gqa_decode_workspace_bytes(b, hq, hkv, d, max_seq)


def test_config_decode_b64_h32_kv8_d128_lmax8192(oracle):
    """The decode workload of the benchmark set at full size: lengths uniform in [512, 8192] from a seed, N(0,1) bf16
    caches in the contiguous (B, Hkv, Lmax, D) layout."""
    b, hq, hkv, d, max_seq = 64, 32, 8, 128, 8192
    lens = np.random.default_rng(4).integers(512, 8193, size=b).astype(np.int32)
    rng = np.random.default_rng(44)
    n_cache = b * hkv * max_seq * d
    kb = np.empty(n_cache, dtype=np.uint16)
    vb = np.empty(n_cache, dtype=np.uint16)
    step = n_cache // 16
    for i in range(16):  # generate in slices to bound host memory
        kb[i * step:(i + 1) * step] = oracle.f32_to_bf16(rng.standard_normal(step, dtype=np.float32))
        vb[i * step:(i + 1) * step] = oracle.f32_to_bf16(rng.standard_normal(step, dtype=np.float32))
    qb, _ = bf16_round(seeded_normal((b, hq, d), 1))
    got = run_batched(oracle, qb, kb, vb, lens, b, hq, hkv, d, max_seq)
    want = oracle.gqa_decode_batched_bf16(qb, kb, vb, lens, b, hq, hkv, d, max_seq)
    assert np.isfinite(got).all()
    assert_decode_parity(got, want, d, f"lens={lens.tolist()}")


def test_single_sequence_decode_long_contexts_and_streams(oracle):
    """The reference call on the split-K path: contexts long enough for a hundred partials per head, a cache that
    grows between calls (the library's per-stream buffer is re-sized), and two streams used alternately (each has
    a buffer of its own)."""
    hq, hkv, d = 32, 8, 128
    streams = [None, ra.Stream(), ra.Stream()]
    for max_seq, kv_lens in [(96, [1, 33, 96]), (8192, [8192, 4097, 2048, 65]), (300, [300])]:
        qb, _ = bf16_round(seeded_normal((hq, d), max_seq))
        kb, _ = bf16_round(seeded_normal((hkv, max_seq, d), max_seq + 1))
        vb, _ = bf16_round(seeded_normal((hkv, max_seq, d), max_seq + 2))
        dq, dk, dv = dev(qb), dev(kb), dev(vb)
        outs = []
        for i, kv_len in enumerate(kv_lens):
            st = streams[i % len(streams)]
            dout = ra.HipStorage(hq * d * 2)
            K.gqa_decode_online_bf16(st, dq, dk, dv, dout, hq, hkv, kv_len, d, max_seq)
            outs.append((kv_len, dout))
        for st in streams:
            ra.synchronize(st)
        for kv_len, dout in outs:
            want = oracle.gqa_decode_batched_bf16(qb, kb, vb, [kv_len], 1, hq, hkv, d, max_seq)
            assert_decode_parity(oracle.bf16_to_f32(dout.download(np.uint16)), want, d, f"{max_seq} {kv_len}")


def test_shutdown_frees_and_the_library_stays_usable(oracle):
    hq, hkv, d, max_seq, kv_len = 8, 2, 64, 300, 257
    qb, _ = bf16_round(seeded_normal((hq, d), 1))
    kb, _ = bf16_round(seeded_normal((hkv, max_seq, d), 2))
    vb, _ = bf16_round(seeded_normal((hkv, max_seq, d), 3))
    want = oracle.gqa_decode_batched_bf16(qb, kb, vb, [kv_len], 1, hq, hkv, d, max_seq)
    for _ in range(2):
        dout = ra.HipStorage(hq * d * 2)
        K.gqa_decode_online_bf16(None, dev(qb), dev(kb), dev(vb), dout, hq, hkv, kv_len, d, max_seq)
        ra.synchronize()
        assert_decode_parity(oracle.bf16_to_f32(dout.download(np.uint16)), want, d)
        small = ra.flash_forward(ra.AttentionShape.new(1, 1, 4, 4), *[np.ones(16, np.float32)] * 3)  # pinned staging
        assert np.allclose(small, 1.0)
        ra.shutdown()


def test_decode_unaligned_tensors_take_the_elementwise_kernel(oracle):
    """q and caches that start 2 bytes past a 16-byte boundary: the 16-byte loads of the split-K kernels do not apply,
    the call routes to the one-workgroup-per-head kernel and gives the same result; a misaligned workspace is an
    error."""
    b, hq, hkv, d, max_seq = 2, 8, 2, 128, 300
    lens = [300, 77]
    qb, _ = bf16_round(seeded_normal((b, hq, d), 1))
    kb, _ = bf16_round(seeded_normal((b, hkv, max_seq, d), 2))
    vb, _ = bf16_round(seeded_normal((b, hkv, max_seq, d), 3))
    want = oracle.gqa_decode_batched_bf16(qb, kb, vb, lens, b, hq, hkv, d, max_seq)

    def shifted(bits):  # a device buffer whose payload starts at byte 2
        host = np.concatenate([np.zeros(1, np.uint16), bits.ravel()])
        store = dev(host)
        return store, store.ptr + 2

    (sq, pq), (sk, pk), (sv, pv) = shifted(qb), shifted(kb), shifted(vb)
    dlens = dev(np.asarray(lens, dtype=np.int32))
    ws = ra.HipStorage(max(K.gqa_decode_workspace_bytes(b, hq, hkv, d, max_seq), 256))
    dout = ra.HipStorage(b * hq * d * 2)
    K.gqa_decode_batched_bf16(None, pq, pk, pv, dout, dlens, b, hq, hkv, d, max_seq, ws, ws.byte_len)
    ra.synchronize()
    assert_decode_parity(oracle.bf16_to_f32(dout.download(np.uint16)), want, d)
    # the single-sequence call on sequence 1's slabs
    dout1 = ra.HipStorage(hq * d * 2)
    K.gqa_decode_online_bf16(None, pq + hq * d * 2, pk + hkv * max_seq * d * 2, pv + hkv * max_seq * d * 2, dout1, hq, hkv,
                             lens[1], d, max_seq)
    ra.synchronize()
    assert_decode_parity(oracle.bf16_to_f32(dout1.download(np.uint16)), want.reshape(b, hq * d)[1], d)
    with pytest.raises(ra.DeviceError) as ei:
        K.gqa_decode_batched_bf16(None, dev(qb), dev(kb), dev(vb), dout, dlens, b, hq, hkv, d, max_seq, ws.ptr + 4,
                                  ws.byte_len - 4)
    assert ei.value.status == 22
