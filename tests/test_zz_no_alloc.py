"""rt_gqa_decode_batched_bf16_noalloc (the decode entry that allocates nothing: its split-K partials live in a fixed
block of device memory inside the library) against rt_gqa_decode_batched_bf16 with a caller workspace, through the
C ABI.  Same kernels, same arithmetic: the outputs must be equal bit for bit, and within 2e-2 of the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import rustorch_amd as ra
from rustorch_amd import _lib
from _gpu import assert_decode_parity, bf16_round, dev
from _util import seeded_normal

pytestmark = pytest.mark.gpu
K = ra.LlmKernels()


_hip = _lib.hip_runtime()
_hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]


def device_free_bytes():
    free, total = C.c_size_t(), C.c_size_t()
    assert _hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def both(oracle, b, hq, hkv, d, max_seq, lens, seed):
    qb, _ = bf16_round(seeded_normal((b, hq, d), seed))
    kb, _ = bf16_round(seeded_normal((b, hkv, max_seq, d), seed + 1))
    vb, _ = bf16_round(seeded_normal((b, hkv, max_seq, d), seed + 2))
    dq, dk, dv = dev(qb), dev(kb), dev(vb)
    dl = dev(np.asarray(lens, dtype=np.int32))
    ws = ra.HipStorage(max(K.gqa_decode_workspace_bytes(b, hq, hkv, d, max_seq), 256))
    outs = []
    for entry in ("ws", "static"):
        dout = ra.HipStorage(b * hq * d * 2)
        dout.upload(np.full(b * hq * d, 0x7B7B, dtype=np.uint16))
        if entry == "ws":
            K.gqa_decode_batched_bf16(None, dq, dk, dv, dout, dl, b, hq, hkv, d, max_seq, ws, ws.byte_len)
        else:
            free_before = device_free_bytes()
            K.gqa_decode_batched_bf16_noalloc(None, dq, dk, dv, dout, dl, b, hq, hkv, d, max_seq)
            assert device_free_bytes() == free_before, "the no-allocation entry changed the free device memory"
        ra.synchronize()
        outs.append(dout.download(np.uint16))
    want = oracle.gqa_decode_batched_bf16(qb, kb, vb, lens, b, hq, hkv, d, max_seq)
    return outs[0], outs[1], want


def test_noalloc_decode_equals_the_workspace_entry_on_two_calls_in_a_row(oracle):
    ra.init(0)
    # a large ragged batch first, then a smaller one: the second call finds the first call's partials in the block
    cases = [(12, 32, 8, 128, 2100, [2100, 1, 511, 512, 513, 0, 1025, 77, 2048, 1500, 33, 900], 11),
             (3, 8, 2, 64, 300, [300, 17, 129], 21),
             (2, 16, 4, 256, 200, [200, 64], 31),
             # one sequence: spans of two steps, ~125 partials per head, the merge that folds them four ways in parallel
             (1, 32, 8, 128, 8192, [8001], 41),
             (1, 8, 2, 64, 100, [33], 51)]
    for b, hq, hkv, d, max_seq, lens, seed in cases:
        with_ws, static, want = both(oracle, b, hq, hkv, d, max_seq, lens, seed)
        assert np.array_equal(with_ws, static), (b, hq, hkv, d)
        assert_decode_parity(oracle.bf16_to_f32(static), want, d)


def test_noalloc_decode_limits():
    d = 128
    z = ra.HipStorage(1 << 20)
    lens = dev(np.zeros(4096, dtype=np.int32))
    # more (sequence, kv head) segments than the fixed block holds partials for
    with pytest.raises(ra.DeviceError) as ei:
        K.gqa_decode_batched_bf16_noalloc(None, z, z, z, z, lens, 4096, 32, 8, d, 16)
    assert ei.value.status == 22 and ei.value.got == 8 << 20 and ei.value.expected > 8 << 20
    # a group of 3 query heads per kv head has no split-K kernel
    with pytest.raises(ra.DeviceError) as ei:
        K.gqa_decode_batched_bf16_noalloc(None, z, z, z, z, lens, 2, 6, 2, 96, 16)
    assert ei.value.status == 21
    # misaligned q
    with pytest.raises(ra.DeviceError) as ei:
        K.gqa_decode_batched_bf16_noalloc(None, z.ptr + 2, z, z, z, lens, 2, 8, 2, d, 16)
    assert ei.value.status == 21
