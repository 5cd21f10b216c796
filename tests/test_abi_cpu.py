"""CPU-side checks of the C ABI: the library loads without a GPU, exports every symbol the header
declares, and reports the reference's errors (in the reference's order) before touching a device."""
import os
import re

import numpy as np
import pytest

import rustorch_amd as ra
from rustorch_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "rt_attn.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(rt_[a-z0-9_]+)\s*\(", header))
    assert declared == set(L.SYMBOLS), declared ^ set(L.SYMBOLS)
    lib = L.lib()
    for name in declared:
        assert getattr(lib, name) is not None
    assert b"gfx950" in lib.rt_version()
    assert L.status_name(2) == "BufferShapeMismatch"


def test_flash_errors_before_any_device_use():
    e = np.zeros(0, dtype=np.float32)
    with pytest.raises(ra.ZeroDim):
        ra.flash_forward(ra.AttentionShape.new(1, 1, 4, 0), np.zeros(3, np.float32), e, e)
    shape = ra.AttentionShape.new(1, 1, 4, 8)
    good, bad = np.zeros(32, np.float32), np.zeros(16, np.float32)
    for args, which in (((bad, bad, bad), "q"), ((good, bad, bad), "k"), ((good, good, bad), "v")):
        with pytest.raises(ra.BufferShapeMismatch) as ei:
            ra.flash_forward(shape, *args)
        assert (ei.value.which, ei.value.expected, ei.value.got) == (which, 32, 16)
        assert str(ei.value) == f"{which} buffer has 16 elements, expected 32"
    with pytest.raises(ra.OutputShapeMismatch) as ei:
        ra.flash_forward(shape, good, good, good, out=np.zeros(31, np.float32))
    assert (ei.value.expected, ei.value.got) == (32, 31)
    with pytest.raises(ra.PaddingLengthMismatch) as ei:
        ra.flash_forward_masked(ra.AttentionShape.new(1, 1, 4, 4), bad, bad, bad, ra.Mask.padding([True] * 3))
    assert (ei.value.expected, ei.value.got) == (4, 3)
    # seq == 0 is Ok and needs no device (cpu_forward.rs:203-206)
    assert ra.flash_forward(ra.AttentionShape.new(2, 4, 0, 16), e, e, e).size == 0


def test_gqa_errors_before_any_device_use():
    z = lambda n: np.zeros(n, dtype=np.float32)
    with pytest.raises(ra.HeadCountMismatch) as ei:
        ra.gqa_forward_f32(z(20), z(8), z(8), z(20), 1, 5, 2, 1, 1, 4)
    assert (ei.value.n_heads, ei.value.n_kv_heads) == (5, 2)
    with pytest.raises(ra.HeadCountMismatch):
        ra.gqa_forward_f32(z(20), z(8), z(8), z(20), 1, 4, 0, 1, 1, 4)
    for args, which, exp, got in (((z(7), z(8), z(8), z(16)), "q", 16, 7), ((z(16), z(9), z(8), z(16)), "k", 8, 9),
                                  ((z(16), z(8), z(9), z(16)), "v", 8, 9), ((z(16), z(8), z(8), z(15)), "out", 16, 15)):
        with pytest.raises(ra.WrongInputLen) as ei:
            ra.gqa_forward_f32(*args, 1, 4, 2, 1, 1, 4)
        assert (ei.value.which, ei.value.expected, ei.value.got) == (which, exp, got)


def test_decode_argument_errors_before_any_device_use():
    K = ra.LlmKernels()
    with pytest.raises(ra.HeadCountMismatch):
        K.gqa_decode_online_bf16(None, 1, 1, 1, 1, 5, 2, 4, 8, 16)
    with pytest.raises(ra.Overflow):
        K.gqa_decode_online_bf16(None, 1, 1, 1, 1, 4, 2, 17, 8, 16)
    with pytest.raises(ra.Overflow):
        K.kv_append_bf16(None, 1, 1, 1, 1, 16, 2, 8, 16)
    assert K.gqa_decode_workspace_bytes(64, 32, 8, 128, 8192) > 0


def test_mask_helper_matches_reference_rule():
    m = ra.Mask.padding([True, False, True, True, False])
    assert [m.is_masked(0, j) for j in range(5)] == [False, True, False, False, True]
    assert not m.is_masked(0, 9)
    assert ra.Mask.causal().is_masked(2, 3) and not ra.Mask.causal().is_masked(2, 2)
    assert not ra.Mask.none().is_masked(0, 5)


def test_no_device_is_reported_not_hidden():
    """Without a GPU a compute call must fail with NoDeviceFound, never fall back to the CPU."""
    import ctypes as C
    err = L.RtErr()
    if L.lib().rt_init(0, C.byref(err)) == 0:
        pytest.skip("a gfx950 device is present")
    shape = ra.AttentionShape.new(1, 1, 4, 8)
    z = np.zeros(32, np.float32)
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_forward(shape, z, z, z)
    assert ei.value.status == L.RT_ERR_NO_DEVICE


def test_bf16_prefill_argument_errors_before_any_device_use():
    """Head dims above 512 are refused by the host checks; everything else reaches the device lookup."""
    import ctypes as C
    lib = L.lib()

    def call(fn, b, h, n, d, q=0x1000, k=0x2000, v=0x3000, o=0x4000):
        err = L.RtErr()
        s = ra.AttentionShape.new(b, h, n, d)._c()
        return fn(None, C.byref(s), 0, q, k, v, 1, None, o, C.byref(err)), err

    for d in (513, 1000):  # above what any kernel covers
        rc, err = call(lib.rt_flash_forward_bf16_dev, 1, 1, 8, d)
        assert rc == L.RT_ERR_UNSUPPORTED and err.expected == 512
    # head dims that are not a multiple of 8, and tensors that are not 16-byte aligned, are served (by the
    # one-workgroup-per-row kernel): without a GPU the call gets as far as looking for one
    for d, q in ((100, 0x1000), (264, 0x1000), (4, 0x1000), (128, 0x1008)):
        rc, err = call(lib.rt_flash_forward_bf16_dev, 1, 1, 8, d, q=q)
        assert rc in (L.RT_ERR_NO_DEVICE, L.RT_OK)
    rc, err = call(lib.rt_flash_forward_bf16_dev, 1, 1, 8, 0)
    assert rc == L.RT_ERR_ZERO_DIM
    rc, err = call(lib.rt_flash_forward_bf16_dev, 1, 1, 0, 128, q=None)  # seq == 0: Ok, nothing touched
    assert rc == L.RT_OK


def test_prepare_and_cache_argument_errors_before_any_device_use():
    import ctypes as C
    lib = L.lib()
    err = L.RtErr()
    p = 0x1000  # never dereferenced: every call below fails (or returns) in the host checks

    def prepare(pos, table_rows, batch, seq, hq, hkv, d, max_seq, positions=None):
        return lib.rt_qk_norm_rope_kv_append_bf16(None, p, p, p, p, p, positions, pos, None, None, 1e-6, p, p,
                                                  table_rows, batch, seq, hq, hkv, d, max_seq, C.byref(err))

    assert prepare(16, 16, 1, 1, 1, 1, 8, 32) == L.RT_ERR_ROPE_POSITION_OVERFLOW and (err.expected, err.got) == (16, 17)
    assert prepare(12, 16, 1, 5, 1, 1, 8, 32) == L.RT_ERR_ROPE_POSITION_OVERFLOW and (err.expected, err.got) == (16, 17)
    assert prepare(4, 16, 1, 1, 1, 1, 8, 4) == L.RT_ERR_KV_OVERFLOW and (err.expected, err.got) == (4, 5)
    assert prepare(-1, 16, 1, 1, 1, 1, 8, 4) == L.RT_ERR_ROPE_POSITION_OVERFLOW
    assert prepare(0, 16, 1, 1, 1, 1, 7, 4) == L.RT_ERR_UNSUPPORTED
    assert prepare(0, 16, 1, 1, 1, 1, 514, 4) == L.RT_ERR_UNSUPPORTED
    assert prepare(0, 16, 0, 1, 1, 1, 8, 4) == L.RT_OK  # empty batch
    assert prepare(0, 16, 1, 0, 1, 1, 8, 4) == L.RT_OK  # no new token

    def append(cur, add, nk, nv, elem=2, batch=1, heads=2, max_seq=8, d=4):
        return lib.rt_kv_cache_append_dev(None, p, p, p, nk, p, nv, batch, heads, max_seq, d, cur, add, elem, C.byref(err))

    assert append(7, 2, 16, 16) == L.RT_ERR_KV_OVERFLOW and (err.expected, err.got) == (8, 9)
    assert append(0, 2, 15, 16) == L.RT_ERR_KV_WRONG_INPUT_LEN and (err.expected, err.got, err.got2) == (16, 15, 16)
    assert append(7, 2, 15, 16) == L.RT_ERR_KV_OVERFLOW  # the overflow is checked first (kv_cache.rs:84-97)
    assert append(0, 2, 16, 16, elem=3) == L.RT_ERR_UNSUPPORTED
    assert append(0, 0, 0, 0) == L.RT_OK
    assert lib.rt_buf_zero(None, 0, None, C.byref(err)) == L.RT_OK
    assert lib.rt_buf_zero(None, 16, None, C.byref(err)) == L.RT_ERR_NULL_POINTER
    assert lib.rt_buf_zero(p, 6, None, C.byref(err)) == L.RT_ERR_UNSUPPORTED
    assert L.status_name(L.RT_ERR_ROPE_POSITION_OVERFLOW) == "PositionOverflow"


def test_backward_errors_before_any_device_use():
    """cpu_backward.rs:59-77: q, k, v, "do" lengths in that order, then the three outputs (got = the longest);
    seq == 0 is Ok; none of this needs a device (cpu_backward.rs:252-278)."""
    import ctypes as C
    shape = ra.AttentionShape.new(1, 1, 4, 4)
    good, bad = np.zeros(16, np.float32), np.zeros(10, np.float32)
    for pos, name in enumerate(("q", "k", "v", "do")):
        args = [good] * pos + [bad] * (4 - pos)
        with pytest.raises(ra.BufferShapeMismatch) as ei:
            ra.flash_backward(shape, *args, dq=np.zeros(3, np.float32))
        assert (ei.value.which, ei.value.expected, ei.value.got) == (name, 16, 10)
    with pytest.raises(ra.OutputShapeMismatch) as ei:
        ra.flash_backward(shape, good, good, good, good, dq=np.zeros(16, np.float32), dk=np.zeros(20, np.float32),
                          dv=np.zeros(7, np.float32))
    assert (ei.value.expected, ei.value.got) == (16, 20)
    e = np.zeros(0, dtype=np.float32)
    dq, dk, dv = ra.flash_backward(ra.AttentionShape.new(1, 1, 0, 4), e, e, e, e)
    assert dq.size == 0 and dk.size == 0 and dv.size == 0
    # the device entry refuses a workspace that is too small before it looks for a device
    s = shape._c()
    need = L.lib().rt_flash_backward_workspace_bytes(C.byref(s))
    assert need == 1 * 1 * 4 * (4 + 2) * 4
    err = L.RtErr()
    rc = L.lib().rt_flash_backward_f32_dev(None, C.byref(s), 16, 16, 16, 16, 16, 16, 16, 16, need - 1, C.byref(err))
    assert rc == L.RT_ERR_WORKSPACE_TOO_SMALL and (err.expected, err.got) == (need, need - 1)


def test_saved_backward_argument_errors_before_any_device_use():
    import ctypes as C
    s = ra.AttentionShape.new(2, 3, 5, 8)._c()
    err = L.RtErr()
    need = 2 * 3 * 5 * 4
    rc = L.lib().rt_flash_backward_saved_f32_dev(None, C.byref(s), *([16] * 9), 16, need - 4, C.byref(err))
    assert rc == L.RT_ERR_WORKSPACE_TOO_SMALL and (err.expected, err.got) == (need, need - 4)
    rc = L.lib().rt_flash_backward_saved_f32_dev(None, C.byref(s), 16, 16, 16, None, 16, 16, 16, 16, 16, 16, need,
                                                 C.byref(err))
    assert rc == L.RT_ERR_NULL_POINTER
    z = ra.AttentionShape.new(1, 1, 4, 0)._c()
    assert L.lib().rt_flash_forward_stats_f32_dev(None, C.byref(z), 16, 16, 16, 16, 16, C.byref(err)) == L.RT_ERR_ZERO_DIM
    e = ra.AttentionShape.new(1, 1, 0, 4)._c()  # nothing to do: Ok without a device
    assert L.lib().rt_flash_forward_stats_f32_dev(None, C.byref(e), 16, 16, 16, 16, 16, C.byref(err)) == L.RT_OK


def test_stream_create_reports_a_missing_device():
    import ctypes as C
    err = L.RtErr()
    if L.lib().rt_init(0, C.byref(err)) == 0:
        s = ra.Stream()
        s.synchronize()
        s.destroy()
        return
    with pytest.raises(ra.DeviceError) as ei:
        ra.Stream()
    assert ei.value.status == L.RT_ERR_NO_DEVICE
    assert L.lib().rt_stream_destroy(None, C.byref(err)) == L.RT_OK


def test_shutdown_without_a_device_is_a_no_op():
    ra.shutdown()
    ra.shutdown()


def test_window_entries_argument_errors_before_any_device_use():
    lib = L.lib()
    err = L.RtErr()
    import ctypes as C
    p = 0x1000
    s = ra.AttentionShape.new(1, 2, 16, 64)._c()
    for fn in (lib.rt_flash_forward_window_bf16_dev, lib.rt_flash_forward_window_bnhd_bf16_dev):
        assert fn(None, C.byref(s), 0, p, p, p, 0, p, C.byref(err)) == L.RT_ERR_UNSUPPORTED and err.expected == 1
        assert fn(None, C.byref(s), 3, p, p, p, 4, p, C.byref(err)) == L.RT_ERR_HEAD_COUNT_MISMATCH
        assert fn(None, C.byref(s), 0, None, p, p, 4, p, C.byref(err)) == L.RT_ERR_NULL_POINTER
        assert fn(None, C.byref(s), 0, p + 2, p, p, 4, p, C.byref(err)) == L.RT_ERR_UNSUPPORTED
        s20 = ra.AttentionShape.new(1, 2, 16, 20)._c()
        assert fn(None, C.byref(s20), 0, p, p, p, 4, p, C.byref(err)) == L.RT_ERR_UNSUPPORTED
        s0 = ra.AttentionShape.new(1, 2, 16, 0)._c()
        assert fn(None, C.byref(s0), 0, p, p, p, 4, p, C.byref(err)) == L.RT_ERR_ZERO_DIM
        assert fn(None, C.byref(s), 0, p, p, p, 4, p, C.byref(err)) in (L.RT_ERR_NO_DEVICE, L.RT_OK)


def test_process_wide_switches_need_no_device():
    lib = L.lib()
    assert lib.rt_set_strict_non_finite_v(1) == 0 and lib.rt_set_strict_non_finite_v(0) == 1
    assert lib.rt_set_strict_non_finite_v(0) == 0
    assert lib.rt_debug_force_bf16_prefill_kernel(7) == L.RT_ERR_UNSUPPORTED
    assert lib.rt_debug_force_bf16_prefill_kernel(0) == L.RT_OK


def test_general_bf16_entries_argument_errors_before_any_device_use():
    """rt_mha_forward_masked_bf16_dev, rt_gqa_decode_chunk_bf16 and rt_gqa_decode_batched_bf16_noalloc refuse bad
    arguments in the host checks (the pointers below are never dereferenced)."""
    import ctypes as C
    lib = L.lib()
    err = L.RtErr()
    p = 0x1000
    assert lib.rt_mha_forward_masked_bf16_dev(None, p, p, p, None, 0, p, 1, 4, 4, 2, 0, C.byref(err)) == L.RT_ERR_ZERO_DIM
    rc = lib.rt_mha_forward_masked_bf16_dev(None, p, p, p, p, 15, p, 1, 4, 4, 2, 16, C.byref(err))
    assert rc == L.RT_ERR_WRONG_INPUT_LEN and err.which == 5 and (err.expected, err.got) == (16, 15)
    assert lib.rt_mha_forward_masked_bf16_dev(None, p, p, p, None, 0, p, 1, 4, 4, 2, 520, C.byref(err)) == L.RT_ERR_UNSUPPORTED
    # a q that is only 2-byte aligned is served by the row kernel: the call gets as far as looking for a device
    assert lib.rt_mha_forward_masked_bf16_dev(None, p + 2, p, p, None, 0, p, 1, 4, 4, 2, 16, C.byref(err)) in (L.RT_ERR_NO_DEVICE, L.RT_OK)
    assert lib.rt_mha_forward_masked_bf16_dev(None, None, p, p, None, 0, p, 1, 4, 4, 2, 16, C.byref(err)) == L.RT_ERR_NULL_POINTER
    assert lib.rt_mha_forward_masked_bf16_dev(None, None, None, None, None, 0, None, 0, 4, 4, 2, 16, C.byref(err)) == L.RT_OK

    def chunk(kv_lens, kv_len, batch, s, hq, hkv, d, max_seq, q=p):
        return lib.rt_gqa_decode_chunk_bf16(None, q, p, p, p, kv_lens, kv_len, batch, s, hq, hkv, d, max_seq, C.byref(err))

    assert chunk(None, 8, 1, 4, 8, 3, 64, 16) == L.RT_ERR_HEAD_COUNT_MISMATCH
    assert chunk(None, 8, 1, 4, 8, 2, 0, 16) == L.RT_ERR_ZERO_DIM
    assert chunk(None, 3, 1, 4, 8, 2, 64, 16) == L.RT_ERR_KV_OVERFLOW   # fewer keys than new positions
    assert chunk(None, 17, 1, 4, 8, 2, 64, 16) == L.RT_ERR_KV_OVERFLOW  # more keys than the cache holds
    assert chunk(None, 8, 1, 4, 8, 2, 20, 16) == L.RT_ERR_UNSUPPORTED
    assert chunk(None, 8, 1, 4, 8, 2, 64, 16, q=p + 2) == L.RT_ERR_UNSUPPORTED
    assert chunk(None, 8, 1, 0, 8, 2, 64, 16) == L.RT_OK  # no new position: nothing to do
    assert chunk(None, 8, 1, 4, 8, 2, 64, 16, q=None) == L.RT_ERR_NULL_POINTER

    def noalloc(batch, hq, hkv, d, max_seq, lens=p, q=p):
        return lib.rt_gqa_decode_batched_bf16_noalloc(None, q, p, p, p, lens, batch, hq, hkv, d, max_seq, C.byref(err))

    assert noalloc(2, 8, 3, 128, 16) == L.RT_ERR_HEAD_COUNT_MISMATCH
    assert noalloc(2, 8, 2, 0, 16) == L.RT_ERR_ZERO_DIM
    assert noalloc(2, 8, 2, 128, 16, lens=None) == L.RT_ERR_NULL_POINTER
    assert noalloc(0, 8, 2, 128, 16) == L.RT_OK
