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
