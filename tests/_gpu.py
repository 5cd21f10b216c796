"""Helpers of the GPU parity tests: device buffers through the C ABI, bf16 bit patterns."""
import numpy as np

import rustorch_amd as ra
from oracle import attn_oracle as oracle


def bf16_round(x):
    """f32 array -> (bf16 bit patterns uint16, the same values as f32)."""
    bits = oracle.f32_to_bf16(np.asarray(x, dtype=np.float32))
    return bits, oracle.bf16_to_f32(bits)


def dev(a):
    return ra.HipStorage.from_numpy(np.ascontiguousarray(a))


def max_abs(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.max(np.abs(a - b))) if a.size else 0.0


def same_nan_pattern(a, b):
    return bool(np.array_equal(np.isnan(a), np.isnan(b)))


def assert_close_nan(got, want, tol, label=""):
    """NaN positions must coincide exactly; elsewhere max-abs <= tol."""
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, label
    assert same_nan_pattern(got, want), f"{label}: NaN pattern differs"
    ok = ~np.isnan(want)
    if ok.any():
        d = max_abs(got[ok], want[ok])
        assert d <= tol, f"{label}: max-abs {d:.3e} > {tol:.1e}"


def assert_bf16_parity(got, want, dim, slab_rows=None, label="", block_rows=256, min_elems=512):
    """The bar of every bf16 comparison with the oracle: NaN positions exact, max-abs <= 2e-2, and per block of 256
    rows of a (batch, head) slab a relative Frobenius error <= 1e-2 (a kernel that loses a 32-key item of a long
    row stays under the absolute bar and fails this one).  `slab_rows`: rows per (batch, head) pair; None takes the
    array as one slab.  Decode outputs: one block per (sequence, head) row, see assert_decode_parity."""
    assert_close_nan(got, want, oracle.BF16_MAX_ABS, label)
    rel = oracle.rel_fro_blocks(got, want, dim, slab_rows, block_rows, min_elems)
    assert rel <= oracle.BF16_REL_FRO, f"{label}: relative Frobenius error {rel:.3e} > {oracle.BF16_REL_FRO:.0e}"


def assert_decode_parity(got, want, dim, label=""):
    """Decode outputs [.., heads, dim]: the bf16 bar with one block per (sequence, head) row."""
    assert_bf16_parity(got, want, dim, None, label, block_rows=1, min_elems=64)


def flash_bf16(shape, q_bits, k_bits, v_bits, mask=None, n_kv_heads=0):
    """Run the bf16 device entry point on host bit-pattern arrays; returns f32 values of the bf16 output."""
    dq, dk, dv = dev(q_bits), dev(k_bits), dev(v_bits)
    n_out = shape.buffer_len()
    dout = ra.HipStorage(max(n_out, 1) * 2)
    dout.upload(np.full(max(n_out, 1), 0x7B7B, dtype=np.uint16))  # poison: every element must be written
    mask = mask or ra.Mask.none()
    dkeep = dev(mask.keep) if mask.keep is not None else None
    ra.flash_forward_bf16_dev(shape, dq, dk, dv, dout, mask, dkeep, n_kv_heads)
    ra.synchronize()
    return oracle.bf16_to_f32(dout.download(np.uint16, n_out))
