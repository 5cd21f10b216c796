"""Sliding-window causal attention without the mask tensor (rt_flash_forward_window[_bnhd]_bf16_dev) against the
oracle's composed MultiHeadAttention path fed with sliding_window_mask (crates/rustorch-nn/src/masks.rs:41-60,
attention.rs:371-399), and against this library's own additive-mask entry on the same inputs."""
import numpy as np
import pytest

import rustorch_amd as ra
from _gpu import assert_bf16_parity, bf16_round, dev
from _util import seeded_normal

pytestmark = pytest.mark.gpu


def to_bhnd(x, b, n, h, d):
    return np.ascontiguousarray(x.reshape(b, n, h, d).transpose(0, 2, 1, 3)).ravel()


def window_bnhd(oracle, b, n, h, hkv, d, window, seed):
    qb, qf = bf16_round(seeded_normal((b, n, h, d), seed).ravel())
    kb, kf = bf16_round(seeded_normal((b, n, hkv, d), seed + 1).ravel())
    vb, vf = bf16_round(seeded_normal((b, n, hkv, d), seed + 2).ravel())
    out = ra.HipStorage(b * n * h * d * 2)
    out.upload(np.full(b * n * h * d, 0x7B7B, dtype=np.uint16))
    dq, dk, dv = dev(qb), dev(kb), dev(vb)
    ra.flash_forward_window_bf16_dev(ra.AttentionShape.new(b, h, n, d), dq, dk, dv, out, window, n_kv_heads=hkv, bnhd=True)
    ra.synchronize()
    got = oracle.bf16_to_f32(out.download(np.uint16))
    g = h // hkv
    k_rep = np.repeat(kf.reshape(b, n, hkv, d), g, axis=2).ravel()
    v_rep = np.repeat(vf.reshape(b, n, hkv, d), g, axis=2).ravel()
    want = oracle.mha_forward_masked(qf, k_rep, v_rep, b, n, n, h, d, attn_mask=oracle.sliding_window_mask(n, window))
    return got, want, (qb, k_rep, v_rep)


@pytest.mark.parametrize("b,n,h,hkv,d", [(2, 300, 4, 4, 64), (1, 1000, 4, 2, 128), (2, 129, 2, 1, 32), (1, 700, 2, 2, 96),
                                         (1, 260, 2, 2, 256), (1, 64, 3, 3, 8)])
@pytest.mark.parametrize("window", [1, 2, 33, 64, 65, 128, 200, 5000])
def test_window_matches_the_masked_path_of_multi_head_attention(oracle, b, n, h, hkv, d, window):
    got, want, _ = window_bnhd(oracle, b, n, h, hkv, d, window, 7 * window + n)
    assert_bf16_parity(got.reshape(b, n, h * d), want.reshape(b, n, h * d), h * d, None, f"window {window}", block_rows=64)


def test_window_of_one_is_v_and_a_window_of_the_sequence_is_the_causal_mask(oracle):
    b, n, h, d = 1, 200, 2, 64
    got, want, (qb, k_rep, v_rep) = window_bnhd(oracle, b, n, h, h, d, 1, 3)
    vb, _ = bf16_round(seeded_normal((b, n, h, d), 5).ravel())
    assert np.array_equal(oracle.f32_to_bf16(got), vb)  # softmax over one key is 1: the row is V's, bit for bit
    # window >= n: the same bits as the causal mask through the plain entry
    (q4, _), (k4, _), (v4, _) = (bf16_round(seeded_normal((b, h, n, d), s).ravel()) for s in (11, 12, 13))
    shape = ra.AttentionShape.new(b, h, n, d)
    outs = []
    for win in (n, 10 * n, None):
        o = ra.HipStorage(b * h * n * d * 2)
        dq, dk, dv = dev(q4), dev(k4), dev(v4)
        if win is None:
            ra.debug_force_bf16_prefill_kernel("tile")
            try:
                ra.flash_forward_bf16_dev(shape, dq, dk, dv, o, ra.Mask.causal())
            finally:
                ra.debug_force_bf16_prefill_kernel("auto")
        else:
            ra.flash_forward_window_bf16_dev(shape, dq, dk, dv, o, win)
        ra.synchronize()
        outs.append(o.download(np.uint16))
    assert np.array_equal(outs[0], outs[2]) and np.array_equal(outs[1], outs[2])


def test_window_on_a_long_sequence_agrees_with_the_additive_mask_entry(oracle):
    """T = 4096, window 256, [B,T,H*hd] tensors: the entry that walks window + 128 keys per query tile against the one
    that is handed the 64 MB mask and scores every pair.  Also one (batch, head) slab against the oracle."""
    b, n, h, d, window = 1, 4096, 4, 64, 256
    qb, qf = bf16_round(seeded_normal((b, n, h, d), 21).ravel())
    kb, kf = bf16_round(seeded_normal((b, n, h, d), 22).ravel())
    vb, vf = bf16_round(seeded_normal((b, n, h, d), 23).ravel())
    dq, dk, dv = dev(qb), dev(kb), dev(vb)
    o_win, o_mask = ra.HipStorage(b * n * h * d * 2), ra.HipStorage(b * n * h * d * 2)
    ra.flash_forward_window_bf16_dev(ra.AttentionShape.new(b, h, n, d), dq, dk, dv, o_win, window, bnhd=True)
    mask = ra.masks.sliding_window_mask(n, window).astype(np.float32)
    dm = dev(mask.ravel())
    ra.mha_forward_masked_bf16_dev(dq, dk, dv, o_mask, b, n, n, h, d, attn_mask=dm, mask_len=n * n)
    ra.synchronize()
    got_w, got_m = oracle.bf16_to_f32(o_win.download(np.uint16)), oracle.bf16_to_f32(o_mask.download(np.uint16))
    assert np.abs(got_w - got_m).max() <= 2 ** -6  # two bf16 roundings of values below 4
    head = 2
    q1, k1, v1 = (x.reshape(b, n, h, d)[0, :, head] for x in (qf, kf, vf))
    want = oracle.mha_forward_masked(q1, k1, v1, 1, n, n, 1, d, attn_mask=oracle.sliding_window_mask(n, window))
    assert_bf16_parity(got_w.reshape(n, h, d)[:, head], want.reshape(n, d), d, None, "slab of head 2")


def test_window_errors():
    shape = ra.AttentionShape.new(1, 2, 16, 64)
    z = ra.HipStorage(1 << 16)
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_forward_window_bf16_dev(shape, z, z, z, z, 0)
    assert ei.value.status == 21 and ei.value.expected == 1  # window must be >= 1
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_forward_window_bf16_dev(ra.AttentionShape.new(1, 2, 16, 20), z, z, z, z, 4)
    assert ei.value.status == 21
    with pytest.raises(ra.DeviceError) as ei:
        ra.flash_forward_window_bf16_dev(shape, z.ptr + 2, z, z, z, 4)
    assert ei.value.status == 21
