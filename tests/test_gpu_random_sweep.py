"""Randomised parity sweep through the C ABI: shapes, masks, layouts and head groupings drawn from a seed, every
case compared with the oracle (f32 max-abs <= 1e-5; bf16 max-abs <= 2e-2 and relative Frobenius error <= 1e-2 per
block of 256 rows, per row for decode; NaN patterns exact).  Sizes are kept small so
that the oracle answers in milliseconds; the full-size cases live in the other GPU test files."""
import numpy as np
import pytest

import rustorch_amd as ra

pytestmark = pytest.mark.gpu


def _bf(oracle, x):
    return oracle.f32_to_bf16(np.asarray(x, dtype=np.float32))


def _compare(name, got, want, tol):
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{name}: NaN pattern differs"
    if np.isfinite(want).any():
        err = float(np.nanmax(np.abs(got - want)))
        assert err <= tol, f"{name}: max-abs {err} > {tol}"


def _compare_bf16(oracle, name, got, want, dim, slab_rows=None, **blocks):
    _compare(name, got, want, oracle.BF16_MAX_ABS)
    rel = oracle.rel_fro_blocks(got, want, dim, slab_rows, **blocks)
    assert rel <= oracle.BF16_REL_FRO, f"{name}: relative Frobenius error {rel:.3e}"


def _mask(rng, n):
    kind = int(rng.integers(0, 3))
    if kind == 0:
        return ra.Mask.none(), None, None
    if kind == 1:
        return ra.Mask.causal(), "causal", None
    keep = rng.random(n) > 0.3
    keep[int(rng.integers(0, n))] = True
    return ra.Mask.padding(keep), ("padding", keep), keep


def _bf16_prefill(oracle, rng):
    b, hkv, g = int(rng.integers(1, 4)), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4]))
    h, n, d = hkv * g, int(rng.choice([1, 31, 64, 127, 128, 129, 255, 256, 257, 300, 511, 640, 777])), int(rng.choice([64, 128]))
    bnhd = bool(rng.integers(0, 2))
    qb = _bf(oracle, rng.standard_normal(b * h * n * d) * rng.choice([1.0, 2.0]))
    kb, vb = _bf(oracle, rng.standard_normal(b * hkv * n * d)), _bf(oracle, rng.standard_normal(b * hkv * n * d))
    m, om, keep = _mask(rng, n)
    kf = np.repeat(oracle.bf16_to_f32(kb).reshape(b, hkv, n, d), g, axis=1).ravel()
    vf = np.repeat(oracle.bf16_to_f32(vb).reshape(b, hkv, n, d), g, axis=1).ravel()
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), oracle.bf16_to_f32(qb), kf, vf, om)
    if bnhd:
        def tr(x, hh):
            return np.ascontiguousarray(x.reshape(b, hh, n, d).transpose(0, 2, 1, 3)).ravel()
        qb, kb, vb = tr(qb, h), tr(kb, hkv), tr(vb, hkv)
    dq, dk, dv = (ra.HipStorage.from_numpy(x) for x in (qb, kb, vb))
    do = ra.HipStorage(b * h * n * d * 2)
    kd = ra.HipStorage.from_numpy(keep.astype(np.uint8)) if keep is not None else None
    fn = ra.flash_forward_bnhd_bf16_dev if bnhd else ra.flash_forward_bf16_dev
    fn(ra.AttentionShape.new(b, h, n, d), dq, dk, dv, do, m, keep_dev=kd, n_kv_heads=hkv)
    ra.synchronize()
    got = oracle.bf16_to_f32(do.download(np.uint16))
    if bnhd:
        got = got.reshape(b, n, h, d).transpose(0, 2, 1, 3).ravel()
    _compare_bf16(oracle, f"bf16 prefill B{b} H{h}/{hkv} N{n} D{d} {m.kind} bnhd={bnhd}", got, want, d, n)


def _f32_prefill(oracle, rng):
    b, h = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    n, d = int(rng.choice([1, 5, 33, 64, 65, 100, 129, 200])), int(rng.choice([4, 8, 24, 32, 40, 64, 96, 128]))
    q, k, v = (rng.standard_normal(b * h * n * d).astype(np.float32) for _ in range(3))
    m, om, _ = _mask(rng, n)
    got = ra.flash_forward_masked(ra.AttentionShape.new(b, h, n, d), q, k, v, m)
    want = oracle.flash_forward_masked(oracle.AttentionShape(b, h, n, d), q, k, v, om)
    _compare(f"f32 prefill B{b} H{h} N{n} D{d} {m.kind}", got, want, 1e-5)


def _decode(oracle, rng):
    b, hkv, g = int(rng.integers(1, 9)), int(rng.choice([1, 2, 8])), int(rng.choice([1, 2, 4, 8]))
    hq, d, lmax = hkv * g, int(rng.choice([64, 128])), int(rng.choice([16, 100, 257, 1024]))
    lens = rng.integers(0, lmax + 1, size=b).astype(np.int32)
    kc, vc = _bf(oracle, rng.standard_normal(b * hkv * lmax * d)), _bf(oracle, rng.standard_normal(b * hkv * lmax * d))
    q = _bf(oracle, rng.standard_normal(b * hq * d))
    K = ra.LlmKernels()
    dq, dk, dv, dl = (ra.HipStorage.from_numpy(x) for x in (q, kc, vc, lens))
    do = ra.HipStorage(b * hq * d * 2)
    ws = ra.HipStorage(max(K.gqa_decode_workspace_bytes(b, hq, hkv, d, lmax), 256))
    K.gqa_decode_batched_bf16(None, dq, dk, dv, do, dl, b, hq, hkv, d, lmax, ws, ws.byte_len)
    ra.synchronize()
    want = oracle.gqa_decode_batched_bf16(q, kc, vc, lens, b, hq, hkv, d, lmax)
    _compare_bf16(oracle, f"decode B{b} Hq{hq}/{hkv} D{d} Lmax{lmax} lens={lens.tolist()}",
                  oracle.bf16_to_f32(do.download(np.uint16)), want, d, block_rows=1, min_elems=64)


def _varlen(oracle, rng):
    b, h, n, d = int(rng.integers(1, 5)), int(rng.choice([1, 2, 4])), int(rng.choice([64, 130, 256, 300, 513])), int(rng.choice([64, 128]))
    lens = rng.integers(1, n + 1, size=b).astype(np.int32)
    q, k, v = (_bf(oracle, rng.standard_normal(b * h * n * d)) for _ in range(3))
    dq, dk, dv, dl = (ra.HipStorage.from_numpy(x) for x in (q, k, v, lens))
    do = ra.HipStorage(b * h * n * d * 2)
    ra.flash_forward_varlen_bf16_dev(ra.AttentionShape.new(b, h, n, d), dq, dk, dv, dl, do, zero_padded_rows=True)
    ra.synchronize()
    want = oracle.varlen_causal_forward(oracle.bf16_to_f32(q), oracle.bf16_to_f32(k), oracle.bf16_to_f32(v), lens, b, h, n, d,
                                        zero_padded_rows=True)
    got = oracle.bf16_to_f32(do.download(np.uint16))
    _compare_bf16(oracle, f"varlen B{b} H{h} N{n} D{d} lens={lens.tolist()}", got, np.asarray(want, dtype=np.float32), d, n)
    # padded rows are exact zeros, not merely small
    pad = np.concatenate([np.arange(n)[None, :] >= lens[:, None]] * 1).reshape(b, 1, n, 1)
    assert not got.reshape(b, h, n, d)[np.broadcast_to(pad, (b, h, n, d))].any()


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_cases_match_oracle(oracle, seed):
    rng = np.random.default_rng(seed)
    cases = (_bf16_prefill, _f32_prefill, _decode, _varlen)
    for _ in range(60):
        cases[int(rng.integers(0, len(cases)))](oracle, rng)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_backward_cases_match_oracle(oracle, seed):
    """f32 backward on random shapes (every head dim class, ragged tails, single rows), inputs in (-1, 1) or N(0, 0.5);
    max-abs <= 2e-5 relative to gradients of order one."""
    rng = np.random.default_rng(seed)
    for _ in range(40):
        b, h = int(rng.integers(1, 3)), int(rng.integers(1, 10))
        n = int(rng.choice([1, 2, 5, 31, 32, 33, 64, 65, 100, 129, 200, 257]))
        d = int(rng.choice([1, 4, 8, 20, 24, 32, 40, 64, 72, 96, 100, 128]))
        size = b * h * n * d
        if rng.integers(0, 2):
            bufs = [rng.uniform(-1.0, 1.0, size).astype(np.float32) for _ in range(4)]
        else:
            bufs = [(rng.standard_normal(size) * 0.5).astype(np.float32) for _ in range(4)]
        got = ra.flash_backward(ra.AttentionShape.new(b, h, n, d), *bufs)
        want = oracle.flash_backward(oracle.AttentionShape(b, h, n, d), *bufs)
        for name, g, w in zip(("dq", "dk", "dv"), got, want):
            err = float(np.abs(g - w).max())
            assert np.isfinite(g).all() and err <= 2e-5 * max(1.0, float(np.abs(w).max())), \
                f"backward B{b} H{h} N{n} D{d} {name}: max-abs {err}"


@pytest.mark.parametrize("seed", [31, 32])
def test_random_mha_and_gqa_cases_match_oracle(oracle, seed):
    """The masked / cross-attention core and gqa_forward_f32 on random shapes: self and cross lengths, head dims that
    are and are not multiples of 4 or 32 (the tiled kernel, its zero-padded form and the row kernel), shared and
    per-head additive masks, every grouping of query heads."""
    rng = np.random.default_rng(seed)
    for _ in range(100):
        b, h = int(rng.integers(1, 4)), int(rng.integers(1, 5))
        tq = int(rng.choice([1, 2, 7, 31, 32, 33, 64, 100, 129, 257]))
        tkv = tq if rng.random() < 0.4 else int(rng.choice([1, 3, 32, 33, 65, 128, 200, 300, 513]))
        d = int(rng.choice([1, 3, 4, 8, 12, 16, 20, 32, 40, 64, 80, 96, 100, 128, 132, 160]))
        q = rng.standard_normal(b * tq * h * d).astype(np.float32)
        k = rng.standard_normal(b * tkv * h * d).astype(np.float32)
        v = rng.standard_normal(b * tkv * h * d).astype(np.float32)
        kind = int(rng.integers(0, 4))
        mask = None
        if kind == 1:
            mask = np.where(rng.random((tq, tkv)) > 0.3, 0.0, -1.0e4).astype(np.float32)
        elif kind == 2:
            mask = rng.standard_normal((b * h, tq, tkv)).astype(np.float32)
        elif kind == 3 and tq == tkv:
            mask = ra.causal_mask(tq)
        got = ra.mha_forward_masked_f32(q, k, v, b, tq, tkv, h, d, mask)
        want = oracle.mha_forward_masked(q, k, v, b, tq, tkv, h, d, mask)
        _compare(f"mha B{b} Tq{tq} Tkv{tkv} H{h} D{d} mask{kind}", got, want, 1e-5)
        hkv = int(rng.choice([x for x in (1, 2, 4) if h % x == 0]))
        kk = rng.standard_normal(b * hkv * tkv * d).astype(np.float32)
        vv = rng.standard_normal(b * hkv * tkv * d).astype(np.float32)
        out = np.zeros(b * h * tq * d, dtype=np.float32)
        ra.gqa_forward_f32(q, kk, vv, out, b, h, hkv, tq, tkv, d)
        _compare(f"gqa B{b} H{h}/{hkv} Sq{tq} Skv{tkv} D{d}", out, oracle.gqa_forward_f32(q, kk, vv, b, h, hkv, tq, tkv, d), 1e-5)


def _window(oracle, rng):
    """rt_flash_forward_window_bnhd_bf16_dev against MultiHeadAttention's masked path with sliding_window_mask."""
    b = int(rng.integers(1, 3))
    hkv = int(rng.choice([1, 2]))
    g = int(rng.choice([1, 2, 4]))
    h = hkv * g
    n = int(rng.choice([1, 33, 64, 65, 127, 200, 257, 500, 900]))
    d = int(rng.choice([32, 64, 96, 128]))
    w = int(rng.choice([1, 2, 31, 64, 65, 100, 300, 2000]))
    q, k, v = (_bf(oracle, rng.standard_normal(x)) for x in (b * n * h * d, b * n * hkv * d, b * n * hkv * d))
    out = ra.HipStorage(b * n * h * d * 2)
    dq, dk, dv = (ra.HipStorage.from_numpy(x) for x in (q, k, v))
    ra.flash_forward_window_bf16_dev(ra.AttentionShape.new(b, h, n, d), dq, dk, dv, out, w, n_kv_heads=hkv, bnhd=True)
    ra.synchronize()
    got = oracle.bf16_to_f32(out.download(np.uint16))
    kf = np.repeat(oracle.bf16_to_f32(k).reshape(b, n, hkv, d), g, axis=2).ravel()
    vf = np.repeat(oracle.bf16_to_f32(v).reshape(b, n, hkv, d), g, axis=2).ravel()
    want = oracle.mha_forward_masked(oracle.bf16_to_f32(q), kf, vf, b, n, n, h, d, attn_mask=oracle.sliding_window_mask(n, w))
    _compare(f"window B{b} T{n} H{h}/{hkv} D{d} w{w}", got, np.asarray(want, dtype=np.float32).ravel(), oracle.BF16_MAX_ABS)


def _chunk_decode(oracle, rng):
    """rt_gqa_decode_chunk_bf16 on every grouping (one head per kv head included), caches short and long enough for
    spans, sequences shorter than the chunk and empty ones."""
    b = int(rng.integers(1, 4))
    hkv = int(rng.choice([1, 2, 8]))
    g = int(rng.choice([1, 2, 4]))
    hq = hkv * g
    d = int(rng.choice([64, 96, 128]))
    max_seq = int(rng.choice([64, 300, 1100, 4000]))
    s = int(rng.choice([1, 3, 8, 16, 40]))
    lens = [int(rng.integers(0, max_seq + 1)) for _ in range(b)]
    if rng.random() < 0.3:
        lens[0] = int(rng.integers(0, s + 1))  # fewer keys than new positions
    q, k, v = (_bf(oracle, rng.standard_normal(x)) for x in (b * s * hq * d, b * hkv * max_seq * d, b * hkv * max_seq * d))
    out = ra.HipStorage(q.size * 2)
    dq, dk, dv, dl = (ra.HipStorage.from_numpy(x) for x in (q, k, v, np.asarray(lens, dtype=np.int32)))
    ra.LlmKernels().gqa_decode_chunk_bf16(None, dq, dk, dv, out, dl, b, s, hq, hkv, d, max_seq)
    ra.synchronize()
    got = oracle.bf16_to_f32(out.download(np.uint16))
    want = oracle.gqa_decode_chunk_bf16(q, k, v, lens, b, s, hq, hkv, d, max_seq)
    _compare(f"chunk B{b} S{s} H{hq}/{hkv} D{d} max{max_seq} lens={lens}", got, np.asarray(want, dtype=np.float32).ravel(),
             oracle.BF16_MAX_ABS)


def _masked_bf16(oracle, rng):
    """rt_mha_forward_masked_bf16_dev: self and cross lengths, shared and per-head additive masks."""
    b, h = int(rng.integers(1, 3)), int(rng.integers(1, 5))
    tq = int(rng.choice([1, 7, 32, 33, 64, 100, 129, 257]))
    tkv = tq if rng.random() < 0.4 else int(rng.choice([1, 3, 32, 65, 128, 200, 513]))
    d = int(rng.choice([8, 16, 32, 40, 64, 96, 128, 256]))
    q, k, v = (_bf(oracle, rng.standard_normal(x)) for x in (b * tq * h * d, b * tkv * h * d, b * tkv * h * d))
    kind = int(rng.integers(0, 3))
    mask = None
    if kind == 1:
        mask = np.where(rng.random((tq, tkv)) > 0.3, 0.0, -1.0e4).astype(np.float32)
    elif kind == 2:
        mask = rng.standard_normal((b * h, tq, tkv)).astype(np.float32)
    out = ra.HipStorage(b * tq * h * d * 2)
    dq, dk, dv = (ra.HipStorage.from_numpy(x) for x in (q, k, v))
    dm = ra.HipStorage.from_numpy(mask.ravel()) if mask is not None else None
    ra.mha_forward_masked_bf16_dev(dq, dk, dv, out, b, tq, tkv, h, d, attn_mask=dm, mask_len=0 if mask is None else mask.size)
    ra.synchronize()
    got = oracle.bf16_to_f32(out.download(np.uint16))
    want = oracle.mha_forward_masked(oracle.bf16_to_f32(q), oracle.bf16_to_f32(k), oracle.bf16_to_f32(v), b, tq, tkv, h, d, mask)
    _compare(f"masked bf16 B{b} Tq{tq} Tkv{tkv} H{h} D{d} mask{kind}", got, np.asarray(want, dtype=np.float32).ravel(),
             oracle.BF16_MAX_ABS)


@pytest.mark.parametrize("seed", [41, 42, 43])
def test_random_window_chunk_and_masked_bf16_cases_match_oracle(oracle, seed):
    rng = np.random.default_rng(seed)
    cases = (_window, _chunk_decode, _masked_bf16)
    for _ in range(60):
        cases[int(rng.integers(0, len(cases)))](oracle, rng)
