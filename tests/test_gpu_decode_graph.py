"""The decode inner loop of a token -- per layer: q/k RMSNorm + RoPE + cache append, then GQA decode over the cache
(crates/rustorch-llm/src/cuda_backend.rs:516-556) -- recorded into a HIP graph through the C ABI and replayed, every
replay compared with the oracle's composition of the same steps.

Two forms.  (1) The reference's own calls with the position as a host scalar (`rt_qk_norm_rope_kv_append_bf16` with
`pos`, `rt_gqa_decode_online_bf16` with `kv_len`), recorded as the FIRST work a fresh stream ever sees: the capture
runs in the mode that refuses device allocations, so it also shows that neither entry allocates.  (2) The same loop
with positions and context lengths kept on the device and advanced by `rt_i32_add_dev` at the end of the graph: one
graph serves token after token.  Between replays the test does eager work of its own (uploads of the next token's
inputs, downloads, synchronisations), and a graph must not contain a memset node."""
import ctypes as C

import numpy as np
import pytest

import rustorch_amd as ra
from rustorch_amd import _lib
from _gpu import assert_decode_parity

pytestmark = pytest.mark.gpu
K = ra.LlmKernels()

NODE_TYPE_MEMSET = 2  # hipGraphNodeTypeMemset


class Hip:
    def __init__(self):
        self.lib = _lib.hip_runtime()
        vp = C.c_void_p
        self.lib.hipStreamBeginCapture.argtypes = [vp, C.c_int]
        self.lib.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
        self.lib.hipGraphInstantiate.argtypes = [C.POINTER(vp), vp, C.POINTER(vp), C.c_char_p, C.c_size_t]
        self.lib.hipGraphLaunch.argtypes = [vp, vp]
        self.lib.hipGraphGetNodes.argtypes = [vp, C.POINTER(vp), C.POINTER(C.c_size_t)]
        self.lib.hipGraphNodeGetType.argtypes = [vp, C.POINTER(C.c_int)]
        self.lib.hipGraphExecDestroy.argtypes = [vp]
        self.lib.hipGraphDestroy.argtypes = [vp]

    def ok(self, rc, what):
        assert rc == 0, f"{what}: hipError {rc}"

    def capture(self, stream, record):
        """Runs `record()` under stream capture (global mode: an allocation anywhere in the process fails the
        capture) and returns (graph, executable graph, node types)."""
        self.ok(self.lib.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        try:
            record()
        finally:
            graph = C.c_void_p()
            rc = self.lib.hipStreamEndCapture(stream, C.byref(graph))
        self.ok(rc, "hipStreamEndCapture")
        n = C.c_size_t(0)
        self.ok(self.lib.hipGraphGetNodes(graph, None, C.byref(n)), "hipGraphGetNodes")
        nodes = (C.c_void_p * n.value)()
        self.ok(self.lib.hipGraphGetNodes(graph, nodes, C.byref(n)), "hipGraphGetNodes")
        types = []
        for node in nodes:
            t = C.c_int()
            self.ok(self.lib.hipGraphNodeGetType(node, C.byref(t)), "hipGraphNodeGetType")
            types.append(t.value)
        exe = C.c_void_p()
        self.ok(self.lib.hipGraphInstantiate(C.byref(exe), graph, None, None, 0), "hipGraphInstantiate")
        return graph, exe, types

    def launch(self, exe, stream):
        self.ok(self.lib.hipGraphLaunch(exe, stream), "hipGraphLaunch")

    def destroy(self, graph, exe):
        self.lib.hipGraphExecDestroy(exe)
        self.lib.hipGraphDestroy(graph)


def bf16(oracle, rng, n):
    return oracle.f32_to_bf16(rng.standard_normal(n).astype(np.float32))


class Layer:
    """Device and host state of one layer: caches, norm weights, and the token's q / k / v inputs."""

    def __init__(self, oracle, rng, b, hq, hkv, d, lmax):
        self.kc, self.vc = bf16(oracle, rng, b * hkv * lmax * d), bf16(oracle, rng, b * hkv * lmax * d)
        self.qg = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        self.kg = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        self.d_kc, self.d_vc = ra.HipStorage.from_numpy(self.kc), ra.HipStorage.from_numpy(self.vc)
        self.d_qg, self.d_kg = ra.HipStorage.from_numpy(self.qg), ra.HipStorage.from_numpy(self.kg)
        self.d_q, self.d_k, self.d_v = (ra.HipStorage(n * 2) for n in (b * hq * d, b * hkv * d, b * hkv * d))
        self.d_out = ra.HipStorage(b * hq * d * 2)

    def new_token(self, oracle, rng, b, hq, hkv, d):
        self.q, self.k, self.v = bf16(oracle, rng, b * hq * d), bf16(oracle, rng, b * hkv * d), bf16(oracle, rng, b * hkv * d)
        self.d_q.upload(self.q)  # the prepare step rewrites q in place: every token brings its own
        self.d_k.upload(self.k)
        self.d_v.upload(self.v)

    def expect(self, oracle, oro, positions, b, hq, hkv, d, lmax):
        """The CPU composition on the host copies of the caches (which advance with the device's)."""
        want_q = oracle.decode_prepare_bf16(self.q, self.k, self.v, self.kc, self.vc, positions, self.qg, self.kg, 1e-6,
                                            oro, b, hq, hkv, d, lmax)
        return oracle.gqa_decode_batched_bf16(want_q, self.kc, self.vc, np.asarray(positions) + 1, b, hq, hkv, d, lmax)


def ropes(oracle, d, lmax):
    rope = ra.RoPE(d, lmax)
    oro = oracle.RoPE(d, lmax)
    oro.cos, oro.sin = rope.cos.copy(), rope.sin.copy()
    rope.device_tables()  # uploaded before any capture starts
    return rope, oro


def test_reference_decode_calls_record_into_a_graph_on_a_fresh_stream(oracle):
    ra.init(0)
    hip = Hip()
    rng = np.random.default_rng(2027)
    hq, hkv, d, lmax, pos, n_layers = 32, 8, 128, 3000, 2500, 3
    rope, oro = ropes(oracle, d, lmax)
    layers = [Layer(oracle, rng, 1, hq, hkv, d, lmax) for _ in range(n_layers)]
    stream = ra.Stream()  # never used before: the first decode call on it happens under capture

    def record():
        for L in layers:
            K.qk_norm_rope_kv_append_bf16(stream.handle, L.d_q, L.d_k, L.d_v, L.d_kc, L.d_vc, pos, rope, 1, hq, hkv, d,
                                          lmax, q_gamma=L.d_qg, k_gamma=L.d_kg)
            K.gqa_decode_online_bf16(stream.handle, L.d_q, L.d_kc, L.d_vc, L.d_out, hq, hkv, pos + 1, d, lmax)

    graph, exe, types = hip.capture(stream.handle, record)
    assert len(types) == 3 * n_layers  # prepare, split, merge per layer
    assert NODE_TYPE_MEMSET not in types
    for replay in range(3):
        for L in layers:
            L.new_token(oracle, rng, 1, hq, hkv, d)
        ra.synchronize()
        hip.launch(exe, stream.handle)
        stream.synchronize()
        for i, L in enumerate(layers):
            want = L.expect(oracle, oro, [pos], 1, hq, hkv, d, lmax)
            got = oracle.bf16_to_f32(L.d_out.download(np.uint16))
            assert_decode_parity(got, want, d, f"replay {replay} layer {i}")
            assert np.array_equal(L.d_kc.download(np.uint16), L.kc), "cache row written by the graph"
    hip.destroy(graph, exe)
    stream.destroy()


def test_decode_loop_with_positions_on_the_device_replays_token_after_token(oracle):
    ra.init(0)
    hip = Hip()
    rng = np.random.default_rng(2028)
    b, hq, hkv, d, lmax, n_layers, n_tokens = 3, 32, 8, 128, 1200, 2, 5
    positions = np.array([1100, 0, 511], dtype=np.int32)
    rope, oro = ropes(oracle, d, lmax)
    layers = [Layer(oracle, rng, b, hq, hkv, d, lmax) for _ in range(n_layers)]
    d_pos = ra.HipStorage.from_numpy(positions)
    d_len = ra.HipStorage.from_numpy(positions + 1)
    stream = ra.Stream()

    def record():
        for L in layers:
            K.qk_norm_rope_kv_append_bf16(stream.handle, L.d_q, L.d_k, L.d_v, L.d_kc, L.d_vc, d_pos, rope, b, hq, hkv,
                                          d, lmax, q_gamma=L.d_qg, k_gamma=L.d_kg)
            K.gqa_decode_batched_bf16_noalloc(stream.handle, L.d_q, L.d_kc, L.d_vc, L.d_out, d_len, b, hq, hkv, d, lmax)
        ra.i32_add_dev(d_pos, b, 1, stream.handle)  # the next token's position and context length
        ra.i32_add_dev(d_len, b, 1, stream.handle)

    graph, exe, types = hip.capture(stream.handle, record)
    assert NODE_TYPE_MEMSET not in types and len(types) == 3 * n_layers + 2
    for token in range(n_tokens):
        for L in layers:
            L.new_token(oracle, rng, b, hq, hkv, d)
        ra.synchronize()
        hip.launch(exe, stream.handle)
        stream.synchronize()
        for i, L in enumerate(layers):
            want = L.expect(oracle, oro, positions + token, b, hq, hkv, d, lmax)
            got = oracle.bf16_to_f32(L.d_out.download(np.uint16))
            assert_decode_parity(got, want, d, f"token {token} layer {i}")
        assert np.array_equal(d_pos.download(np.int32), positions + token + 1)
    for L in layers:  # the caches hold what the CPU path appended, token after token
        assert np.array_equal(L.d_kc.download(np.uint16), L.kc) and np.array_equal(L.d_vc.download(np.uint16), L.vc)
    hip.destroy(graph, exe)
    stream.destroy()


def test_nine_streams_fall_back_and_slots_come_back(oracle):
    """The fixed block has eight slots: a ninth stream in use at the same time takes the allocating path (not under
    capture) and gives the same result; destroying streams frees their slots."""
    rng = np.random.default_rng(5)
    hq, hkv, d, lmax, kv_len = 8, 2, 64, 700, 650
    q, kc, vc = bf16(oracle, rng, hq * d), bf16(oracle, rng, hkv * lmax * d), bf16(oracle, rng, hkv * lmax * d)
    want = oracle.gqa_decode_batched_bf16(q, kc, vc, [kv_len], 1, hq, hkv, d, lmax)
    dq, dk, dv = ra.HipStorage.from_numpy(q), ra.HipStorage.from_numpy(kc), ra.HipStorage.from_numpy(vc)
    for _ in range(2):
        streams = [ra.Stream() for _ in range(10)]
        outs = [ra.HipStorage(hq * d * 2) for _ in streams]
        for s, o in zip(streams, outs):
            K.gqa_decode_online_bf16(s.handle, dq, dk, dv, o, hq, hkv, kv_len, d, lmax)
        for s, o in zip(streams, outs):
            s.synchronize()
            assert_decode_parity(oracle.bf16_to_f32(o.download(np.uint16)), want, d)
        for s in streams:
            s.destroy()
