"""ctypes binding of librt_attn_hip.so (the C ABI declared in include/rt_attn.h).

The library is the only compute path: if it is missing, loading raises and every operation
of the package fails with it.  There is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librt_attn_hip.so")

# every symbol include/rt_attn.h declares
SYMBOLS = (
    "rt_init", "rt_shutdown", "rt_version", "rt_status_name", "rt_hip_runtime_path",
    "rt_flash_forward_f32", "rt_flash_forward_masked_f32", "rt_gqa_forward_f32", "rt_gqa_forward_f32_dev",
    "rt_flash_backward_f32", "rt_flash_backward_f32_dev", "rt_flash_backward_workspace_bytes",
    "rt_flash_forward_stats_f32_dev", "rt_flash_backward_saved_f32_dev",
    "rt_flash_forward_f32_dev", "rt_flash_forward_bf16_dev", "rt_flash_forward_varlen_bf16_dev",
    "rt_mha_flash_forward_f32", "rt_mha_forward_masked_f32", "rt_mha_forward_masked_f32_dev", "rt_mha_forward_masked_bf16_dev", "rt_gqa_decode_chunk_bf16", "rt_flash_forward_bnhd_f32_dev", "rt_flash_forward_bnhd_bf16_dev",
    "rt_kv_append_bf16", "rt_kv_cache_append_dev", "rt_qk_norm_rope_kv_append_bf16", "rt_gqa_decode_online_bf16", "rt_gqa_decode_naive_bf16", "rt_gqa_decode_batched_bf16",
    "rt_gqa_decode_workspace_bytes", "rt_gqa_decode_batched_bf16_noalloc",
    "rt_buf_alloc", "rt_buf_free", "rt_buf_zero", "rt_memcpy_h2d", "rt_memcpy_d2h", "rt_stream_synchronize",
    "rt_stream_create", "rt_stream_destroy", "rt_i32_add_dev", "rt_debug_force_bf16_prefill_kernel", "rt_set_strict_non_finite_v",
    "rt_flash_forward_window_bf16_dev", "rt_flash_forward_window_bnhd_bf16_dev",
)

RT_OK = 0
RT_ERR_ZERO_DIM = 1
RT_ERR_BUFFER_SHAPE_MISMATCH = 2
RT_ERR_OUTPUT_SHAPE_MISMATCH = 3
RT_ERR_PADDING_LENGTH_MISMATCH = 4
RT_ERR_HEAD_COUNT_MISMATCH = 5
RT_ERR_WRONG_INPUT_LEN = 6
RT_ERR_KV_OVERFLOW = 7
RT_ERR_KV_WRONG_INPUT_LEN = 8
RT_ERR_ROPE_WRONG_INPUT_LEN = 9
RT_ERR_ROPE_POSITION_OVERFLOW = 10
RT_ERR_NULL_POINTER = 20
RT_ERR_UNSUPPORTED = 21
RT_ERR_WORKSPACE_TOO_SMALL = 22
RT_ERR_NO_DEVICE = 30
RT_ERR_HIP = 31

RT_MASK_NONE, RT_MASK_CAUSAL, RT_MASK_PADDING = 0, 1, 2
WHICH = {0: "q", 1: "k", 2: "v", 3: "out", 4: "flash_forward", 5: "mask", 6: "do", -1: ""}


class RtShape(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("batch", "heads", "seq", "dim", "br", "bc")]


class RtErr(C.Structure):
    _fields_ = [("which", C.c_int32), ("expected", C.c_uint64), ("got", C.c_uint64), ("got2", C.c_uint64),
                ("hip_error", C.c_int32), ("message", C.c_char * 160)]


class LibraryMissing(RuntimeError):
    pass


_lib = None


def lib():
    """Load librt_attn_hip.so (built by __graft_entry__.build() / `make -C rustorch_amd/csrc`)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            f"{LIB_PATH} is missing: build it with `make -C rustorch_amd/csrc` (hipcc, gfx950). "
            "rustorch_amd has no CPU fallback.")
    L = C.CDLL(LIB_PATH)
    vp, sz, fp, u8p, i32p = C.c_void_p, C.c_size_t, C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.c_void_p
    errp, shp = C.POINTER(RtErr), C.POINTER(RtShape)
    i32, u64 = C.c_int32, C.c_uint64
    L.rt_init.argtypes = [C.c_int, errp]
    L.rt_version.restype = C.c_char_p
    L.rt_hip_runtime_path.restype = C.c_char_p
    L.rt_status_name.argtypes = [C.c_int]
    L.rt_status_name.restype = C.c_char_p
    L.rt_flash_forward_f32.argtypes = [shp, fp, sz, fp, sz, fp, sz, fp, sz, errp]
    L.rt_flash_forward_masked_f32.argtypes = [shp, fp, sz, fp, sz, fp, sz, C.c_int, u8p, sz, fp, sz, errp]
    L.rt_gqa_forward_f32.argtypes = [fp, sz, fp, sz, fp, sz, fp, sz, sz, sz, sz, sz, sz, sz, errp]
    L.rt_gqa_forward_f32_dev.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, errp]
    L.rt_flash_backward_f32.argtypes = [shp] + [fp, sz] * 7 + [errp]
    L.rt_flash_backward_f32_dev.argtypes = [vp, shp] + [vp] * 8 + [sz, errp]
    L.rt_flash_backward_workspace_bytes.argtypes = [shp]
    L.rt_flash_forward_stats_f32_dev.argtypes = [vp, shp] + [vp] * 5 + [errp]
    L.rt_flash_backward_saved_f32_dev.argtypes = [vp, shp] + [vp] * 10 + [sz, errp]
    L.rt_flash_backward_workspace_bytes.restype = sz
    L.rt_flash_forward_f32_dev.argtypes = [vp, shp, u64, vp, vp, vp, C.c_int, vp, vp, errp]
    L.rt_flash_forward_bf16_dev.argtypes = [vp, shp, u64, vp, vp, vp, C.c_int, vp, vp, errp]
    L.rt_flash_forward_varlen_bf16_dev.argtypes = [vp, shp, u64, vp, vp, vp, i32p, C.c_int, vp, errp]
    L.rt_mha_flash_forward_f32.argtypes = [fp, sz, fp, sz, fp, sz, fp, sz, sz, sz, sz, sz, errp]
    L.rt_mha_forward_masked_f32.argtypes = [fp, sz, fp, sz, fp, sz, fp, sz, fp, sz, sz, sz, sz, sz, sz, errp]
    L.rt_mha_forward_masked_f32_dev.argtypes = [vp, vp, vp, vp, vp, sz, vp, sz, sz, sz, sz, sz, errp]
    L.rt_mha_forward_masked_bf16_dev.argtypes = [vp, vp, vp, vp, vp, sz, vp, sz, sz, sz, sz, sz, errp]
    L.rt_gqa_decode_chunk_bf16.argtypes = [vp, vp, vp, vp, vp, i32p, i32, i32, i32, i32, i32, i32, i32, errp]
    L.rt_flash_forward_bnhd_f32_dev.argtypes = [vp, shp, u64, vp, vp, vp, C.c_int, vp, vp, errp]
    L.rt_flash_forward_bnhd_bf16_dev.argtypes = [vp, shp, u64, vp, vp, vp, C.c_int, vp, vp, errp]
    L.rt_flash_forward_window_bf16_dev.argtypes = [vp, shp, u64, vp, vp, vp, u64, vp, errp]
    L.rt_flash_forward_window_bnhd_bf16_dev.argtypes = [vp, shp, u64, vp, vp, vp, u64, vp, errp]
    L.rt_kv_append_bf16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, errp]
    L.rt_kv_cache_append_dev.argtypes = [vp, vp, vp, vp, sz, vp, sz, sz, sz, sz, sz, sz, sz, sz, errp]
    L.rt_qk_norm_rope_kv_append_bf16.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, vp, vp, C.c_float, vp, vp, i32, i32,
                                                 i32, i32, i32, i32, i32, errp]
    L.rt_gqa_decode_online_bf16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, errp]
    L.rt_gqa_decode_naive_bf16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, errp]
    L.rt_gqa_decode_batched_bf16.argtypes = [vp, vp, vp, vp, vp, i32p, i32, i32, i32, i32, i32, vp, sz, errp]
    L.rt_gqa_decode_batched_bf16_noalloc.argtypes = [vp, vp, vp, vp, vp, i32p, i32, i32, i32, i32, i32, errp]
    L.rt_gqa_decode_workspace_bytes.argtypes = [i32, i32, i32, i32, i32]
    L.rt_gqa_decode_workspace_bytes.restype = sz
    L.rt_buf_alloc.argtypes = [sz, errp]
    L.rt_buf_alloc.restype = vp
    L.rt_buf_free.argtypes = [vp, errp]
    L.rt_buf_zero.argtypes = [vp, sz, vp, errp]
    L.rt_memcpy_h2d.argtypes = [vp, vp, sz, vp, errp]
    L.rt_memcpy_d2h.argtypes = [vp, vp, sz, vp, errp]
    L.rt_stream_synchronize.argtypes = [vp, errp]
    L.rt_shutdown.argtypes = [errp]
    L.rt_stream_create.argtypes = [errp]
    L.rt_stream_create.restype = vp
    L.rt_stream_destroy.argtypes = [vp, errp]
    L.rt_i32_add_dev.argtypes = [vp, vp, sz, i32, errp]
    L.rt_debug_force_bf16_prefill_kernel.argtypes = [C.c_int]
    L.rt_set_strict_non_finite_v.argtypes = [C.c_int]
    L.rt_set_strict_non_finite_v.restype = C.c_int
    _lib = L
    return L


def hip_runtime():
    """The HIP runtime librt_attn_hip.so is bound to, as a ctypes handle (loaded by the path the library reports for
    it): a caller that wants streams, events or graphs of its own must talk to that runtime instance.  A process
    that has imported PyTorch holds a second copy of the runtime, and `CDLL("libamdhip64.so")` may return that one."""
    path = lib().rt_hip_runtime_path().decode()
    return C.CDLL(path if path else "libamdhip64.so")


def status_name(code: int) -> str:
    return lib().rt_status_name(code).decode()
