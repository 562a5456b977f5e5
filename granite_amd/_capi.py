"""ctypes binding of libgranite_hip.so (the C ABI declared in include/granite_hip.h).

The library is loaded from granite_amd/lib/ inside the source tree.  There is
no fallback: if the library is missing or a call fails, a GraniteHipError is
raised.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libgranite_hip.so"

# constants of granite_hip.h
OK = 0
EINVAL, ENOTINIT, ENOMEM, EUNSUPPORTED, ENULL, EOVERFLOW, ESCRATCH = -1, -2, -3, -4, -5, -6, -7
F32, F16 = 0, 1
ROUND_TRUNCATE, ROUND_NEAREST = 0, 1
MEM_DEVICE, MEM_SHARED, MEM_MANAGED = 0, 1, 2
MASK_NONE, MASK_CAUSAL, MASK_TREE = 0, 1, 2


class GraniteHipError(RuntimeError):
    def __init__(self, code: int, what: str, message: str):
        super().__init__(f"{what} failed: {message} (code {code})")
        self.code = code


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 32),
        ("total_memory", C.c_size_t),
        ("max_buffer_size", C.c_size_t),
        ("shared_memory_per_block", C.c_size_t),
        ("max_threads_per_block", C.c_int),
        ("wavefront_size", C.c_int),
        ("compute_units", C.c_int),
        ("clock_khz", C.c_int),
    ]


class DecodeArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("q_dtype", C.c_int),
        ("k_cache", C.c_void_p),
        ("v_cache", C.c_void_p),
        ("block_tables", C.c_void_p),
        ("seq_lens", C.c_void_p),
        ("out", C.c_void_p),
        ("lse", C.c_void_p),
        ("batch_size", C.c_uint32),
        ("num_heads", C.c_uint32),
        ("num_kv_heads", C.c_uint32),
        ("head_dim", C.c_uint32),
        ("block_size", C.c_uint32),
        ("max_blocks_per_seq", C.c_uint32),
        ("max_seq", C.c_uint32),
        ("scale", C.c_float),
        ("fixed_seq_len", C.c_uint32),
        ("chunk_tokens", C.c_uint32),
    ]


class AttentionArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("q_dtype", C.c_int),
        ("q_tok_stride", C.c_int64),
        ("q_head_stride", C.c_int64),
        ("out", C.c_void_p),
        ("out_dtype", C.c_int),
        ("out_tok_stride", C.c_int64),
        ("out_head_stride", C.c_int64),
        ("lse", C.c_void_p),
        ("k_cache", C.c_void_p),
        ("v_cache", C.c_void_p),
        ("block_table", C.c_void_p),
        ("block_size", C.c_uint32),
        ("max_seq", C.c_uint32),
        ("cache_len", C.c_uint32),
        ("k_extra", C.c_void_p),
        ("v_extra", C.c_void_p),
        ("extra_len", C.c_uint32),
        ("parents", C.c_void_p),
        ("mask_mode", C.c_int),
        ("start_pos", C.c_uint32),
        ("seq_q", C.c_uint32),
        ("num_heads", C.c_uint32),
        ("num_kv_heads", C.c_uint32),
        ("head_dim", C.c_uint32),
        ("scale", C.c_float),
    ]


class RopeArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("q_f16", C.c_void_p),
        ("k", C.c_void_p),
        ("v", C.c_void_p),
        ("cache_k", C.c_void_p),
        ("cache_v", C.c_void_p),
        ("block_table", C.c_void_p),
        ("cos_table", C.c_void_p),
        ("sin_table", C.c_void_p),
        ("table_positions", C.c_uint32),
        ("num_heads_q", C.c_uint32),
        ("num_heads_k", C.c_uint32),
        ("seq_len", C.c_uint32),
        ("head_dim", C.c_uint32),
        ("start_pos", C.c_uint32),
        ("max_seq_len", C.c_uint32),
        ("block_size", C.c_uint32),
        ("freq_base", C.c_float),
        ("write_k_back", C.c_int),
        ("rounding", C.c_int),
        ("positions", C.c_void_p),
        ("table_stride", C.c_int64),
        ("max_blocks_per_seq", C.c_uint32),
    ]


_u32, _i64, _vp, _int, _f32 = C.c_uint32, C.c_int64, C.c_void_p, C.c_int, C.c_float

# name -> (restype, argtypes); every symbol granite_hip.h declares
SIGNATURES = {
    "granite_hip_init": (_int, [_int]),
    "granite_hip_shutdown": (_int, []),
    "granite_hip_is_initialized": (_int, []),
    "granite_hip_get_device_info": (_int, [C.POINTER(DeviceInfo)]),
    "granite_hip_error_string": (C.c_char_p, [_int]),
    "granite_hip_version": (C.c_char_p, []),
    "granite_hip_malloc": (_int, [C.POINTER(_vp), C.c_size_t, _int]),
    "granite_hip_free": (_int, [_vp, _int]),
    "granite_hip_memcpy_h2d": (_int, [_vp, _vp, C.c_size_t]),
    "granite_hip_memcpy_d2h": (_int, [_vp, _vp, C.c_size_t]),
    "granite_hip_memcpy_d2d": (_int, [_vp, _vp, C.c_size_t]),
    "granite_hip_memset": (_int, [_vp, _int, C.c_size_t]),
    "granite_hip_sync": (_int, []),
    "granite_hip_set_stream": (_int, [_vp]),
    "granite_hip_get_stream": (_vp, []),
    "granite_hip_event_create": (_int, [C.POINTER(_vp)]),
    "granite_hip_event_destroy": (_int, [_vp]),
    "granite_hip_event_record": (_int, [_vp]),
    "granite_hip_event_synchronize": (_int, [_vp]),
    "granite_hip_event_elapsed_ms": (_int, [_vp, _vp, C.POINTER(_f32)]),
    "granite_hip_enable_kernel_timing": (_int, [_int]),
    "granite_hip_reset_kernel_timing": (_int, []),
    "granite_hip_get_kernel_timing": (_int, [C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_uint64)]),
    "granite_hip_kernel_timing_names": (_int, [C.c_char_p, C.c_size_t]),
    "granite_hip_kv_cache_append": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "granite_hip_kv_cache_append_ex": (
        _int, [_vp, _vp, _vp, _vp, _int, _i64, _i64, _u32, _u32, _u32, _u32, _u32, _int]),
    "granite_hip_paged_kv_cache_append": (
        _int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "granite_hip_paged_kv_cache_append_ex": (
        _int, [_vp, _vp, _int, _i64, _i64, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _int, _u32]),
    "granite_hip_paged_kv_gather": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "granite_hip_copy_rows": (_int, [_vp, C.c_int64, _vp, C.c_int64, C.c_uint64, _u32, _u32]),
    "granite_hip_multihead_attention": (
        _int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _f32, _u32]),
    "granite_hip_attention_tree": (
        _int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _f32]),
    "granite_hip_paged_attention_decode": (
        _int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _f32]),
    "granite_hip_batched_paged_attention_decode": (
        _int, [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, _f32]),
    "granite_hip_decode_attention": (_int, [C.POINTER(DecodeArgs)]),
    "granite_hip_attention": (_int, [C.POINTER(AttentionArgs)]),
    "granite_hip_build_tree_mask": (_int, [_vp, _vp, _u32]),
    "granite_hip_kv_commit_accepted": (_int, [_vp, _vp, _int, _i64, _i64, _u32, _vp, _u32, _vp, _vp, _vp, _u32,
                                             _u32, _u32, _u32, _u32, _int]),
    "granite_hip_rope_multihead": (_int, [_vp, _vp, _u32, _u32, _u32, _u32, _u32, _f32]),
    "granite_hip_rope_append": (_int, [C.POINTER(RopeArgs)]),
    "granite_hip_fused_qkv_matvec_q4k": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "granite_hip_fused_qkv_matvec_q4k_batched": (
        _int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _u32, _u32, _u32, _u32]),
    "granite_hip_q4k_workspace_required": (C.c_size_t, [_u32, C.c_uint64, _u32]),
    "granite_hip_matvec_q4k": (_int, [_vp, _vp, _vp, _u32, _u32]),
    "granite_hip_matvec_q4k_batched": (_int, [_vp, _i64, _vp, _vp, _i64, _u32, _u32, _u32]),
    "granite_hip_workspace_bytes": (C.c_size_t, []),
    "granite_hip_reserve_workspace": (_int, [C.c_size_t]),
    "granite_hip_decode_workspace_required": (_int, [C.POINTER(DecodeArgs), C.POINTER(C.c_size_t)]),
    "granite_hip_attention_workspace_required": (_int, [C.POINTER(AttentionArgs), C.POINTER(C.c_size_t)]),
    "granite_hip_decode_attention_ws": (_int, [C.POINTER(DecodeArgs), _vp, C.c_size_t]),
    "granite_hip_attention_ws": (_int, [C.POINTER(AttentionArgs), _vp, C.c_size_t]),
    "granite_hip_decode_attention_static": (_int, [C.POINTER(DecodeArgs)]),
    "granite_hip_static_scratch_bytes": (C.c_size_t, []),
}

_lib = None


def load() -> C.CDLL:
    """Load libgranite_hip.so (once) and attach the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise GraniteHipError(
            ENOTINIT, "load",
            f"{LIB_PATH} is missing: build it with `python -m granite_amd.build` "
            "(there is no CPU fallback)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = ABI drift, let it surface
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != OK:
        msg = load().granite_hip_error_string(code)
        raise GraniteHipError(code, what, msg.decode() if msg else "?")
