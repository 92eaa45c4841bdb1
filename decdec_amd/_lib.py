"""ctypes binding of libdecdec_hip.so (the C ABI declared in include/decdec_hip.h).

There is no CPU fallback: if the library is missing or cannot be loaded, every op raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdecdec_hip.so")

_lib = None


class ConfigInfo(ctypes.Structure):
    """Mirror of ``decdec_config_info``."""
    _fields_ = [(name, ctypes.c_int32) for name in (
        "num_chunks", "chunk_size", "k_chunk", "channels_per_tb", "n_tb",
        "block_dim_x", "block_dim_y", "shared_memory_size", "reduced_shared_memory",
        "hip_dec_blocks", "hip_chunk_groups", "hip_segment_groups", "hip_vec_words",
        "hip_lds_bytes", "hip_slots_per_block", "hip_lds_reduce", "hip_residual_on_host")]


REFERENCE_KEYS = ("num_chunks", "chunk_size", "k_chunk", "channels_per_tb", "n_tb",
                  "block_dim_x", "block_dim_y", "shared_memory_size", "reduced_shared_memory")

_vp, _u32, _u64, _i32, _i64, _f32 = (ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64,
                                     ctypes.c_int, ctypes.c_int64, ctypes.c_float)

# name -> argtypes; every function returns int except the two noted below
SIGNATURES = {
    "decdec_set_option": [ctypes.c_char_p, _i32],
    "decdec_get_option": [ctypes.c_char_p, ctypes.POINTER(_i32)],
    "decdec_create_dec_context": [_u32, _i32, _u64, _vp, _vp, ctypes.POINTER(_u64)],
    "decdec_destroy_dec_context": [_u64],
    "decdec_create_dec_config": [_u64, _u32, _i32, _vp, _i32, _vp, _i32, _vp, _u32, _u32, ctypes.POINTER(_u64)],
    "decdec_read_dec_config": [_u64, ctypes.POINTER(ConfigInfo)],
    "decdec_update_dec_config": [_u64, _u64, _u32],
    "decdec_destroy_dec_config": [_u64],
    "decdec_dec": [_u64, _vp, _vp, _i32, _u32, _u32, _vp],
    "decdec_unfused_dec": [_u64, _vp, _vp, _i32, _u32, _u32, _vp],
    "decdec_anyprec_gemv": [_vp, _vp, _vp, _vp, _i32, _i32, _u32, _u32, _vp],
    "decdec_anyprec_dequant": [_vp, _vp, _vp, _i32, _i32, _u32, _u32, _vp],
    "decdec_lutgemm_gemv": [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _u32, _u32, _vp],
    "decdec_sqllm_gemv": [_vp, _vp, _vp, _vp, _i32, _i32, _u32, _u32, _vp],
    "decdec_dec_anyprec": [_u64, _vp, _vp, _vp, _vp, _i32, _i32, _u32, _u32, _vp],
    "decdec_dec_anyprec_batch": [_u32, ctypes.POINTER(_u64), _vp, ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                                 ctypes.POINTER(_vp), _i32, _i32, _u32, ctypes.POINTER(_u32), _vp],
    "decdec_dec_lutgemm": [_u64, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _u32, _u32, _vp],
    "decdec_dec_lutgemm_batch": [_u32, ctypes.POINTER(_u64), _vp, ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                                 ctypes.POINTER(_vp), ctypes.POINTER(_vp), _i32, _i32, _i32, _u32, ctypes.POINTER(_u32), _vp],
    "decdec_dec_sqllm_batch": [_u32, ctypes.POINTER(_u64), _vp, ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                               ctypes.POINTER(_vp), _i32, _i32, _u32, ctypes.POINTER(_u32), _vp],
    "decdec_dec_sqllm": [_u64, _vp, _vp, _vp, _vp, _i32, _i32, _u32, _u32, _vp],
    "decdec_dummy_anyprec": [_vp, _vp, _vp, _vp, _i32, _i32, _u32, _u32, _i32, _i64, _vp],
    "decdec_dummy_lutgemm": [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _u32, _u32, _i32, _i64, _vp],
    "decdec_dummy_sqllm": [_vp, _vp, _vp, _vp, _i32, _i32, _u32, _u32, _i32, _i64, _vp],
    "decdec_rope_cache_update": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _u32, _u32, _u32, _u32, _vp],
    "decdec_decode_attention": [_vp, _vp, _vp, _vp, _vp, _i32, _u32, _u32, _u32, _u32, _vp, _u64, _vp],
    "decdec_decode_attention_static": [_vp, _vp, _vp, _vp, _vp, _i32, _u32, _u32, _u32, _u32, _vp],
    "decdec_rope_attention": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _u32, _u32, _u32, _u32, _vp, _u64, _vp],
    "decdec_dense_gemv": [_vp, _vp, _vp, _i32, _u32, _u32, _vp],
    "decdec_silu_mul": [_vp, _vp, _i32, _u32, _vp],
    "decdec_add_rmsnorm": [_vp, _vp, _vp, _vp, _vp, _i32, _u32, _u32, _f32, _vp],
    "decdec_greedy_pick": [_vp, _u32, _i32, _vp, _vp, _vp, _vp, _u32, _vp, _vp, _vp],
    "decdec_debug_read_trace": [ctypes.POINTER(_u64), _i32],
    "decdec_debug_read_probe": [_vp, _u64, _u64, _u32, _u32, _i32, _vp, _vp],
    "decdec_bucket_floors": [_f32, _f32, _i32, ctypes.POINTER(_f32)],
    "decdec_reference_geometry": [_u32, _u32, _u32, _u32, _i32, _u32, ctypes.POINTER(ConfigInfo)],
    "decdec_dec_launch_plan": [_u32, _u32, _u32, _u32, _u32, ctypes.POINTER(ConfigInfo)],
    "decdec_fused_launch_form": [_i32, _i32, _u32, _u32, _u32, ctypes.POINTER(_i32)],
}
OTHER_SYMBOLS = {"decdec_last_error": ([], ctypes.c_char_p), "decdec_version": ([], _i32),
                 "decdec_decode_attention_workspace_bytes": ([_u32, _u32, _u32], _u64),
                 "decdec_greedy_pick_workspace_bytes": ([], _u64)}


def load():
    """Load the shared library once; raise RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m decdec_amd.build` "
            "(there is no CPU or PyTorch fallback for these ops)")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as exc:  # pragma: no cover - depends on the machine
        raise RuntimeError(f"cannot load {LIB_PATH}: {exc}") from exc
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _i32
    for name, (argtypes, restype) in OTHER_SYMBOLS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    _lib = lib
    return lib


def last_error() -> str:
    msg = load().decdec_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(status: int) -> None:
    """Turn a non-zero status into the RuntimeError the reference's TORCH_CHECK would raise."""
    if status != 0:
        raise RuntimeError(last_error())


def set_option(name: str, value: int) -> None:
    check(load().decdec_set_option(name.encode(), int(value)))


def get_option(name: str) -> int:
    v = _i32(0)
    check(load().decdec_get_option(name.encode(), ctypes.byref(v)))
    return v.value
