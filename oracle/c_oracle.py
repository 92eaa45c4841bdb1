"""ctypes front end of the C oracle (oracle/decdec_oracle.c).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libdecdec_oracle.so")
_lib = None

DTYPE_CODE = {"fp32": 0, "fp16": 1, "bf16": 2}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "decdec_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "all"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u32, i32, f32 = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int, ctypes.c_float
        L.dd_bucket_floors.argtypes = [f32, f32, i32, vp]
        L.dd_select.argtypes = [vp, i32, u32, f32, f32, u32, vp, vp]
        L.dd_select.restype = i32
        L.dd_dec_apply.argtypes = [vp, i32, vp, vp, vp, u32, u32, u32, vp]
        L.dd_anyprec_gemv.argtypes = [vp, i32, vp, vp, i32, u32, u32, vp]
        L.dd_lutgemm_gemv.argtypes = [vp, i32, vp, vp, vp, i32, i32, u32, u32, vp]
        L.dd_sqllm_gemv.argtypes = [vp, i32, vp, vp, i32, u32, u32, vp]
        L.dd_layer_anyprec_dec.argtypes = [vp, i32, vp, vp, i32, vp, vp, f32, f32, u32, u32, u32, vp, vp]
        L.dd_f32_to_half.argtypes = [f32]; L.dd_f32_to_half.restype = ctypes.c_uint16
        L.dd_half_to_f32.argtypes = [ctypes.c_uint16]; L.dd_half_to_f32.restype = f32
        L.dd_f32_to_bf16.argtypes = [f32]; L.dd_f32_to_bf16.restype = ctypes.c_uint16
        _lib = L
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def as_bits(a: np.ndarray, dtype: str) -> np.ndarray:
    """Typed values -> the raw storage the C side expects (uint16 for fp16/bf16, float32 for fp32).
    bf16 inputs are float32 arrays holding bf16-representable values."""
    if dtype == "fp32":
        return np.ascontiguousarray(a, dtype=np.float32)
    if dtype == "fp16":
        return np.ascontiguousarray(np.asarray(a, dtype=np.float16)).view(np.uint16)
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return (u >> 16).astype(np.uint16)


def bucket_floors(a: float, b: float, dtype: str = "fp16") -> np.ndarray:
    out = np.zeros(32, dtype=np.float32)
    lib().dd_bucket_floors(float(a), float(b), DTYPE_CODE[dtype], _p(out))
    return out


def select(x, thresholds, k_chunk: int, dtype: str = "fp16"):
    xb = as_bits(np.asarray(x).reshape(-1), dtype)
    K = xb.shape[0]
    k = k_chunk * K // 1024
    nchunks = (K + 1023) // 1024
    rows = np.full(nchunks * max(k_chunk, 1), -1, dtype=np.int32)
    acts = np.zeros(nchunks * max(k_chunk, 1), dtype=xb.dtype)
    if k == 0:
        return rows, acts
    th = np.asarray(thresholds).reshape(-1).astype(np.float32)
    lib().dd_select(_p(xb), DTYPE_CODE[dtype], K, float(th[0]), float(th[k - 1]), k_chunk, _p(rows), _p(acts))
    return rows, acts


def dec_apply(x, cheatsheet, reordered_scales, rows, dtype: str = "fp16") -> np.ndarray:
    xb = as_bits(np.asarray(x).reshape(-1), dtype)
    K, M = cheatsheet.shape
    out = np.zeros(M * 8, dtype=np.float64)
    cs = np.ascontiguousarray(cheatsheet).view(np.uint32)
    sc = as_bits(np.asarray(reordered_scales).reshape(-1), dtype)
    r = np.ascontiguousarray(rows, dtype=np.int32)
    lib().dd_dec_apply(_p(xb), DTYPE_CODE[dtype], _p(cs), _p(sc), _p(r), r.shape[0], K, M * 8, _p(out))
    return out


def anyprec_gemv(x, qweight, lut, bits: int, dtype: str = "fp16") -> np.ndarray:
    xb = as_bits(np.asarray(x).reshape(-1), dtype)
    q = np.ascontiguousarray(qweight).view(np.uint32)
    _, N, W = q.shape
    out = np.zeros(N, dtype=np.float64)
    lb = as_bits(np.asarray(lut), dtype)
    lib().dd_anyprec_gemv(_p(xb), DTYPE_CODE[dtype], _p(q), _p(lb), bits, N, W * 32, _p(out))
    return out


def lutgemm_gemv(x, q_weight, alpha, q_bias, bits: int, group_size: int, dtype: str = "fp16") -> np.ndarray:
    xb = as_bits(np.asarray(x).reshape(-1), dtype)
    q = np.ascontiguousarray(q_weight).view(np.uint32)
    KT, B, N = q.shape
    out = np.zeros(N, dtype=np.float64)
    lib().dd_lutgemm_gemv(_p(xb), DTYPE_CODE[dtype], _p(q), _p(as_bits(np.asarray(alpha), dtype)),
                          _p(as_bits(np.asarray(q_bias), dtype)), bits, group_size, N, KT * 32, _p(out))
    return out


def sqllm_gemv(x, mat, lut, bits: int, dtype: str = "fp16") -> np.ndarray:
    xb = as_bits(np.asarray(x).reshape(-1), dtype)
    m = np.ascontiguousarray(mat).view(np.uint32)
    R, N = m.shape
    K = R * 32 // bits
    out = np.zeros(N, dtype=np.float64)
    lib().dd_sqllm_gemv(_p(xb), DTYPE_CODE[dtype], _p(m), _p(as_bits(np.asarray(lut), dtype)), bits, N, K, _p(out))
    return out


def layer_anyprec_dec(x, qweight, lut, bits, cheatsheet, reordered_scales, thr_a, thr_b, k_chunk,
                      dtype: str = "fp16"):
    """One DEC-compensated any-precision layer on the CPU; returns (y float64[N], rows int32)."""
    xb = as_bits(np.asarray(x).reshape(-1), dtype)
    q = np.ascontiguousarray(qweight).view(np.uint32)
    _, N, W = q.shape
    K = W * 32
    nchunks = (K + 1023) // 1024
    rows = np.full(nchunks * max(k_chunk, 1), -1, dtype=np.int32)
    out = np.zeros(N, dtype=np.float64)
    cs = np.ascontiguousarray(cheatsheet).view(np.uint32)
    lib().dd_layer_anyprec_dec(_p(xb), DTYPE_CODE[dtype], _p(q), _p(as_bits(np.asarray(lut), dtype)), bits,
                               _p(cs), _p(as_bits(np.asarray(reordered_scales).reshape(-1), dtype)),
                               float(thr_a), float(thr_b), k_chunk, N, K, _p(rows), _p(out))
    return out, rows
