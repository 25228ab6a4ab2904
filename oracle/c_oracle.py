"""ctypes binding of the plain-C oracle (oracle/fp8_oracle.c).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfp8_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libfp8_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_e4m3_decode.restype = ctypes.c_float
        L.orc_e4m3_decode.argtypes = [ctypes.c_uint8]
        L.orc_e4m3_encode.restype = ctypes.c_uint8
        L.orc_e4m3_encode.argtypes = [ctypes.c_float]
        L.orc_bf16_bits.restype = ctypes.c_uint16
        L.orc_bf16_bits.argtypes = [ctypes.c_float]
        L.orc_moe_align.restype = ctypes.c_int32
        _lib = L
    return _lib


def _p(a, ct):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ct))


def gemm_block_scaled(A, B, As, Bs, bn=128, bk=128, alpha=1.0):
    """A (M,K) uint8 codes, B (N,K) uint8 codes, As/Bs float32 or None -> (M,N) float32."""
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    As = None if As is None else np.ascontiguousarray(As, dtype=np.float32)
    Bs = None if Bs is None else np.ascontiguousarray(Bs, dtype=np.float32)
    M, K = A.shape
    N = B.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    lib().orc_gemm_block_scaled(_p(A, ctypes.c_uint8), _p(B, ctypes.c_uint8), _p(As, ctypes.c_float),
                                _p(Bs, ctypes.c_float), ctypes.c_int64(M), ctypes.c_int64(N),
                                ctypes.c_int64(K), ctypes.c_int64(bn), ctypes.c_int64(bk),
                                ctypes.c_float(alpha), _p(out, ctypes.c_float))
    return out


def gemm_per_tensor(A, B, sa, sb):
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    M, K = A.shape
    N = B.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    lib().orc_gemm_per_tensor(_p(A, ctypes.c_uint8), _p(B, ctypes.c_uint8), ctypes.c_float(sa),
                              ctypes.c_float(sb), ctypes.c_int64(M), ctypes.c_int64(N),
                              ctypes.c_int64(K), _p(out, ctypes.c_float))
    return out


def gemm_ragged(A, B, As, Bs, indptr, bn=128, bk=128):
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    As = None if As is None else np.ascontiguousarray(As, dtype=np.float32)
    Bs = None if Bs is None else np.ascontiguousarray(Bs, dtype=np.float32)
    indptr = np.ascontiguousarray(indptr, dtype=np.int32)
    total_m, K = A.shape
    Q, N, _ = B.shape
    out = np.zeros((total_m, N), dtype=np.float32)
    lib().orc_gemm_ragged(_p(A, ctypes.c_uint8), _p(B, ctypes.c_uint8), _p(As, ctypes.c_float),
                          _p(Bs, ctypes.c_float), _p(indptr, ctypes.c_int32), ctypes.c_int64(Q),
                          ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int64(bn),
                          ctypes.c_int64(bk), _p(out, ctypes.c_float))
    return out


def decode_table():
    out = np.empty(256, dtype=np.float32)
    lib().orc_e4m3_decode_table(_p(out, ctypes.c_float))
    return out


def moe_align(topk_ids, block_size, num_experts):
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32).reshape(-1)
    numel = ids.size
    cap = numel + num_experts * (block_size - 1)
    sorted_ids = np.empty(cap, dtype=np.int32)
    expert_ids = np.empty(-(-cap // block_size), dtype=np.int32)
    cumsum = np.empty(num_experts + 1, dtype=np.int32)
    mx = ctypes.c_int32(0)
    post = lib().orc_moe_align(_p(ids, ctypes.c_int32), ctypes.c_int64(numel), ctypes.c_int32(num_experts),
                               ctypes.c_int32(block_size), _p(sorted_ids, ctypes.c_int32),
                               _p(expert_ids, ctypes.c_int32), _p(cumsum, ctypes.c_int32),
                               ctypes.byref(mx))
    return sorted_ids, expert_ids, int(post), cumsum, int(mx.value)
