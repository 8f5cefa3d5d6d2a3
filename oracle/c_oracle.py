"""ctypes access to oracle/libfp8_oracle.so (the C restatement).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(_HERE, "libfp8_oracle.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "fp8_oracle.c")
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libfp8_oracle.so"], check=True,
                       capture_output=True)
    return LIB


def load() -> ctypes.CDLL:
    if not os.path.exists(LIB):
        build()
    lib = ctypes.CDLL(LIB)
    i64, p = ctypes.c_int64, ctypes.c_void_p
    lib.oracle_num_threads.restype = ctypes.c_int
    lib.oracle_group_quant_bf16.argtypes = [p, p, p, i64, i64, ctypes.c_int, ctypes.c_float, ctypes.c_int]
    lib.oracle_block_gemm.argtypes = [p, p, p, p, p, i64, i64, i64]
    lib.oracle_scaled_mm.argtypes = [p, p, p, p, p, p, i64, i64, i64]
    lib.oracle_w8a16_block_gemm.argtypes = [p, p, p, p, p, i64, i64, i64]
    return lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def group_quant_bf16(lib, x_bits: np.ndarray, group: int, eps_eff: float, ue8m0: bool = False):
    """x_bits uint16 [M,K] (bf16 patterns) -> (q uint8 [M,K], s float32 [M,K/group])."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    M, K = x_bits.shape
    q = np.empty((M, K), dtype=np.uint8)
    s = np.empty((M, K // group), dtype=np.float32)
    lib.oracle_group_quant_bf16(_ptr(x_bits), _ptr(q), _ptr(s), M, K, group, eps_eff, 1 if ue8m0 else 0)
    return q, s


def block_gemm(lib, A, B, As, Bs):
    """-> bf16 bit patterns uint16 [M,N]."""
    A = np.ascontiguousarray(A, np.uint8); B = np.ascontiguousarray(B, np.uint8)
    As = np.ascontiguousarray(As, np.float32); Bs = np.ascontiguousarray(Bs, np.float32)
    M, K = A.shape
    N = B.shape[0]
    C = np.empty((M, N), dtype=np.uint16)
    lib.oracle_block_gemm(_ptr(A), _ptr(B), _ptr(As), _ptr(Bs), _ptr(C), M, N, K)
    return C


def scaled_mm(lib, A, B, sa, sb, bias=None):
    A = np.ascontiguousarray(A, np.uint8); B = np.ascontiguousarray(B, np.uint8)
    sa = np.ascontiguousarray(sa, np.float32); sb = np.ascontiguousarray(sb, np.float32)
    M, K = A.shape
    N = B.shape[0]
    C = np.empty((M, N), dtype=np.uint16)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    lib.oracle_scaled_mm(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), None if b is None else _ptr(b), _ptr(C), M, N, K)
    return C


def w8a16_block_gemm(lib, A_bits, B, Bs, bias=None):
    """The reference CPU twin's algorithm (W8A16, see fp8_oracle.c): A_bits uint16 [M,K] bf16 patterns, B uint8 [N,K],
    Bs float32 [ceil(N/128), K/128] -> bf16 bit patterns uint16 [M,N]."""
    A_bits = np.ascontiguousarray(A_bits, np.uint16); B = np.ascontiguousarray(B, np.uint8)
    Bs = np.ascontiguousarray(Bs, np.float32)
    M, K = A_bits.shape
    N = B.shape[0]
    C = np.empty((M, N), dtype=np.uint16)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    lib.oracle_w8a16_block_gemm(_ptr(A_bits), _ptr(B), _ptr(Bs), None if b is None else _ptr(b), _ptr(C), M, N, K)
    return C
