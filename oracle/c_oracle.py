"""ctypes access to the C part of the CPU oracle (oracle/moe_oracle.c).  TEST INFRASTRUCTURE ONLY."""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libmoe_oracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(build())
        L.oracle_e4m3_decode.restype = ctypes.c_float
        L.oracle_e4m3_decode.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3_encode.restype = ctypes.c_uint8
        L.oracle_e4m3_encode.argtypes = [ctypes.c_float]
        p = ctypes.c_void_p
        i64 = ctypes.c_int64
        L.oracle_quant_rows_bf16.argtypes = [p, i64, i64, p, p]
        L.oracle_dequant_rows_bf16.argtypes = [p, p, i64, i64, p]
        L.oracle_permute_plan.argtypes = [p, i64, i64, p, p, p, p]
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def quant_rows_bf16(x_bits):
    """x_bits: uint16 [N,H] bf16 bit patterns -> (codes uint8 [N,H], scale float32 [N])."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    n, h = x_bits.shape
    q = np.empty((n, h), dtype=np.uint8)
    s = np.empty(n, dtype=np.float32)
    lib().oracle_quant_rows_bf16(_ptr(x_bits), n, h, _ptr(q), _ptr(s))
    return q, s


def dequant_rows_bf16(q, scale):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    n, h = q.shape
    out = np.empty((n, h), dtype=np.uint16)
    lib().oracle_dequant_rows_bf16(_ptr(q), _ptr(scale), n, h, _ptr(out))
    return out


def permute_plan(expert_idx, num_experts):
    e = np.ascontiguousarray(expert_idx, dtype=np.int64)
    n = e.size
    order, inv, within = (np.empty(n, dtype=np.int64) for _ in range(3))
    counts = np.empty(num_experts, dtype=np.int64)
    lib().oracle_permute_plan(_ptr(e), n, num_experts, _ptr(order), _ptr(inv), _ptr(counts), _ptr(within))
    return order, inv, counts, within
