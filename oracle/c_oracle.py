"""ctypes front end of the C restatement (``psg_oracle_c.c``).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

KIND = {"int8": 0, "fp8": 1}
EPI = {"none": 0, "bias": 1, "bias_relu": 2, "bias_silu": 3, "bias_gelu": 4}


def build() -> str:
    """Compile ``libpsg_oracle.so`` next to its source (gcc, OpenMP)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libpsg_oracle.so"], check=True, capture_output=True)
    return os.path.join(_HERE, "libpsg_oracle.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libpsg_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(arr):
    return None if arr is None else arr.ctypes.data_as(ctypes.c_void_p)


def a8w8(a, b_shuf, sa, sb, kind, *, bias_bf16_bits=None, epilogue="none", want_acc_i32=False):
    """Returns dict(acc_i32|None, acc_f32, c_bf16_bits) computed from the wire format."""
    a = np.ascontiguousarray(a).view(np.uint8)
    b = np.ascontiguousarray(b_shuf).view(np.uint8)
    m, k = a.shape
    n = b.shape[0]
    sa = np.ascontiguousarray(sa, dtype=np.float32).reshape(-1)
    sb = np.ascontiguousarray(sb, dtype=np.float32).reshape(-1)
    acc_i = np.empty((m, n), np.int32) if want_acc_i32 else None
    acc_f = np.empty((m, n), np.float32)
    c = np.empty((m, n), np.uint16)
    bias = None if bias_bf16_bits is None else np.ascontiguousarray(bias_bf16_bits, dtype=np.uint16)
    f = lib().psg_oracle_a8w8
    f.restype = ctypes.c_int
    rc = f(_p(a), _p(b), _p(sa), _p(sb), _p(bias), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
           ctypes.c_int(KIND[kind]), ctypes.c_int(EPI[epilogue]), _p(acc_i), _p(acc_f), _p(c))
    if rc != 0:
        raise ValueError(f"psg_oracle_a8w8 rc={rc}")
    return {"acc_i32": acc_i, "acc_f32": acc_f, "c_bf16_bits": c}


def mxfp4(a_packed, b_shuf, sa_shuf, sb_shuf, m, n, k):
    a = np.ascontiguousarray(a_packed).view(np.uint8)
    b = np.ascontiguousarray(b_shuf).view(np.uint8)
    sa = np.ascontiguousarray(sa_shuf).view(np.uint8)
    sb = np.ascontiguousarray(sb_shuf).view(np.uint8)
    out = np.empty((m, n), np.float32)
    c = np.empty((m, n), np.uint16)
    f = lib().psg_oracle_mxfp4
    f.restype = ctypes.c_int
    rc = f(_p(a), _p(b), _p(sa), _p(sb), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k), _p(out), _p(c))
    if rc != 0:
        raise ValueError(f"psg_oracle_mxfp4 rc={rc}")
    return {"out_f32": out, "c_bf16_bits": c}


def run_torch_f32(a, b, sa, sb, kind):
    a = np.ascontiguousarray(a).view(np.uint8)
    b = np.ascontiguousarray(b).view(np.uint8)
    m, k = a.shape
    n = b.shape[0]
    sa = np.ascontiguousarray(sa, dtype=np.float32).reshape(-1)
    sb = np.ascontiguousarray(sb, dtype=np.float32).reshape(-1)
    c = np.empty((m, n), np.float32)
    f = lib().psg_oracle_run_torch_f32
    f.restype = ctypes.c_int
    rc = f(_p(a), _p(b), _p(sa), _p(sb), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
           ctypes.c_int(KIND[kind]), _p(c))
    if rc != 0:
        raise ValueError(f"psg_oracle_run_torch_f32 rc={rc}")
    return c


def num_threads() -> int:
    return int(lib().psg_oracle_num_threads())
