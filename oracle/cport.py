"""ctypes loader for oracle/liboracle_metal.so.  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle_metal.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "liboracle_metal.so"], check=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.tome_oracle_metal_log_softmax.restype = ctypes.c_int
        _lib.tome_oracle_metal_log_softmax.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_float]
        _lib.tome_oracle_local_compute_logprobs.restype = ctypes.c_int
        _lib.tome_oracle_local_compute_logprobs.argtypes = [
            ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
            ctypes.c_float, ctypes.c_void_p]
    return _lib


def _dtype_code(a: np.ndarray) -> int:
    if a.dtype == np.float32:
        return 0
    if a.dtype == np.uint16:
        return 1
    raise TypeError("float32 or bf16 bit patterns (uint16) expected")


def metal_log_softmax(logits: np.ndarray, temperature: float = 1.0) -> np.ndarray:
    """Thread-faithful C restatement of mlx-impl/model.py:16-66; out dtype = in dtype."""
    x = np.ascontiguousarray(logits)
    flat = x.reshape(-1, x.shape[-1])
    out = np.empty_like(flat)
    rc = lib().tome_oracle_metal_log_softmax(flat.ctypes.data, out.ctypes.data, _dtype_code(flat),
                                             flat.shape[0], flat.shape[1], float(temperature))
    if rc != 0:
        raise ValueError("bad arguments")
    return out.reshape(x.shape)


def local_compute_logprobs_c(logits: np.ndarray, ids: np.ndarray, temp: float) -> np.ndarray:
    """mlx-impl/node.py:400-404 in scalar C with OpenMP over rows."""
    x = np.ascontiguousarray(logits)
    flat = x.reshape(-1, x.shape[-1])
    t = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
    out = np.empty(flat.shape[0], dtype=np.float32)
    rc = lib().tome_oracle_local_compute_logprobs(flat.ctypes.data, _dtype_code(flat), flat.shape[0],
                                                  flat.shape[1], t.ctypes.data, float(temp), out.ctypes.data)
    if rc != 0:
        raise ValueError("bad arguments")
    return out
