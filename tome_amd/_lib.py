"""ctypes binding of libtome_logprob.so (the C ABI declared in include/tome_logprob.h)."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG_DIR, "libtome_logprob.so")
_lib: ctypes.CDLL | None = None

TOME_F32, TOME_BF16 = 0, 1
ABI_VERSION = 3

# name -> (restype, argtypes); must list every function the header declares.
SIGNATURES = {
    "tome_abi_version": (c_int, []),
    "tome_strerror": (c_char_p, [c_int]),
    "tome_last_hip_error": (c_int, []),
    "tome_row_logprob_workspace": (c_size_t, [c_int64, c_int64]),
    "tome_row_logprob": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_float,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tome_row_logprob_rows": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_float,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tome_row_logprob_noalloc": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_float,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "tome_row_logprob_noalloc_limit": (c_size_t, [c_size_t]),
    "tome_row_sample_workspace": (c_size_t, [c_int, c_int64, c_int64, c_int]),
    "tome_row_sample": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_float, c_int,
                                c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                c_void_p]),
    "tome_full_log_softmax": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_float,
                                      c_void_p, c_void_p, c_size_t, c_void_p]),
    "tome_select_fused_kernel": (None, [c_int]),
    "tome_fused_lmhead_logprob_workspace": (c_size_t, [c_int64, c_int64, c_int64]),
    "tome_fused_lmhead_logprob": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                          c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_size_t, c_void_p]),
    "tome_norm_lmhead_logprob_workspace": (c_size_t, [c_int64, c_int64, c_int64]),
    "tome_norm_lmhead_logprob": (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                         c_int64, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_size_t, c_void_p]),
    "tome_grpo_dual_workspace": (c_size_t, [c_int64, c_int64, c_int64]),
    "tome_grpo_dual": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                               c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_size_t, c_void_p]),
    "tome_grpo_pair_workspace": (c_size_t, [c_int64, c_int64, c_int64, c_int]),
    "tome_grpo_pair": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                               c_int64, c_int64, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_size_t, c_void_p]),
    "tome_probe_mfma_ceiling": (c_int, [c_void_p, c_size_t, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "tome_lora_merge_workspace": (c_size_t, [c_void_p, c_int64]),
    "tome_lora_merge": (c_int, [c_void_p, c_int64, c_void_p, c_size_t, c_void_p]),
}


class TomeLoraJob(ctypes.Structure):
    """``TomeLoraJob`` of include/tome_logprob.h."""
    _fields_ = [("base", c_void_p), ("out", c_void_p), ("lora_a", c_void_p), ("lora_b", c_void_p),
                ("rows", c_int64), ("cols", c_int64), ("rank", c_int64), ("base_stride", c_int64),
                ("out_stride", c_int64), ("scale", c_float), ("reserved", ctypes.c_int32)]


class TomeError(RuntimeError):
    """A C-ABI call returned a negative TOME_E_* code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libtome_logprob: {message} (code {code})")
        self.code = code


def lib_path() -> str:
    return _LIB_PATH


def load_library() -> ctypes.CDLL:
    """Load the in-tree shared library; raise (never fall back) if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: build it with `python -m tome_amd.build` "
            "(hipcc --offload-arch=gfx950).  tome_amd has no CPU fallback.")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.tome_abi_version() != ABI_VERSION:
        raise ImportError(f"ABI version mismatch: library {lib.tome_abi_version()}, binding {ABI_VERSION}")
    _lib = lib
    return lib


def check(code: int) -> None:
    if code == 0:
        return
    lib = load_library()
    msg = lib.tome_strerror(code).decode()
    if code == -7:
        msg += f" [hipError_t {lib.tome_last_hip_error()}]"
    if code in (-1, -2, -3, -5, -6, -8):
        raise ValueError(f"libtome_logprob: {msg} (code {code})")
    raise TomeError(code, msg)
