"""Build recipe for libtome_logprob.so (hipcc, gfx950 only)."""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libtome_logprob.so")
SOURCES = ["capi.hip", "row_logprob.hip", "row_sample.hip", "full_log_softmax.hip", "fused_lmhead.hip", "lora_merge.hip", "mfma_probe.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
    # hipcc -O3 would otherwise form packed-fp32 instructions from ordinary float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile every HIP source into the in-tree shared library and return its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *(extra_flags or []), "-o", LIB_PATH] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; drop that noise
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, extra_flags=sys.argv[1:]))
