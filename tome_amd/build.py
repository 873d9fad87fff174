"""Build recipe for libtome_logprob.so (hipcc, gfx950 only)."""
from __future__ import annotations

import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libtome_logprob.so")
SOURCES = ["capi.hip", "row_logprob.hip", "row_sample.hip", "full_log_softmax.hip", "fused_lmhead.hip", "lora_merge.hip", "mfma_probe.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # hipcc -O3 would otherwise form packed-fp32 instructions from ordinary float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; drop that noise
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, extra_flags: list[str] | None = None, out: str | None = None) -> str:
    """Compile every HIP source (one hipcc process per file, side by side) and link the in-tree shared library;
    returns its path.  Objects go to a temporary directory and nothing but the library is left behind."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    out = out or LIB_PATH
    flags = HIPCC_FLAGS + list(extra_flags or [])
    jobs = max(1, min(len(SOURCES), int(os.environ.get("MAX_JOBS", os.cpu_count() or 1))))
    with tempfile.TemporaryDirectory(prefix="tome_build_") as tmp:
        objs = [os.path.join(tmp, s.replace(".hip", ".o")) for s in SOURCES]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(lambda so: _run([hipcc, *flags, "-c", os.path.join(CSRC, so[0]), "-o", so[1]], verbose),
                          zip(SOURCES, objs)))
        _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-fno-gpu-rdc", "-o", out, *objs], verbose)
    return out


if __name__ == "__main__":
    print(build(verbose=True, extra_flags=sys.argv[1:]))
