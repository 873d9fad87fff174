"""The C-ABI library loads, exports everything include/tome_logprob.h declares, and rejects bad
arguments on the host before any GPU work (so these run without a GPU)."""
import ctypes
import os
import re

import pytest

import tome_amd
from tome_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tome_logprob.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tome_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert "tome_row_logprob" in names and "tome_fused_lmhead_logprob" in names and "tome_grpo_dual" in names
    assert sorted(_lib.SIGNATURES) == names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(tome_amd.lib_path())
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert tome_amd.load_library().tome_abi_version() == 3


def test_header_cites_reference_for_each_entry_point():
    text = open(HEADER).read()
    for ref in ("mlx-impl/node.py:400-404", "mlx-impl/model.py:77-89", "mlx-impl/model.py:538"):
        assert ref in text


def test_strerror_and_codes():
    lib = tome_amd.load_library()
    assert lib.tome_strerror(0) == b"ok"
    for code in range(-8, 0):
        assert lib.tome_strerror(code) not in (b"ok", b"unknown error code")
    assert lib.tome_strerror(-99) == b"unknown error code"


def test_workspace_queries():
    lib = tome_amd.load_library()
    assert lib.tome_row_logprob_workspace(4096, 151936) == 0          # one workgroup per row
    small = lib.tome_row_logprob_workspace(64, 151936)
    assert small > 0 and small % 256 == 0
    assert lib.tome_row_logprob_workspace(0, 151936) == 0
    one = lib.tome_fused_lmhead_logprob_workspace(4096, 1024, 151936)
    two = lib.tome_grpo_dual_workspace(4096, 1024, 151936)
    assert 0 < one < two and one % 256 == 0
    normed = lib.tome_norm_lmhead_logprob_workspace(4096, 1024, 151936)
    assert normed >= one + 4096 * 1024 * 2 and normed % 256 == 0      # room for the normalised rows


def test_argument_checks_run_on_host():
    """Every call below must return before touching the GPU (pointers are fake but non-NULL)."""
    lib = tome_amd.load_library()
    P = 0x1000  # 16-byte aligned dummy
    row = lambda **k: lib.tome_row_logprob(k.get("logits", P), k.get("dtype", 1), k.get("rows", 4), k.get("V", 64),
                                           k.get("stride", 64), k.get("targets", P), None, k.get("T", 1.0),
                                           k.get("lp", P), None, None, None, None, 0, None)
    assert row(dtype=7) == -2
    assert row(V=0) == -3 and row(rows=-1) == -3 and row(stride=63) == -3
    assert row(T=0.0) == -5 and row(T=-1.0) == -5 and row(T=float("nan")) == -5 and row(T=float("inf")) == -5
    assert row(logits=None) == -1 and row(targets=None) == -1
    assert row(lp=None) == -1                      # no output requested at all
    assert row(rows=0) == 0                        # empty batch is a no-op
    assert row(rows=64, V=151936, stride=151936) == -4   # split rows need a workspace
    assert row(logits=P + 1) == -6
    na = lambda **k: lib.tome_row_logprob_noalloc(k.get("logits", P), k.get("dtype", 1), k.get("rows", 4), k.get("V", 64),
                                                  k.get("stride", 64), k.get("targets", P), None, k.get("T", 1.0),
                                                  k.get("lp", P), None, None, None, None)
    assert na(dtype=7) == -2 and na(V=0) == -3 and na(stride=63) == -3 and na(T=0.0) == -5
    assert na(logits=None) == -1 and na(targets=None) == -1 and na(lp=None) == -1 and na(rows=0) == 0
    assert na(logits=P + 1) == -6
    # TOME_E_SCRATCH: no shape needs more than 16 KiB of the 64 KiB array, so the limit is lowered to reach the path
    assert lib.tome_row_logprob_noalloc_limit(4096) == 4096
    try:
        assert na(rows=300, V=151936, stride=151936) == -8           # 300 rows x 2 splits x 16 B of partials > 4096
        assert na(rows=300, V=151936, stride=151936, logits=None) == -1   # argument checks still come first
        with pytest.raises(ValueError, match="scratch"):
            _lib.check(-8)
    finally:
        assert lib.tome_row_logprob_noalloc_limit(0) == 64 * 1024   # 0 restores the whole array
    assert lib.tome_row_logprob_noalloc_limit(1 << 30) == 64 * 1024  # and nothing raises it beyond the array
    rl = lambda **k: lib.tome_row_logprob_rows(k.get("logits", P), k.get("dtype", 1), k.get("rows", 4), k.get("V", 64),
                                               k.get("stride", 64), k.get("idx", P), k.get("n", 3), k.get("targets", P),
                                               k.get("T", 1.0), k.get("lp", P), None, None, None, None, 0, None)
    assert rl(dtype=7) == -2 and rl(V=0) == -3 and rl(stride=63) == -3 and rl(n=-1) == -3 and rl(rows=-1) == -3
    assert rl(T=0.0) == -5 and rl(logits=None) == -1 and rl(idx=None) == -1 and rl(targets=None) == -1 and rl(lp=None) == -1
    assert rl(n=0) == 0 and rl(logits=P + 1) == -6
    assert rl(rows=4096, V=151936, stride=151936, n=64) == -4        # 64 listed rows are split: workspace needed
    fused = lambda **k: lib.tome_fused_lmhead_logprob(k.get("h", P), k.get("w", P), k.get("n", 8), k.get("H", 64),
                                                      k.get("V", 100), k.get("hs", 64), k.get("ws", 64), P, None,
                                                      k.get("T", 1.0), k.get("lp", P), None, None, None, None, 0, None)
    assert fused(H=0) == -3 and fused(hs=32) == -3 and fused(T=0.0) == -5
    assert fused(H=60, hs=60, ws=60) == -6 and fused(h=P + 2) == -6
    assert fused(h=None) == -1 and fused(n=0) == 0
    assert fused(n=1 << 25, H=72, hs=72, ws=72) == -3                # generic kernel (H % 64 != 0): > 4 GiB of hidden
    assert fused(n=1 << 20, H=4096, hs=4096, ws=4096) == -4          # the other kernels take it (64-bit addresses)
    assert fused(hs=1 << 31) == -3 and fused(ws=1 << 40) == -3       # strides are 32-bit byte counts
    assert fused() == -4                                             # workspace missing
    norm = lambda **k: lib.tome_norm_lmhead_logprob(P, k.get("nw", P), k.get("eps", 1e-6), P, 8, k.get("H", 64), 100, 64, 64,
                                                    P, None, 1.0, P, None, None, None, None, 0, None)
    assert norm(nw=None) == -1 and norm(nw=P + 4) == -6 and norm(eps=-1.0) == -3 and norm(eps=float("nan")) == -3
    assert norm(H=0) == -3 and norm() == -4
    samp = lambda **k: lib.tome_row_sample(k.get("logits", P), k.get("dtype", 0), 4, k.get("V", 64), max(64, k.get("V", 64)), None, None, k.get("T", 1.0),
                                           k.get("k", 20), k.get("tok", P), None, None, None, None, None, None, 0, None)
    assert samp(dtype=3) == -2 and samp(V=0) == -3 and samp(k=0) == -3 and samp(k=33) == -3 and samp(T=0.0) == -5
    assert samp(logits=None) == -1 and samp(tok=None) == -1 and samp(logits=P + 2) == -6
    assert samp(V=151936) == -4                                      # a small batch splits its rows: workspace needed
    assert lib.tome_row_sample_workspace(0, 4096, 151936, 20) == 0 and lib.tome_row_sample_workspace(0, 64, 151936, 20) > 0
    dual = lib.tome_grpo_dual(P, P, None, 8, 64, 100, 64, 64, P, None, 1.0, P, P, P, P, None, 0, None)
    assert dual == -1
    pair = lambda **k: lib.tome_grpo_pair(P, k.get("href", P), k.get("nw", None), k.get("eps", 1e-6), P, k.get("wref", P), 8, 64,
                                          100, 64, 64, P, None, k.get("T", 1.0), P, k.get("ref_lp", P), P, P, None, 0, None)
    assert pair(href=None) == -1 and pair(wref=None) == -1 and pair(ref_lp=None) == -1
    assert pair(href=P + 2) == -6 and pair(nw=P + 8) == -6 and pair(nw=P, eps=-1.0) == -3 and pair(T=0.0) == -5
    assert pair() == -4
    assert lib.tome_grpo_pair_workspace(4096, 1024, 151936, 0) == lib.tome_grpo_dual_workspace(4096, 1024, 151936)
    assert lib.tome_grpo_pair_workspace(4096, 1024, 151936, 1) >= lib.tome_grpo_dual_workspace(4096, 1024, 151936) + 2 * 4096 * 1024 * 2

    probe = lambda **k: lib.tome_probe_mfma_ceiling(k.get("ops", P), k.get("ob", 65536), k.get("wg", 256), k.get("steps", 16),
                                                    k.get("flags", 0), k.get("sink", P), k.get("sb", 256 * 512 * 4), None)
    assert probe(ops=None) == -1 and probe(sink=None) == -1 and probe(ops=P + 4) == -6
    assert probe(ob=65535) == -3 and probe(sb=256 * 512 * 4 - 1) == -3          # buffers smaller than the kernel touches
    assert probe(wg=0) == -3 and probe(wg=4097) == -3 and probe(steps=0) == -3 and probe(steps=65537) == -3
    assert probe(flags=8) == -3 and probe(flags=-1) == -3

    def merge(**k):
        j = _lib.TomeLoraJob()
        j.base, j.out, j.lora_a, j.lora_b = k.get("base", P), k.get("out", P), k.get("a", P), k.get("b", P)
        j.rows, j.cols, j.rank = k.get("rows", 32), k.get("cols", 64), k.get("rank", 8)
        j.base_stride, j.out_stride, j.scale = k.get("bs", 64), k.get("os", 64), k.get("scale", 2.5)
        jp = ctypes.cast(ctypes.pointer(j), ctypes.c_void_p)
        if k.get("query"):
            return lib.tome_lora_merge_workspace(jp, k.get("n", 1))
        return lib.tome_lora_merge(jp, k.get("n", 1), k.get("ws", P), k.get("wsb", 1 << 20), None)
    assert merge(n=0) == 0 and merge(n=-1) == -3
    assert lib.tome_lora_merge(None, 1, None, 0, None) == -1
    table = 256                                    # the job table, rounded up
    assert merge(query=True) == table + 64 * 32 * 2
    assert merge(query=True, rank=40, cols=1024, bs=1024, os=1024) == table + 1024 * 64 * 2
    assert merge(query=True, a=None, b=None) == table and merge(query=True, rank=12) == 0
    assert merge(ws=None) == -4 and merge(wsb=100) == -4 and merge(ws=P + 4) == -6
    assert merge(base=None) == -1 and merge(out=None) == -1 and merge(a=None) == -1 and merge(b=None) == -1
    assert merge(rows=-1) == -3 and merge(cols=0) == -3 and merge(bs=56) == -3 and merge(os=8) == -3
    assert merge(rank=0) == -3 and merge(rank=136) == -3 and merge(scale=float("inf")) == -3
    assert merge(rank=12) == -6 and merge(cols=60, bs=64) == -6 and merge(bs=68) == -6 and merge(base=P + 8) == -6
    assert merge(b=P + 4) == -6


def test_check_maps_codes_to_exceptions():
    with pytest.raises(ValueError):
        _lib.check(-3)
    with pytest.raises(tome_amd.TomeError) as e:
        _lib.check(-4)
    assert e.value.code == -4
    _lib.check(0)


def test_header_is_plain_c():
    """The boundary is a C ABI: the header must compile as C99 on its own, with no C++ or HIP types."""
    import subprocess
    hdr = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "tome_logprob.h")
    src = '#include "%s"\nint main(void) { return tome_abi_version() == TOME_ABI_VERSION ? 0 : 1; }\n' % hdr
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-x", "c", "-"],
                       input=src, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
