"""Seeded random sweep over shapes, strides, masks and temperatures: every entry point against the oracle.
Sizes are kept small enough for the fp64 oracle; the point is coverage of tile edges, ragged sizes, schedule
regimes and mask patterns that the hand-picked cases may have missed."""
import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import bf16_bits_of, check_argmax

pytestmark = pytest.mark.gpu


def _mask(rng, n, kind):
    if kind == "none":
        return None
    if kind == "random":
        m = (rng.random(n) < rng.uniform(0.1, 0.9)).astype(np.int32)
    elif kind == "prefix":
        m = (np.arange(n) < rng.integers(1, n + 1)).astype(np.int32)
    else:   # "segments": valid prefixes of fixed-length sequences, like completion rows of a padded batch
        L = int(rng.integers(8, 65))
        lens = rng.integers(0, L + 1, size=(n + L - 1) // L)
        m = (np.arange(n) % L < np.repeat(lens, L)[:n]).astype(np.int32)
    if m.sum() == 0:
        m[int(rng.integers(0, n))] = 1
    return m


@pytest.mark.parametrize("seed", range(24))
def test_sweep_fused(dev, seed):
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.choice([1, 3, 64, 127, 128, 129, 255, 256, 257, 300, 513, 700, 1100, 2500]))
    H = int(rng.choice([8, 24, 64, 72, 128, 192, 256, 320, 1024]))
    V = int(rng.integers(17, 6000)) if H <= 320 else int(rng.integers(300, 1500))
    T = float(rng.choice([0.5, 0.7, 1.0, 1.3, 2.0]))
    kind = str(rng.choice(["none", "random", "prefix", "segments"]))
    h = torch.from_numpy(rng.standard_normal((n, H)).astype(np.float32)).to(dev).to(torch.bfloat16)
    w = torch.from_numpy((rng.standard_normal((V, H)) * rng.uniform(0.02, 0.3)).astype(np.float32)).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    m = _mask(rng, n, kind)
    rv = None if m is None else torch.from_numpy(m).to(dev)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), T, row_valid=rv, want_lse=True, want_entropy=True,
                                       want_argmax=True)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, T)
    mb = np.ones(n, bool) if m is None else m.astype(bool)
    for name, got in (("lp", r.lp), ("lse", r.lse), ("entropy", r.entropy)):
        np.testing.assert_allclose(got.cpu().numpy()[mb], want[name][mb], atol=2e-3, rtol=0, err_msg=f"{name} n={n} H={H} V={V} {kind}")
    check_argmax(h, w, r.argmax.cpu().numpy(), want, T, rows=np.flatnonzero(mb), min_clear=0.0)
    assert (r.lp.cpu().numpy()[~mb] == 0).all() and (r.argmax.cpu().numpy()[~mb] == -1).all()


@pytest.mark.parametrize("seed", range(16))
def test_sweep_rows_and_sampler(dev, seed):
    rng = np.random.default_rng(2000 + seed)
    rows = int(rng.choice([1, 2, 7, 33, 64, 200, 513]))
    V = int(rng.choice([5, 16, 17, 255, 1024, 2048, 2049, 4096, 4097, 8191, 12345, 40000]))
    dtype = torch.float32 if rng.random() < 0.5 else torch.bfloat16
    T = float(rng.choice([0.6, 1.0, 1.7]))
    pad = int(rng.choice([0, 0, 1, 8, 24]))                    # row stride V + pad: aligned and unaligned rows
    off = int(rng.choice([0, 0, 1, 4]))                        # first column of the view
    base = torch.from_numpy((rng.standard_normal((rows, V + pad + off)) * 2.5).astype(np.float32)).to(dev).to(dtype)
    x = base[:, off:off + V]
    x64 = x.float().cpu().numpy().astype(np.float64)
    t = rng.integers(0, V, size=rows).astype(np.int32)
    m = _mask(rng, rows, str(rng.choice(["none", "random", "prefix"])))
    rv = None if m is None else torch.from_numpy(m).to(dev)
    mb = np.ones(rows, bool) if m is None else m.astype(bool)
    r = tome_amd.token_logprobs(x, torch.from_numpy(t).to(dev), T, row_valid=rv, want_lse=True, want_entropy=True, want_argmax=True)
    np.testing.assert_allclose(r.lp.cpu().numpy()[mb], oracle.logprob_rows(x64, t, T)[mb], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy()[mb], oracle.lse_rows(x64, T)[mb], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[mb], oracle.entropy_rows(x64, T)[mb], atol=1e-4, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy()[mb], oracle.argmax_rows(x64)[mb])
    # sampler on the same rows: candidates and greedy ids bit-exact, log-prob of the drawn id to 1e-4
    k = int(rng.choice([1, 5, 20, 32]))
    us = rng.random(rows).astype(np.float32)
    s = tome_amd.sample_tokens(x, T, k, uniforms=torch.from_numpy(us).to(dev), row_valid=rv, want_topk=True)
    want_idx, _ = oracle.top_k_rows(x64, k)
    np.testing.assert_array_equal(s.topk_idx.cpu().numpy()[mb], want_idx[mb])
    tok = s.token.cpu().numpy()
    assert all(tok[i] in want_idx[i] for i in np.flatnonzero(mb)) and (tok[~mb] == -1).all()
    np.testing.assert_allclose(s.lp.cpu().numpy()[mb], oracle.logprob_rows(x64, np.where(mb, tok, 0), T)[mb], atol=1e-4, rtol=0)
    np.testing.assert_array_equal(s.argmax.cpu().numpy()[mb], oracle.argmax_rows(x64)[mb])


@pytest.mark.parametrize("seed", range(20))
def test_sweep_fused_decode_batches(dev, seed):
    """<= 64 tokens over hidden sizes on and off the streaming kernel's shape rules (K slices of 256 / 512 over 2..8
    waves), ragged vocabularies (partial last 16-row tile, fewer tiles than CUs), masks, strided hidden states."""
    rng = np.random.default_rng(5000 + seed)
    n = int(rng.integers(1, 65))
    H = int(rng.choice([512, 768, 1024, 1280, 1536, 2048, 2304, 2560, 3072, 4096, 320]))
    V = int(rng.choice([64, 65, 100, 257, 1000, 4095, 4100, 9001]))
    T = float(rng.choice([0.5, 0.7, 1.0, 1.6]))
    kind = str(rng.choice(["none", "random", "prefix"]))
    pad = int(rng.choice([0, 0, 8, 64]))
    base = torch.from_numpy(rng.standard_normal((n, H + pad)).astype(np.float32)).to(dev).to(torch.bfloat16)
    h = base[:, :H]
    w = torch.from_numpy((rng.standard_normal((V, H)) * rng.uniform(0.01, 0.08)).astype(np.float32)).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    m = _mask(rng, n, kind)
    rv = None if m is None else torch.from_numpy(m).to(dev)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), T, row_valid=rv, want_lse=True, want_entropy=True,
                                       want_argmax=True)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, T)
    mb = np.ones(n, bool) if m is None else m.astype(bool)
    tag = f"n={n} H={H} V={V} {kind} pad={pad}"
    for name, got in (("lp", r.lp), ("lse", r.lse), ("entropy", r.entropy)):
        np.testing.assert_allclose(got.cpu().numpy()[mb], want[name][mb], atol=2e-3, rtol=0, err_msg=f"{name} {tag}")
    clear = mb & ((want["top1"] - want["top2"]) > 1e-2)
    np.testing.assert_array_equal(r.argmax.cpu().numpy()[clear], want["argmax"][clear], err_msg=tag)
    assert (r.lp.cpu().numpy()[~mb] == 0).all() and (r.argmax.cpu().numpy()[~mb] == -1).all()
    lp_only = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), T, row_valid=rv).lp
    np.testing.assert_allclose(lp_only.cpu().numpy()[mb], want["lp"][mb], atol=2e-3, rtol=0, err_msg=tag)


@pytest.mark.parametrize("seed", range(12))
def test_sweep_lora_merge(dev, seed):
    """Random batches of merges (ranks 8..128, ragged rows and columns, strides, base-only jobs) on inputs whose
    rank-long sums are exact in fp32: bit-exact against the oracle."""
    from tome_amd import weights
    rng = np.random.default_rng(6000 + seed)
    to_dev = lambda b: torch.from_numpy(b.view(np.int16).copy()).to(dev).view(torch.bfloat16)
    jobs, want, outs = [], [], []
    for _ in range(int(rng.integers(1, 9))):
        rows = int(rng.choice([1, 15, 16, 17, 100, 255, 512, 700]))
        cols = 8 * int(rng.choice([1, 2, 31, 32, 63, 64, 65, 129, 200, 385]))
        rank = int(rng.choice([8, 16, 24, 32, 40, 64, 96, 128]))
        scale = float(rng.choice([2.5, 1.0, 0.3, -2.0, 20.0 / 8]))
        base = oracle.bf16_round((rng.standard_normal((rows, cols)) * 0.05).astype(np.float32))
        a = oracle.bf16_round((rng.integers(-8, 9, size=(rank, cols)) / 16).astype(np.float32))
        b = oracle.bf16_round((rng.integers(-8, 9, size=(rows, rank)) / 16).astype(np.float32))
        spad = 8 * int(rng.integers(0, 3))
        bt = torch.zeros((rows, cols + spad), device=dev, dtype=torch.bfloat16)
        bt[:, :cols] = to_dev(base)
        ot = torch.full((rows, cols + 8), 9.0, device=dev, dtype=torch.bfloat16)
        if rng.random() < 0.2:
            jobs.append((bt[:, :cols], ot[:, :cols], None, None, 1.0))
            want.append(base)
        else:
            jobs.append((bt[:, :cols], ot[:, :cols], to_dev(a), to_dev(b), scale))
            want.append(oracle.lora_merge_bf16(base, a, b, scale))
        outs.append((ot, cols))
    weights.lora_merge(jobs)
    for i, ((ot, cols), w) in enumerate(zip(outs, want)):
        np.testing.assert_array_equal(bf16_bits_of(ot[:, :cols]), w, err_msg=f"seed {seed} job {i} shape {w.shape}")
        assert (ot[:, cols:].float() == 9.0).all()
