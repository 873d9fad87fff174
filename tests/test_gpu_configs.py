"""GPU parity at the full sizes of the benchmark configurations (2, 4 and 5): size-independent properties on every row
plus the fp64 oracle on a sample of rows.  Inputs are generated on the GPU with the distributions the
configs name; sampled rows are copied back bit-exactly for the oracle."""
import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import V_QWEN3, bf16_bits_of

pytestmark = pytest.mark.gpu
V = V_QWEN3


def _first_argmax(x):
    """Index of the first maximum of every row, exactly (no reliance on a library argmax's tie rule)."""
    m = x.max(dim=-1, keepdim=True).values
    idx = torch.arange(x.shape[-1], device=x.device, dtype=torch.int32).expand_as(x)
    return torch.where(x == m, idx, torch.full_like(idx, x.shape[-1])).min(dim=-1).values


def test_config2_full_size(dev):
    """bf16 logits [8 x 512, 151936] ~ N(0, 3^2) + one +15 spike per row, 50 % spike targets, length mask."""
    g = torch.Generator(device=dev).manual_seed(22)
    G, L = 8, 512
    logits = torch.empty((G, L, V), device=dev, dtype=torch.bfloat16)
    for i in range(G):
        logits[i] = (torch.randn((L, V), device=dev, generator=g) * 3.0).to(torch.bfloat16)
    flat = logits.view(G * L, V)
    rows = torch.arange(G * L, device=dev)
    spike = torch.randint(0, V, (G * L,), device=dev, generator=g)
    flat[rows, spike] = (flat[rows, spike].float() + 15.0).to(torch.bfloat16)
    uniform = torch.randint(0, V, (G * L,), device=dev, generator=g)
    targets = torch.where(torch.rand(G * L, device=dev, generator=g) < 0.5, spike, uniform).to(torch.int32)
    lengths = torch.randint(64, 513, (G,), device=dev, generator=g)
    r = tome_amd.token_logprobs(logits, targets.view(G, L), 1.0, lengths=lengths, want_lse=True, want_argmax=True)
    full = tome_amd.token_logprobs(logits, targets.view(G, L), 1.0, want_lse=True, want_entropy=True, want_argmax=True)
    mask = (torch.arange(L, device=dev)[None, :] < lengths[:, None])
    # masked launch == unmasked launch on valid rows, zeros elsewhere
    assert torch.equal(r.lp[mask], full.lp[mask]) and torch.equal(r.argmax[mask], full.argmax[mask])
    assert (r.lp[~mask] == 0).all() and (r.lse[~mask] == 0).all() and (r.argmax[~mask] == -1).all()
    # properties on all 4096 rows
    lp, lse = full.lp.view(-1), full.lse.view(-1)
    assert torch.isfinite(lp).all() and (lp <= 1e-6).all()
    assert (full.entropy >= 0).all() and (full.entropy <= np.log(V) + 1e-4).all()
    picked = flat[rows, targets.long()].float()
    torch.testing.assert_close(lp, picked - lse, atol=1e-5, rtol=0)          # lp = x_t - lse, same lse
    want_amax = torch.empty(G * L, dtype=torch.int32, device=dev)
    for i in range(0, G * L, 512):
        want_amax[i:i + 512] = _first_argmax(flat[i:i + 512])
    assert torch.equal(full.argmax.view(-1), want_amax)                     # bit-exact, first maximum
    # oracle on a sample of rows
    sample = np.arange(0, G * L, 61)
    bits = bf16_bits_of(flat[torch.from_numpy(sample).to(dev)])
    t = targets.cpu().numpy()[sample]
    np.testing.assert_allclose(lp.cpu().numpy()[sample], oracle.logprob_rows(bits, t, 1.0), atol=1e-4, rtol=0)
    np.testing.assert_allclose(full.entropy.view(-1).cpu().numpy()[sample], oracle.entropy_rows(bits, 1.0), atol=1e-4, rtol=0)
    np.testing.assert_array_equal(full.argmax.view(-1).cpu().numpy()[sample], oracle.argmax_rows(bits))
    # the sampler over the same 4096 rows (streaming variant: rows too long to keep in registers): the greedy
    # id is the spike, the drawn id is a candidate, its log-prob is the row kernel's, candidates match the oracle
    us = torch.rand(G * L, device=dev, generator=g)
    s = tome_amd.sample_tokens(flat, 1.0, 20, uniforms=us, want_topk=True)
    assert torch.equal(s.argmax, want_amax) and torch.equal(s.topk_idx[:, 0], want_amax)
    assert (s.topk_idx == s.token[:, None]).any(dim=1).all()
    assert (s.topk_logit[:, :-1] >= s.topk_logit[:, 1:]).all()
    torch.testing.assert_close(s.lp, tome_amd.token_logprobs(flat, s.token, 1.0).lp, atol=2e-6, rtol=0)
    want_idx, _ = oracle.top_k_rows(bits, 20)
    np.testing.assert_array_equal(s.topk_idx.cpu().numpy()[sample], want_idx)


def _sample_stats(hidden2d, weight, targets, T, sample, dev):
    """fp64 oracle statistics for a sample of rows; the fp64 product of the exactly-upcast bf16
    inputs is taken with a library GEMM on the GPU, everything after it by the oracle."""
    idx = torch.from_numpy(sample).to(dev)
    logits64 = (hidden2d[idx].double() @ weight.double().t()).cpu().numpy()
    t = targets.reshape(-1).cpu().numpy()[sample]
    return {"lp": oracle.logprob_rows(logits64, t, T), "lse": oracle.lse_rows(logits64, T),
            "entropy": oracle.entropy_rows(logits64, T)}


def test_config4_full_size(dev):
    """hidden [16 x 1024, 2560], W [151936, 2560], T = 0.7, lengths ~ U[128, 1024]."""
    g = torch.Generator(device=dev).manual_seed(44)
    B, L, H, T = 16, 1024, 2560, 0.7
    hidden = torch.randn((B, L, H), device=dev, generator=g).to(torch.bfloat16)
    weight = (torch.randn((V, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    targets = torch.randint(0, V, (B, L), device=dev, generator=g).to(torch.int32)
    lengths = torch.randint(128, 1025, (B,), device=dev, generator=g)
    r = tome_amd.fused_lmhead_logprobs(hidden, weight, targets, T, lengths=lengths, want_lse=True, want_entropy=True)
    mask = (torch.arange(L, device=dev)[None, :] < lengths[:, None])
    assert (r.lp[~mask] == 0).all() and (r.entropy[~mask] == 0).all()
    assert torch.isfinite(r.lp).all() and (r.lp <= 1e-5).all()
    assert (r.entropy[mask] > 0).all() and (r.entropy <= np.log(V) + 1e-3).all()
    valid = torch.nonzero(mask.view(-1)).view(-1).cpu().numpy()
    sample = valid[:: max(1, len(valid) // 48)]
    want = _sample_stats(hidden.view(-1, H), weight, targets, T, sample, dev)
    np.testing.assert_allclose(r.lp.view(-1).cpu().numpy()[sample], want["lp"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.lse.view(-1).cpu().numpy()[sample], want["lse"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.entropy.view(-1).cpu().numpy()[sample], want["entropy"], atol=2e-3, rtol=0)
    # a row's result does not depend on which other rows are masked
    alone = tome_amd.fused_lmhead_logprobs(hidden, weight, targets, T, want_lse=True)
    torch.testing.assert_close(alone.lp[mask], r.lp[mask], atol=1e-5, rtol=0)


def test_config5_full_size(dev):
    """hidden [32 x 2048, 4096]; W_ref = bf16(W_pol + N(0, 0.002^2)); lp, ref_lp, k3, entropy."""
    g = torch.Generator(device=dev).manual_seed(55)
    B, L, H = 32, 2048, 4096
    hidden = torch.randn((B * L, H), device=dev, generator=g).to(torch.bfloat16)
    w32 = torch.randn((V, H), device=dev, generator=g) * 0.02
    w_pol = w32.to(torch.bfloat16)
    w32 += torch.randn((V, H), device=dev, generator=g) * 0.002
    w_ref = w32.to(torch.bfloat16)
    del w32
    targets = torch.randint(0, V, (B * L,), device=dev, generator=g).to(torch.int32)
    r = tome_amd.grpo_dual_logprobs(hidden, w_pol, w_ref, targets, 1.0)
    for o in r:
        assert o.shape == (B * L,) and torch.isfinite(o).all()
    assert (r.lp <= 1e-5).all() and (r.ref_lp <= 1e-5).all() and (r.k3 >= -1e-6).all()
    d = (r.ref_lp - r.lp).double()
    torch.testing.assert_close(r.k3.double(), torch.expm1(d) - d, atol=1e-5, rtol=0)   # k3 from its own lp pair
    sample = np.arange(0, B * L, B * L // 24)
    pol = _sample_stats(hidden, w_pol, targets, 1.0, sample, dev)
    ref = _sample_stats(hidden, w_ref, targets, 1.0, sample, dev)
    np.testing.assert_allclose(r.lp.cpu().numpy()[sample], pol["lp"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.ref_lp.cpu().numpy()[sample], ref["lp"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[sample], pol["entropy"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.k3.cpu().numpy()[sample], oracle.k3(pol["lp"], ref["lp"]), atol=4e-3, rtol=0)
