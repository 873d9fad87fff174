"""The decode loops' extraction sites (Rollout node.py:556-612, Judge node.py:325-374) on the batched sampler,
against the oracle's row-by-row restatement: token lists bit-exact, log-probs to 1e-4."""
import numpy as np
import pytest
import torch

import oracle
import tome_amd

pytestmark = pytest.mark.gpu
V = 3001


def _setup(dev, seed, B):
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((V, V)) * 2.5).astype(np.float32)        # next-token logits = row of the last token
    first = (rng.standard_normal((B, V)) * 2.5).astype(np.float32)
    Wt = torch.from_numpy(W).to(dev)
    return rng, W, first, (lambda toks: Wt[toks]), (lambda toks: W[np.asarray(toks)])


def _safe(run_oracle, rng, steps, rows, T, k, W, first, tries=50):
    """Uniforms for which no draw of the oracle run sits within 1e-4 of a CDF step (fp32 and fp64 sums may
    disagree there, and one different token changes the rest of the sequence)."""
    for _ in range(tries):
        us = rng.random((steps, rows)).astype(np.float32)
        seq = run_oracle(us)
        ok = True
        for b, s in enumerate(seq):
            rows_seen = [first[b * first.shape[0] // rows]] + [W[t] for t in s["tokens"][:-1]]
            for st, row in enumerate(rows_seen):
                _, val = oracle.top_k_rows(row[None].astype(np.float64), k)
                p = np.exp((val[0] - val[0, 0]) / T); cdf = np.cumsum(p) / p.sum()
                if np.abs(cdf - us[st, b]).min() < 1e-4:
                    ok = False
        if ok:
            return us, seq
    raise AssertionError("no safe uniforms found")


@pytest.mark.parametrize("T,G,eos", [(0.8, 3, 7), (1.0, 1, -1), (0.0, 2, 11)])
def test_rollout_decode_matches_oracle(dev, T, G, eos):
    rng, W, first, model_t, model_np = _setup(dev, 41, 4)
    max_tokens, k = 9, 20
    if eos >= 0:
        W[:, eos] += 4.0                                               # make EOS likely enough to end some sequences early
        model_t = (lambda Wt: (lambda toks: Wt[toks]))(torch.from_numpy(W).to(dev))
    run = lambda us: oracle.rollout_decode(model_np, first, G, T, max_tokens, eos, us, k)
    if T > 0:
        us, want = _safe(run, rng, max_tokens, 4 * G, T, k, W, first)
        src = lambda step, rows: torch.from_numpy(us[step])
    else:
        want, src = run(None), None
    got = tome_amd.rollout_decode(model_t, torch.from_numpy(first).to(dev), G, T, max_tokens, eos, top_k=k, uniform_source=src)
    assert [g["tokens"] for g in got] == [w["tokens"] for w in want]
    for g, w in zip(got, want):
        assert len(g["log_probs"]) == len(g["tokens"])
        np.testing.assert_allclose(g["log_probs"], w["log_probs"], atol=1e-4, rtol=0)
    if eos >= 0:
        assert any(g["tokens"][-1] == eos and len(g["tokens"]) < max_tokens for g in got)   # EOS kept (node.py:604-608)


@pytest.mark.parametrize("T,eos", [(0.9, 5), (0.0, 3)])
def test_judge_decode_matches_oracle(dev, T, eos):
    rng, W, first, _, model_np = _setup(dev, 43, 6)
    W[:, eos] += 4.0
    Wt = torch.from_numpy(W).to(dev)
    model_t = lambda toks: Wt[toks]
    max_tokens, k = 8, 20
    run = lambda us: oracle.judge_decode(model_np, first, T, max_tokens, eos, us, k)
    if T > 0:
        us, want = _safe(run, rng, max_tokens, 6, T, k, W, first)
        src = lambda step, rows: torch.from_numpy(us[step])
    else:
        want, src = run(None), None
    got = tome_amd.judge_decode(model_t, torch.from_numpy(first).to(dev), T, max_tokens, eos, top_k=k, uniform_source=src)
    assert [g["tokens"] for g in got] == [w["tokens"] for w in want]
    for g, w in zip(got, want):
        np.testing.assert_allclose(g["log_probs"], w["log_probs"], atol=1e-4, rtol=0)
    assert all(eos not in g["tokens"][1:] for g in got)                # EOS never recorded after the first token (node.py:369-370)
