"""GPU parity of the decode-step sampler (tome_row_sample) against the oracle's restatement of
_sample_token (mlx-impl/node.py:894-907): candidate sets and drawn ids bit-exact, log-probs to 1e-4."""
import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import V_QWEN3

pytestmark = pytest.mark.gpu


def _safe_uniforms(x64, T, k, rng):
    """Uniforms that stay clear of the CDF steps (fp32 vs fp64 cumulative sums may differ there)."""
    idx, val = oracle.top_k_rows(x64, k)
    us = np.empty(x64.shape[0], dtype=np.float32)
    for r in range(x64.shape[0]):
        n = int((idx[r] >= 0).sum())
        p = np.exp((val[r, :n] - val[r, 0]) / T)
        cdf = np.cumsum(p) / p.sum()
        while True:
            u = np.float32(rng.random())
            if np.abs(cdf - u).min() > 1e-4 and u < 1.0:
                us[r] = u
                break
    return us


@pytest.mark.parametrize("rows,V,dtype,T,k", [
    (64, V_QWEN3, torch.float32, 1.0, 20), (32, V_QWEN3, torch.bfloat16, 0.7, 20), (7, 4099, torch.float32, 1.3, 20),
    (5, 2048, torch.float32, 1.0, 5), (9, 2049, torch.bfloat16, 0.5, 32), (3, 17, torch.float32, 1.0, 20),
    (4, 300, torch.bfloat16, 2.0, 1), (130, 8191, torch.float32, 0.9, 20),
    # 512 rows and more: still cut into ranges of 8192 elements (fp32, and bf16 while the batch is small) ...
    (600, 30000, torch.float32, 1.0, 20), (700, 40000, torch.bfloat16, 0.8, 20),
])
def test_sampler_matches_oracle(dev, rows, V, dtype, T, k):
    rng = np.random.default_rng(rows * 31 + V)
    x = torch.from_numpy((rng.standard_normal((rows, V)) * 2.0).astype(np.float32)).to(dev).to(dtype)
    x64 = x.float().cpu().numpy().astype(np.float64)
    us = _safe_uniforms(x64, T, k, rng)
    got = tome_amd.sample_tokens(x, T, k, uniforms=torch.from_numpy(us).to(dev), want_topk=True)
    want_idx, want_val = oracle.top_k_rows(x64, k)
    want_tok, want_lp = oracle.sample_top_k(x64, us, T, k)
    np.testing.assert_array_equal(got.topk_idx.cpu().numpy(), want_idx)              # bit-exact candidates, in order
    np.testing.assert_array_equal(got.topk_logit.cpu().numpy()[want_idx >= 0], want_val[want_idx >= 0].astype(np.float32))
    np.testing.assert_array_equal(got.token.cpu().numpy(), want_tok)
    np.testing.assert_allclose(got.lp.cpu().numpy(), want_lp, atol=1e-4, rtol=0)
    np.testing.assert_array_equal(got.argmax.cpu().numpy(), np.argmax(x64, axis=-1))
    # the same pass must agree with the plain row kernel on the drawn ids
    lp2 = tome_amd.token_logprobs(x, got.token, T).lp
    np.testing.assert_allclose(got.lp.cpu().numpy(), lp2.cpu().numpy(), atol=2e-6, rtol=0)


@pytest.mark.parametrize("rows,V,dtype", [(2300, 65536, torch.float32), (1700, 32768, torch.bfloat16)])
def test_sampler_streams_large_batches(dev, rows, V, dtype):
    """Batches beyond ~950 fp32 / ~340 bf16 rows of 151936 (counted in ranges of 8192 elements) take one streaming
    workgroup per row; at that size the check runs on the GPU: the candidates' logits against torch.topk (values: ids
    may differ among equal logits), the greedy id against torch.argmax wherever the maximum is unique, the log-prob of
    the drawn id against the row kernel."""
    k = 20
    g = torch.Generator(device=dev).manual_seed(5)
    x = (torch.randn((rows, V), device=dev, generator=g) * 2.0).to(dtype)
    u = torch.rand(rows, device=dev, generator=g)
    got = tome_amd.sample_tokens(x, 1.1, k, uniforms=u, want_topk=True)
    vals, _ = torch.topk(x.float(), k, dim=-1)
    assert torch.equal(got.topk_logit, vals)
    assert torch.equal(x.float().gather(1, got.topk_idx.long()), vals)
    unique = vals[:, 0] > vals[:, 1]
    assert torch.equal(got.argmax[unique].long(), torch.argmax(x.float(), dim=-1)[unique])
    in_topk = (got.topk_idx == got.token[:, None]).any(dim=1)
    assert bool(in_topk.all())
    lp2 = tome_amd.token_logprobs(x, got.token, 1.1).lp
    np.testing.assert_allclose(got.lp.cpu().numpy(), lp2.cpu().numpy(), atol=2e-6, rtol=0)


def test_sampler_greedy_is_argmax_with_unit_temperature(dev):
    rng = np.random.default_rng(5)
    x = torch.from_numpy(rng.standard_normal((16, 5000)).astype(np.float32)).to(dev)
    got = tome_amd.sample_tokens(x, 0.0)                                              # node.py:896-897
    x64 = x.cpu().numpy().astype(np.float64)
    np.testing.assert_array_equal(got.token.cpu().numpy(), np.argmax(x64, -1))
    np.testing.assert_allclose(got.lp.cpu().numpy(), oracle.logprob_rows(x64, np.argmax(x64, -1), 1.0), atol=1e-4)


def test_sampler_ties_take_lower_ids_first(dev):
    V = 6000
    x = np.zeros((2, V), dtype=np.float32)
    x[0, [4000, 17, 2500]] = 5.0
    x[0, [5999, 3, 1234, 77]] = 3.0
    x[1, :] = 1.25                                                                     # all equal: candidates are ids 0..k-1
    got = tome_amd.sample_tokens(torch.from_numpy(x).to(dev), 1.0, 5, uniforms=[0.0, 0.999], want_topk=True)
    assert got.topk_idx.cpu().numpy().tolist() == [[17, 2500, 4000, 3, 77], [0, 1, 2, 3, 4]]
    assert got.token.cpu().numpy().tolist() == [17, 4]
    np.testing.assert_allclose(got.lp.cpu().numpy()[1], -np.log(V), atol=1e-4)


@pytest.mark.parametrize("pattern", ["ascending", "descending", "sawtooth", "one_lane"])
def test_sampler_adversarial_orderings(dev, pattern):
    """Orderings that defeat the first bound (the k-th largest lane maximum): the candidate buffer overflows
    and the kernel has to tighten the bound and rescan; the result must not change."""
    V, k = 151936, 20
    base = np.arange(V, dtype=np.float32) * 1e-4
    if pattern == "ascending":
        x = base
    elif pattern == "descending":
        x = base[::-1].copy()
    elif pattern == "sawtooth":
        x = (np.arange(V) % 4096).astype(np.float32) * 1e-3
    else:   # every large value sits in the load units of one lane (stride 256 units of 4 floats)
        x = np.full(V, -3.0, dtype=np.float32)
        x[(np.arange(V) // 4) % 256 == 5] = base[(np.arange(V) // 4) % 256 == 5]
    x2 = np.stack([x, x * 0.5])
    got = tome_amd.sample_tokens(torch.from_numpy(x2).to(dev), 1.0, k, uniforms=[0.37, 0.81], want_topk=True)
    want_idx, _ = oracle.top_k_rows(x2.astype(np.float64), k)
    np.testing.assert_array_equal(got.topk_idx.cpu().numpy(), want_idx)
    # uniforms may sit near a CDF step here (values differ by 1e-4): the drawn id must at least be a candidate
    tok = got.token.cpu().numpy()
    assert tok[0] in want_idx[0] and tok[1] in want_idx[1]
    lp = oracle.logprob_rows(x2.astype(np.float64), tok, 1.0)
    np.testing.assert_allclose(got.lp.cpu().numpy(), lp, atol=1e-4, rtol=0)


def test_sampler_law_of_the_draw(dev):
    """Over a fine grid of uniforms the drawn ids follow softmax(top-k logits / T): the categorical of node.py:906."""
    rng = np.random.default_rng(8)
    V, k, T, n = 3000, 6, 0.8, 8192
    row = (rng.standard_normal(V) * 2.0).astype(np.float32)
    x = torch.from_numpy(row).to(dev)[None, :].expand(n, V)                           # stride-0 rows: no copy
    us = torch.from_numpy(((np.arange(n) + 0.5) / n).astype(np.float32)).to(dev)
    got = tome_amd.sample_tokens(x.contiguous(), T, k, uniforms=us).token.cpu().numpy()
    idx, val = oracle.top_k_rows(row[None].astype(np.float64), k)
    p = np.exp(val[0] / T); p /= p.sum()
    freq = np.array([(got == i).mean() for i in idx[0]])
    np.testing.assert_allclose(freq, p, atol=2.0 / n + 1e-6)
    assert set(got.tolist()) <= set(idx[0].tolist())


@pytest.mark.parametrize("V", [4100, 151936])
def test_sampler_masks_nan_and_short_rows(dev, V):
    x = np.random.default_rng(2).standard_normal((5, V)).astype(np.float32)
    x[1, 10] = np.nan                                # NaN is never a candidate, but poisons the row's lse
    x[2, :] = -np.inf
    x[2, [5, 9]] = [1.0, 2.0]                        # only two logits above -inf: fewer than top_k
    x[4, :] = -np.inf                                # no candidate at all
    valid = torch.tensor([1, 1, 1, 0, 1], dtype=torch.int32, device=dev)
    got = tome_amd.sample_tokens(torch.from_numpy(x).to(dev), 1.0, 4, uniforms=[0.5, 0.5, 0.9, 0.5, 0.5], row_valid=valid,
                                 want_topk=True)
    tki, tkl = got.topk_idx.cpu().numpy(), got.topk_logit.cpu().numpy()
    tok, lp = got.token.cpu().numpy(), got.lp.cpu().numpy()
    want_idx, _ = oracle.top_k_rows(x.astype(np.float64), 4)
    np.testing.assert_array_equal(tki[[0, 2, 4]], want_idx[[0, 2, 4]])                # -inf logits are not listed
    assert 10 not in tki[1] and np.isnan(lp[1])
    assert tki[2].tolist() == [9, 5, -1, -1] and tkl[2].tolist() == [2.0, 1.0, 0.0, 0.0]
    assert tok[2] == 5                                                                 # masses e^2 : e^1 -> 0.9 falls on id 5
    want_tok, want_lp = oracle.sample_top_k(x[2:3].astype(np.float64), [0.9], 1.0, 4)
    assert tok[2] == want_tok[0] and abs(lp[2] - want_lp[0]) < 1e-4
    assert tok[3] == -1 and lp[3] == 0 and (tki[3] == -1).all()
    assert tok[4] == -1 and np.isnan(lp[4]) and (tki[4] == -1).all()                  # all -inf: no token


def test_sampler_strided_and_unaligned_rows(dev):
    rng = np.random.default_rng(3)
    big = torch.from_numpy(rng.standard_normal((6, 2, 5003)).astype(np.float32)).to(dev)
    view = big[:, 1, 1:5002]                          # row stride 10006, base offset 4 bytes off 16
    x64 = view.cpu().numpy().astype(np.float64)
    us = _safe_uniforms(x64, 1.0, 20, rng)
    got = tome_amd.sample_tokens(view, 1.0, 20, uniforms=torch.from_numpy(us).to(dev), want_topk=True)
    want_idx, _ = oracle.top_k_rows(x64, 20)
    want_tok, want_lp = oracle.sample_top_k(x64, us, 1.0, 20)
    np.testing.assert_array_equal(got.topk_idx.cpu().numpy(), want_idx)
    np.testing.assert_array_equal(got.token.cpu().numpy(), want_tok)
    np.testing.assert_allclose(got.lp.cpu().numpy(), want_lp, atol=1e-4, rtol=0)


def test_decode_step_graph_replays_match_eager(dev):
    """The sampler captured as a HIP graph: several replays on changing inputs, with eager work and
    synchronisations between them, each compared with the eager call on the same inputs."""
    rng = np.random.default_rng(12)
    rows, V = 48, 30011
    logits = torch.zeros((rows, V), dtype=torch.float32, device=dev)
    step = tome_amd.DecodeStepGraph(logits, 0.8, 20)
    for it in range(4):
        x = torch.from_numpy((rng.standard_normal((rows, V)) * (1.0 + it)).astype(np.float32)).to(dev)
        u = torch.from_numpy(rng.random(rows).astype(np.float32)).to(dev)
        step.logits.copy_(x)
        step.uniforms.copy_(u)
        got = step.replay()
        torch.cuda.synchronize()
        tok, lp, amax = got.token.clone(), got.lp.clone(), got.argmax.clone()
        want = tome_amd.sample_tokens(x, 0.8, 20, uniforms=u)                 # eager, on the same inputs
        torch.cuda.synchronize()
        assert torch.equal(tok, want.token) and torch.equal(amax, want.argmax)
        assert torch.equal(lp, want.lp)                                        # same kernels, same order: bit-identical
        # unrelated eager work between replays
        (x @ x[:8].T).sum().item()
    x64 = x.cpu().numpy().astype(np.float64)
    np.testing.assert_array_equal(amax.cpu().numpy(), np.argmax(x64, -1))
