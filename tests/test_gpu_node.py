"""GPU: the ref-logprob entry (RefLogprobServicer) against the oracle's restatement of node.py:391-461,
and the HIP kernels against the committed golden vectors."""
import asyncio
import copy

import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import bf16_bits_of
from golden_util import load, seeded_case
from test_host_logic import V_STUB, make_batch, stub_logits

pytestmark = pytest.mark.gpu
G = load()


def _torch_model(dev, dtype, calls):
    def model(full_ids, cache=None):
        assert cache is None and full_ids.dtype == torch.int64 and full_ids.is_cuda
        calls.append(tuple(full_ids.shape))
        logits = torch.from_numpy(stub_logits(full_ids.cpu().numpy().astype(np.uint32))).to(dev).to(dtype)
        return logits, None
    return model


@pytest.mark.parametrize("T,batch,dtype", [(1.0, 32, torch.bfloat16), (0.7, 4, torch.float32), (0.0, 1, torch.bfloat16)])
def test_entry_matches_oracle_entry(dev, T, batch, dtype):
    prompts, results = make_batch(seed=3, n_prompts=6, G=3)
    want_results = copy.deepcopy(results)

    def np_model(full_ids):   # the oracle sees the same (bf16-rounded) logits as the GPU
        x = stub_logits(full_ids)
        return oracle.bf16_to_f32(oracle.bf16_round(x)).reshape(x.shape) if dtype == torch.bfloat16 else x
    oracle.process_ref_logprobs_batched(prompts, want_results, 3, T, reference_model=np_model, max_ref_batch_size=batch)
    calls = []
    svc = tome_amd.RefLogprobServicer(_torch_model(dev, dtype, calls), device=dev, max_ref_batch_size=batch)
    asyncio.run(svc._process_ref_logprobs_batched(prompts, results, 3, T))
    # chunks of max_ref_batch_size (node.py:419); a chunk holding only empty completions is not run
    flat = [bool(c.tokens) for r in results for c in r.completions]
    assert len(calls) == sum(any(flat[i:i + batch]) for i in range(0, len(flat), batch))
    n = 0
    for r, w in zip(results, want_results):
        for c, cw in zip(r.completions, w.completions):
            assert len(c.ref_log_probs) == len(c.tokens)               # tests/test_grpo.py:80
            assert all(isinstance(v, float) for v in c.ref_log_probs)
            np.testing.assert_allclose(c.ref_log_probs, cw.ref_log_probs, atol=1e-4, rtol=0)
            n += len(c.tokens)
    assert svc.last_ref_tokens == n


def test_entry_hidden_state_mode_scores_only_completion_rows(dev):
    """Hidden-state mode: the model returns final hidden states, lm_head is folded into the kernel."""
    rng = np.random.default_rng(0)
    H = 64
    emb = oracle.bf16_round((rng.standard_normal((V_STUB, H)) * 0.5).astype(np.float32))
    w_t = torch.from_numpy(emb.view(np.int16).copy()).view(torch.bfloat16).to(dev)

    def hidden_np(full_ids):   # a toy "model": hidden = embedding of the token, rotated by position
        e = oracle.bf16_to_f32(emb)[full_ids.astype(np.int64)]
        pos = np.arange(full_ids.shape[1])[None, :, None]
        return oracle.bf16_round((e * np.cos(0.1 * pos) + np.roll(e, 1, -1) * np.sin(0.1 * pos)).astype(np.float32))

    def model(full_ids, cache=None):
        hb = hidden_np(full_ids.cpu().numpy())
        return torch.from_numpy(hb.view(np.int16).copy()).view(torch.bfloat16).to(dev), None

    def np_model(full_ids):
        return oracle.lmhead_logits64(hidden_np(full_ids).reshape(-1, H), emb).reshape(*full_ids.shape, V_STUB).astype(np.float32)

    prompts, results = make_batch(seed=9, n_prompts=4, G=2)
    want = copy.deepcopy(results)
    oracle.process_ref_logprobs_batched(prompts, want, 2, 0.9, reference_model=np_model)
    svc = tome_amd.RefLogprobServicer(model, device=dev, lm_head_weight=w_t)
    svc.process_ref_logprobs_batched(prompts, results, 2, 0.9)
    for r, w in zip(results, want):
        for c, cw in zip(r.completions, w.completions):
            assert len(c.ref_log_probs) == len(c.tokens)
            np.testing.assert_allclose(c.ref_log_probs, cw.ref_log_probs, atol=2e-3, rtol=0)


def test_entry_prenorm_mode_applies_the_final_norm_to_completion_rows(dev):
    """Pre-norm mode: the model returns the states BEFORE the last RMSNorm (model.py:536); norm, lm_head and
    log-softmax all run on completion rows only."""
    rng = np.random.default_rng(3)
    H = 128
    emb = oracle.bf16_round((rng.standard_normal((V_STUB, H)) * 0.5).astype(np.float32))
    gamma = oracle.bf16_round((1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32))
    to_t = lambda bits: torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(dev)

    def prenorm_np(full_ids):  # toy decoder output with a position-dependent scale, so the norm matters
        e = oracle.bf16_to_f32(emb)[full_ids.astype(np.int64)]
        pos = np.arange(full_ids.shape[1])[None, :, None]
        return oracle.bf16_round((e * (1.0 + 0.5 * pos) + np.roll(e, 3, -1)).astype(np.float32))

    def model(full_ids, cache=None):
        return to_t(prenorm_np(full_ids.cpu().numpy())), None

    def np_model(full_ids):
        normed = oracle.rms_norm_bf16(prenorm_np(full_ids).reshape(-1, H), gamma, 1e-6)
        return oracle.lmhead_logits64(normed, emb).reshape(*full_ids.shape, V_STUB).astype(np.float32)

    prompts, results = make_batch(seed=5, n_prompts=3, G=2)
    want = copy.deepcopy(results)
    oracle.process_ref_logprobs_batched(prompts, want, 2, 1.1, reference_model=np_model)
    svc = tome_amd.RefLogprobServicer(model, device=dev, lm_head_weight=to_t(emb), final_norm_weight=to_t(gamma), norm_eps=1e-6)
    svc.process_ref_logprobs_batched(prompts, results, 2, 1.1)
    for r, w in zip(results, want):
        for c, cw in zip(r.completions, w.completions):
            assert len(c.ref_log_probs) == len(c.tokens)
            # a bf16 rounding of a normalised value may flip where the fp32 statistics differ in the last
            # place: 2e-3 of the fused path plus the effect of a few one-ulp flips
            np.testing.assert_allclose(c.ref_log_probs, cw.ref_log_probs, atol=4e-3, rtol=0)
    with pytest.raises(ValueError):
        tome_amd.RefLogprobServicer(model, device=dev, final_norm_weight=to_t(gamma))


# ---- golden vectors through the C ABI ------------------------------------------------------------------
@pytest.mark.parametrize("name", ["s0", "s1", "s2"])
def test_golden_small(dev, name):
    x, t, T = G[f"{name}_x"], G[f"{name}_t"], float(G[f"{name}_T"])
    r = tome_amd.token_logprobs(torch.from_numpy(x).to(dev), torch.from_numpy(t).to(dev), T, want_lse=True, want_entropy=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), G[f"{name}_lp"], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), G[f"{name}_lse"], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), G[f"{name}_ent"], atol=1e-4, rtol=0)


def _bits_to_torch(bits, dev):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(dev)


def test_golden_bf16_spike(dev):
    r = tome_amd.token_logprobs(_bits_to_torch(G["b0_bits"], dev), torch.from_numpy(G["b0_t"]).to(dev), 1.0,
                                want_entropy=True, want_argmax=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), G["b0_lp"], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), G["b0_ent"], atol=1e-4, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy(), G["b0_argmax"])


@pytest.mark.parametrize("name", ["c1", "c2", "c2t"])
def test_golden_full_vocab(dev, name):
    x, t, T, exp = seeded_case(G, name)
    xt = _bits_to_torch(x, dev) if x.dtype == np.uint16 else torch.from_numpy(x).to(dev)
    r = tome_amd.token_logprobs(xt, torch.from_numpy(t).to(dev), T, want_lse=True, want_entropy=True, want_argmax=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), exp["lp"], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), exp["lse"], atol=1e-4, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), exp["ent"], atol=1e-4, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy(), exp["argmax"])


def test_golden_lmhead(dev):
    h, w = _bits_to_torch(G["f0_h"], dev), _bits_to_torch(G["f0_w"], dev)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(G["f0_t"]).to(dev), float(G["f0_T"]), want_lse=True, want_entropy=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), G["f0_lp"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), G["f0_lse"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), G["f0_ent"], atol=2e-3, rtol=0)
