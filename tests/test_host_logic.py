"""Host-side logic that needs no GPU: input plumbing of the Python mirror, the no-fallback rule,
and the entry-point bookkeeping (restated in the oracle, node.py:391-461) on a stub model."""
import asyncio
import inspect

import numpy as np
import pytest
import torch

import oracle
import tome_amd
from tome_amd import logprob as lp_mod
from tome_amd.node import Completion, Prompt, PromptRollout


def test_cpu_tensors_raise_instead_of_falling_back():
    x = torch.zeros(2, 8)
    t = torch.zeros(2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tome_amd.token_logprobs(x, t)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tome_amd.fused_log_softmax(x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tome_amd.local_compute_logprobs(x, t, 1.0)
    h = torch.zeros(2, 8, dtype=torch.bfloat16)
    w = torch.zeros(16, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tome_amd.fused_lmhead_logprobs(h, w, t)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tome_amd.grpo_dual_logprobs(h, w, w, t)


def test_product_does_not_import_the_oracle():
    import os
    pkg = os.path.dirname(tome_amd.__file__)
    for name in os.listdir(pkg):
        if name.endswith(".py"):
            src = open(os.path.join(pkg, name)).read()
            assert "oracle" not in src, f"{name} mentions the oracle"
    for name in os.listdir(os.path.join(pkg, "csrc")):
        assert "oracle" not in open(os.path.join(pkg, "csrc", name)).read()


def test_signatures_mirror_the_reference():
    # model.py:77  fused_log_softmax(logits, temperature=1.0)
    p = inspect.signature(tome_amd.fused_log_softmax).parameters
    assert list(p) == ["logits", "temperature"] and p["temperature"].default == 1.0
    # node.py:400  local_compute_logprobs(logits, ids, temp)
    assert list(inspect.signature(tome_amd.local_compute_logprobs).parameters) == ["logits", "ids", "temp"]
    # node.py:391-397  _process_ref_logprobs_batched(self, prompts, results, G, temperature=1.0) -> None, async
    m = tome_amd.RefLogprobServicer._process_ref_logprobs_batched
    assert inspect.iscoroutinefunction(m)
    p = inspect.signature(m).parameters
    assert list(p) == ["self", "prompts", "results", "G", "temperature"] and p["temperature"].default == 1.0
    # node.py:58  max_ref_batch_size=32
    assert inspect.signature(tome_amd.RefLogprobServicer.__init__).parameters["max_ref_batch_size"].default == 32
    # node.py:102-106  async UpdateWeights(self, request, context) -> WeightUpdateResponse(success, policy_version)
    m = tome_amd.WeightUpdateServicer.UpdateWeights
    assert inspect.iscoroutinefunction(m) and list(inspect.signature(m).parameters)[:3] == ["self", "request", "context"]
    # inference.proto:68-81  LayerUpdate / WeightUpdateResponse field names
    import dataclasses
    assert [f.name for f in dataclasses.fields(tome_amd.LayerUpdate)] == [
        "layer_idx", "param_name", "lora_A", "lora_B", "shape_A", "shape_B", "lora_scale"]
    assert [f.name for f in dataclasses.fields(tome_amd.WeightUpdateResponse)] == ["success", "policy_version"]
    # node.py:894  _sample_token's top_k = 20
    assert inspect.signature(tome_amd.sample_tokens).parameters["top_k"].default == 20


def test_temperature_validation():
    for bad in (0, 0.0, -1.0, float("nan"), float("inf")):
        with pytest.raises(ValueError):
            lp_mod._check_temperature(bad)
    assert lp_mod._check_temperature(0.7) == 0.7


def test_rows_view_avoids_copies():
    x = torch.zeros(4, 9, 32)
    v = lp_mod._rows_view(x)
    assert v.shape == (36, 32) and v.data_ptr() == x.data_ptr()
    sl = x[2, 3:8]
    v = lp_mod._rows_view(sl)
    assert v.data_ptr() == sl.data_ptr() and v.stride(0) == 32
    assert lp_mod._rows_view(torch.zeros(32)).shape == (1, 32)
    tr = torch.zeros(32, 6).t()            # V axis strided: copied, like ensure_row_contiguous (model.py:73)
    assert lp_mod._rows_view(tr).stride(-1) == 1


def test_row_valid_from_lengths():
    rv = lp_mod._row_valid((3, 5), 15, torch.tensor([5, 0, 2]), None, torch.device("cpu"))
    assert rv.tolist() == [1, 1, 1, 1, 1, 0, 0, 0, 0, 0, 1, 1, 0, 0, 0]
    with pytest.raises(ValueError):
        lp_mod._row_valid((15,), 15, torch.tensor([5]), None, torch.device("cpu"))
    with pytest.raises(ValueError):
        lp_mod._row_valid((3, 5), 15, torch.tensor([5, 0, 2]), torch.ones(15), torch.device("cpu"))


# ---- entry-point bookkeeping, oracle side (known answers from a stub model) --------------------------
V_STUB = 50


def stub_logits(full_ids: np.ndarray) -> np.ndarray:
    """logits[b, pos, v] depends only on (token at pos, pos, v): alignment mistakes change the answer."""
    B, L = full_ids.shape
    v = np.arange(V_STUB, dtype=np.float64)[None, None, :]
    tok = full_ids.astype(np.float64)[:, :, None]
    pos = np.arange(L, dtype=np.float64)[None, :, None]
    return (np.sin(0.37 * tok + 0.11 * v * (1 + pos % 3)) * 3.0).astype(np.float32)


def expected_ref_lps(p_toks, c_toks, T):
    """Direct statement of node.py:434-437,449: row p_len-1+k of the model run on p + c[:-1] scores c[k]."""
    if not c_toks:
        return []
    seq = np.array([p_toks + c_toks[:-1]], dtype=np.uint32)
    logits = stub_logits(seq)[0]
    out = []
    for k, c in enumerate(c_toks):
        out.append(float(oracle.logprob_rows(logits[len(p_toks) - 1 + k][None], [c], T)[0]))
    return out


def make_batch(seed=0, n_prompts=5, G=3):
    rng = np.random.default_rng(seed)
    prompts, results = [], []
    for p in range(n_prompts):
        prompts.append(Prompt(f"p{p}", rng.integers(1, V_STUB, size=rng.integers(1, 9)).tolist()))
        comps = []
        for g in range(G):
            n = 0 if (p == 1 and g == 1) else int(rng.integers(1, 12))     # one empty completion
            comps.append(Completion(tokens=rng.integers(1, V_STUB, size=n).tolist()))
        results.append(PromptRollout(f"p{p}", comps))
    return prompts, results


@pytest.mark.parametrize("T,batch", [(1.0, 32), (0.7, 4), (0.0, 1)])
def test_oracle_entry_known_answers(T, batch):
    prompts, results = make_batch()
    n = oracle.process_ref_logprobs_batched(prompts, results, 3, T, reference_model=stub_logits,
                                            max_ref_batch_size=batch)
    total = 0
    for p, r in zip(prompts, results):
        for c in r.completions:
            assert len(c.ref_log_probs) == len(c.tokens)               # tests/test_grpo.py:80
            want = expected_ref_lps(list(p.tokens), list(c.tokens), T or 1.0)   # temperature 0 -> 1.0, node.py:451
            np.testing.assert_allclose(c.ref_log_probs, want, atol=2e-5)
            total += len(c.tokens)
    assert n == total
    assert results[1].completions[1].ref_log_probs == []               # empty completion: nothing appended


def test_oracle_entry_pads_with_zero_and_extends():
    prompts = [Prompt("a", [3, 4, 5]), Prompt("b", [7])]
    results = [PromptRollout("a", [Completion(tokens=[9, 8])]), PromptRollout("b", [Completion(tokens=[1, 2, 3, 4, 5, 6])])]
    results[0].completions[0].ref_log_probs.append(-1.0)             # extend, not replace (node.py:458)
    seen = []

    def model(full_ids):
        seen.append(full_ids.copy())
        return stub_logits(full_ids)
    oracle.process_ref_logprobs_batched(prompts, results, 1, 1.0, reference_model=model)
    assert len(seen) == 1 and seen[0].dtype == np.uint32
    assert seen[0].tolist() == [[3, 4, 5, 9, 0, 0], [7, 1, 2, 3, 4, 5]]   # p + c[:-1], right-padded with 0
    assert results[0].completions[0].ref_log_probs[0] == -1.0 and len(results[0].completions[0].ref_log_probs) == 3


def test_servicer_is_async_like_the_reference():
    s = tome_amd.RefLogprobServicer(lambda ids, cache=None: (None, None), device="cpu")
    # nothing to score: must finish without calling the model or the GPU
    asyncio.run(s._process_ref_logprobs_batched([Prompt("p", [1])], [PromptRollout("p", [Completion()])], 1))
    assert s.last_ref_tokens == 0


@pytest.mark.parametrize("loop", ["rollout", "judge"])
def test_decode_loops_refuse_a_row_without_a_token(monkeypatch, loop):
    """The sampler answers -1 for an active row with no logit above -inf.  The decode loops must not feed that id
    to the next model step (an out-of-range embedding index on the device); they raise, naming the row.  The
    sampler is stubbed here (greedy over CPU tensors) so that the bookkeeping runs without a GPU."""
    from tome_amd import decode as dec
    from tome_amd.logprob import SampledTokens

    def stub_sampler(logits, temperature, top_k, *, uniforms=None, row_valid=None):
        best, tok = logits.max(dim=-1)
        tok = torch.where(torch.isneginf(best), torch.full_like(tok, -1), tok).to(torch.int32)
        if row_valid is not None:
            tok = torch.where(row_valid != 0, tok, torch.full_like(tok, -1))
        lp = torch.zeros(tok.shape, dtype=torch.float32)
        return SampledTokens(tok, lp, tok, None, None)

    monkeypatch.setattr(dec, "sample_tokens", stub_sampler)
    V, B = 16, 3
    first = torch.zeros(B, V)
    first[:, 4] = 1.0
    seen = []

    def model_step(tokens):
        seen.append(tokens.tolist())
        out = torch.zeros(B, V)
        out[:, 5] = 1.0
        if len(seen) == 2:
            out[1] = float("-inf")                  # row 1 diverges at the second step
        return out

    run = (lambda: dec.rollout_decode(model_step, first, 1, 0.0, 6, 9)) if loop == "rollout" else \
          (lambda: dec.judge_decode(model_step, first, 0.0, 6, 9))
    with pytest.raises(RuntimeError, match=r"rows \[1\]"):
        run()
    assert all(t >= 0 for step in seen for t in step)   # no negative id ever reached the model
    # a masked (finished) row's -1 is not an error: eos = 5 ends every row at the first loop step
    seen.clear()
    done = dec.rollout_decode(lambda t: model_step(t), first, 1, 0.0, 6, 5) if loop == "rollout" else \
        dec.judge_decode(lambda t: model_step(t), first, 0.0, 6, 5)
    assert [d["tokens"] for d in done] == ([[4, 5]] * B if loop == "rollout" else [[4]] * B)
