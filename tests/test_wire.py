"""Host-side container formats: packed variable-length chunks <-> Completion lists
(scheduler/proto/inference.proto:85-112, mlx-impl/node.py:409-458) and the JSON bodies of
knowledge/API.md:30-45."""
import copy
import json

import numpy as np
import pytest

import oracle
import tome_amd
from tome_amd import Completion, Prompt, PromptRollout
from test_host_logic import V_STUB, make_batch, stub_logits


@pytest.mark.parametrize("T,batch", [(1.0, 32), (0.7, 3), (0.0, 1)])
def test_packed_chunks_reproduce_the_entry_bookkeeping(T, batch):
    """pack -> score every valid position -> scatter must equal the oracle's restatement of node.py:391-461."""
    prompts, results = make_batch(seed=4, n_prompts=6, G=3)
    want = copy.deepcopy(results)
    n_want = oracle.process_ref_logprobs_batched(prompts, want, 3, T, reference_model=stub_logits, max_ref_batch_size=batch)
    n_got = 0
    for chunk in tome_amd.pack_ref_work(prompts, results, 3, batch):
        assert chunk.ids.dtype == np.int64 and chunk.ids.shape == chunk.targets.shape == chunk.valid.shape
        assert len(chunk.owners) == chunk.ids.shape[0] <= batch
        assert int(chunk.valid.sum()) == chunk.n_scored
        logits = stub_logits(chunk.ids.astype(np.uint32))
        m = chunk.valid.astype(bool)
        # the packed row list of the chunk names exactly the valid positions, in row-major order
        assert np.array_equal(chunk.scored_rows, np.flatnonzero(m.reshape(-1))) and chunk.scored_rows.dtype == np.int32
        assert np.array_equal(chunk.scored_targets, chunk.targets[m]) and len(chunk.scored_rows) == chunk.n_scored
        flat = oracle.local_compute_logprobs_f32(logits[m], chunk.targets[m].astype(np.uint32), T or 1.0)
        n_got += tome_amd.scatter_ref_logprobs(chunk, flat, results)
    assert n_got == n_want
    for r, w in zip(results, want):
        for c, cw in zip(r.completions, w.completions):
            assert len(c.ref_log_probs) == len(c.tokens)                  # tests/test_grpo.py:78-80
            np.testing.assert_allclose(c.ref_log_probs, cw.ref_log_probs, rtol=0, atol=1e-6)


def test_pack_alignment_padding_and_empty_completions():
    prompts = [Prompt("a", [5, 6, 7]), Prompt("b", [9])]
    results = [PromptRollout("a", [Completion([11, 12]), Completion([])]),
               PromptRollout("b", [Completion([21, 22, 23, 24]), Completion([31])])]
    (chunk,) = tome_amd.pack_ref_work(prompts, results, 2)
    assert chunk.ids.tolist() == [[5, 6, 7, 11], [5, 6, 7, 0], [9, 21, 22, 23], [9, 0, 0, 0]]   # p + c[:-1], pad id 0
    assert chunk.targets.tolist() == [[0, 0, 11, 12], [0, 0, 0, 0], [21, 22, 23, 24], [31, 0, 0, 0]]
    assert chunk.valid.tolist() == [[0, 0, 1, 1], [0, 0, 0, 0], [1, 1, 1, 1], [1, 0, 0, 0]]
    assert chunk.owners == [(0, 0), (0, 1), (1, 0), (1, 1)] and chunk.cu_lens.tolist() == [0, 2, 2, 6, 7]
    tome_amd.scatter_ref_logprobs(chunk, -np.arange(7, dtype=np.float32), results)
    assert results[0].completions[0].ref_log_probs == [0.0, -1.0] and results[0].completions[1].ref_log_probs == []
    assert results[1].completions[0].ref_log_probs == [-2.0, -3.0, -4.0, -5.0] and results[1].completions[1].ref_log_probs == [-6.0]
    with pytest.raises(ValueError):
        tome_amd.scatter_ref_logprobs(chunk, np.zeros(6, dtype=np.float32), results)
    with pytest.raises(ValueError):
        tome_amd.pack_ref_work([Prompt("e", [])], [PromptRollout("e", [Completion([1])])], 1)


def test_rollout_json_round_trip():
    results = [PromptRollout("p0", [Completion([1, 2, 3], [-0.1, -0.2, -0.3], [-0.15, -0.25, -0.35]), Completion([], [], [])]),
               PromptRollout("p1", [Completion([4294967295], [np.float32(-1.5)], [np.float32(-2.25)])])]
    body = tome_amd.rollout_response_to_json("batch-7", results)
    assert set(body) == {"batch_id", "results"} and set(body["results"][0]["completions"][0]) == {"tokens", "log_probs", "ref_log_probs"}
    batch_id, back = tome_amd.rollout_response_from_json(json.loads(json.dumps(body)))    # survives real serialisation
    assert batch_id == "batch-7" and [r.prompt_id for r in back] == ["p0", "p1"]
    for r, b in zip(results, back):
        for c, cb in zip(r.completions, b.completions):
            assert cb.tokens == [int(t) for t in c.tokens]
            assert cb.log_probs == [float(v) for v in c.log_probs] and cb.ref_log_probs == [float(v) for v in c.ref_log_probs]
    bad = {"batch_id": "x", "results": [{"prompt_id": "p", "completions": [{"tokens": [-1]}]}]}
    with pytest.raises(ValueError):
        tome_amd.rollout_response_from_json(bad)
