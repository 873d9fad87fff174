"""Container formats either side of the ref-log-prob path.

* The gRPC messages of scheduler/proto/inference.proto:85-112 (``Prompt``, ``PromptRollout``,
  ``Completion``) carry one Python list per completion; the kernels want flat arrays.
  ``iter_ref_work`` / ``pack_ref_work`` / ``scatter_ref_logprobs`` convert between the two with a packed
  variable-length layout: all scored positions of a chunk concatenated, ``cu_lens`` giving each completion's slice.
* The JSON bodies of ``POST /v1/grpo/rollout`` (knowledge/API.md:30-45) mirror the same messages;
  ``rollout_response_to_json`` / ``rollout_response_from_json`` convert them.

Nothing here touches the GPU.
"""
from __future__ import annotations

from array import array
from dataclasses import dataclass, field
from typing import Any, Iterator, List, Sequence, Tuple

import numpy as np


@dataclass
class PackedRefChunk:
    """One chunk of ``_process_ref_logprobs_batched`` work (mlx-impl/node.py:419-449) as arrays.

    ``ids`` [B, max_len] int64 right-padded with 0 (node.py:440).  Row ``p_len - 1 + k`` of sequence ``i`` scores
    completion token ``k`` (node.py:434-437, :449): ``scored_rows`` (int32, ascending) names those rows of the
    flattened [B * max_len] batch and ``scored_targets`` (int32) their token ids - the packed row list the row
    kernel takes.  ``targets`` / ``valid`` [B, max_len] int32 are the same as dense arrays (built on first use).
    ``owners[j] = (p_idx, g)`` and ``cu_lens[j] : cu_lens[j + 1]`` locate completion ``j``'s log-probs in the
    flat array of scored positions; empty completions own an empty slice.
    """
    ids: np.ndarray
    scored_rows: np.ndarray
    scored_targets: np.ndarray
    owners: List[Tuple[int, int]]
    cu_lens: np.ndarray
    _dense: Any = field(default=None, repr=False, compare=False)

    @property
    def n_scored(self) -> int:
        return int(self.cu_lens[-1])

    def _dense_arrays(self):
        if self._dense is None:
            targets = np.zeros(self.ids.size, dtype=np.int32)
            valid = np.zeros(self.ids.size, dtype=np.int32)
            targets[self.scored_rows] = self.scored_targets
            valid[self.scored_rows] = 1
            self._dense = (targets.reshape(self.ids.shape), valid.reshape(self.ids.shape))
        return self._dense

    @property
    def targets(self) -> np.ndarray:
        return self._dense_arrays()[0]

    @property
    def valid(self) -> np.ndarray:
        return self._dense_arrays()[1]


def _token_array(tokens, what: str) -> np.ndarray:
    """A token list (Python list or protobuf repeated field) as int64.  array.array converts at about two thirds of
    the cost of numpy's own list conversion and refuses anything that is not an integer."""
    try:
        return np.frombuffer(array("q", tokens), dtype=np.int64)
    except (TypeError, OverflowError) as e:
        raise ValueError(f"{what} must be a flat list of integer token ids") from e


def iter_ref_work(prompts: Sequence, results: Sequence, G: int, max_ref_batch_size: int = 32) -> Iterator[PackedRefChunk]:
    """The work list and chunking of mlx-impl/node.py:409-441, one packed chunk at a time (so that a caller can
    launch chunk i before chunk i + 1 is packed).  Each token list is converted to an array once - the prompt's
    once for all its G rows; the scored rows, their targets and the slices are array arithmetic over the chunk."""
    p_arrs = [_token_array(p.tokens, "prompt tokens") for p in prompts]   # node.py:409-414
    work = [(p_idx, g) for p_idx in range(len(prompts)) for g in range(G)]
    for c0 in range(0, len(work), max_ref_batch_size):                    # node.py:419-421
        chunk = work[c0:c0 + max_ref_batch_size]
        nb = len(chunk)
        c_arrs = [_token_array(results[p].completions[g].tokens, "completion tokens") for p, g in chunk]
        p_lens = np.array([p_arrs[p].size for p, _ in chunk], dtype=np.int64)
        c_lens = np.array([c.size for c in c_arrs], dtype=np.int64)
        if ((p_lens == 0) & (c_lens > 0)).any():
            raise ValueError("a prompt needs at least one token to score its completion")
        seq_lens = p_lens + np.maximum(c_lens - 1, 0)                     # p + c[:-1]; just p for an empty completion (node.py:427-437)
        max_len = int(seq_lens.max())
        ids = np.zeros((nb, max_len), dtype=np.int64)                     # right-padding with id 0: node.py:440
        for i, ((p, _), c) in enumerate(zip(chunk, c_arrs)):
            pl = p_arrs[p].size
            ids[i, :pl] = p_arrs[p]
            if c.size > 1:
                ids[i, pl:pl + c.size - 1] = c[:-1]
        # scored positions: rows p_len - 1 .. p_len - 2 + len(c) of each sequence, targets c (node.py:434-437, :449)
        cu = np.zeros(nb + 1, dtype=np.int64)
        np.cumsum(c_lens, out=cu[1:])
        first = np.arange(nb, dtype=np.int64) * max_len + p_lens - 1 - cu[:-1]   # row of target k of sequence i = first[i] + cu[i] + k
        scored_rows = (np.repeat(first, c_lens) + np.arange(int(cu[-1]), dtype=np.int64)).astype(np.int32)
        scored_targets = (np.concatenate(c_arrs) if nb else np.zeros(0, np.int64)).astype(np.int32)
        yield PackedRefChunk(ids, scored_rows, scored_targets, chunk, cu)


def pack_ref_work(prompts: Sequence, results: Sequence, G: int, max_ref_batch_size: int = 32) -> List[PackedRefChunk]:
    """``iter_ref_work`` as a list, one entry per chunk."""
    return list(iter_ref_work(prompts, results, G, max_ref_batch_size))


def scatter_ref_logprobs(chunk: PackedRefChunk, flat_lp: np.ndarray, results: Sequence) -> int:
    """Append each completion's slice of ``flat_lp`` (float32 [n_scored], scored positions in row-major
    order) to ``results[p_idx].completions[g].ref_log_probs`` (node.py:457-458).  Returns tokens written.
    One ``tolist`` per chunk; the slices are taken from the Python list."""
    flat_lp = np.asarray(flat_lp)
    if flat_lp.shape != (chunk.n_scored,):
        raise ValueError(f"expected {chunk.n_scored} log-probs, got {flat_lp.shape}")
    values = flat_lp.tolist()
    bounds = chunk.cu_lens.tolist()
    for j, (p_idx, g) in enumerate(chunk.owners):
        lo, hi = bounds[j], bounds[j + 1]
        if hi > lo:
            results[p_idx].completions[g].ref_log_probs.extend(values[lo:hi])
    return chunk.n_scored


def rollout_response_to_json(batch_id: str, results: Sequence) -> dict:
    """RolloutResponse (inference.proto:98-101) as the JSON body of knowledge/API.md:30-45."""
    return {
        "batch_id": batch_id,
        "results": [
            {"prompt_id": r.prompt_id,
             "completions": [{"tokens": [int(t) for t in c.tokens],
                              "log_probs": [float(v) for v in c.log_probs],
                              "ref_log_probs": [float(v) for v in c.ref_log_probs]} for c in r.completions]}
            for r in results],
    }


def rollout_response_from_json(obj: dict) -> Tuple[str, List[Any]]:
    """Inverse of ``rollout_response_to_json``: ``(batch_id, [PromptRollout])``."""
    from .node import Completion, PromptRollout
    out = []
    for r in obj["results"]:
        comps = []
        for c in r["completions"]:
            toks = [int(t) for t in c["tokens"]]
            if any(t < 0 or t > 0xFFFFFFFF for t in toks):
                raise ValueError("token ids are uint32 on the wire (inference.proto:109)")
            comps.append(Completion(tokens=toks, log_probs=[float(v) for v in c.get("log_probs", [])],
                                    ref_log_probs=[float(v) for v in c.get("ref_log_probs", [])]))
        out.append(PromptRollout(prompt_id=str(r["prompt_id"]), completions=comps))
    return str(obj["batch_id"]), out
