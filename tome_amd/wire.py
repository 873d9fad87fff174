"""Container formats either side of the ref-log-prob path.

* The gRPC messages of scheduler/proto/inference.proto:85-112 (``Prompt``, ``PromptRollout``,
  ``Completion``) carry one Python list per completion; the kernels want flat arrays.
  ``pack_ref_work`` / ``scatter_ref_logprobs`` convert between the two with a packed variable-length
  layout: all scored positions of a chunk concatenated, ``cu_lens`` giving each completion's slice.
* The JSON bodies of ``POST /v1/grpo/rollout`` (knowledge/API.md:30-45) mirror the same messages;
  ``rollout_response_to_json`` / ``rollout_response_from_json`` convert them.

Nothing here touches the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Sequence, Tuple

import numpy as np


@dataclass
class PackedRefChunk:
    """One chunk of ``_process_ref_logprobs_batched`` work (mlx-impl/node.py:419-449) as arrays.

    ``ids`` [B, max_len] int64 right-padded with 0 (node.py:440), ``targets`` / ``valid`` [B, max_len]
    int32: row ``p_len - 1 + k`` of sequence ``i`` scores completion token ``k`` (node.py:434-437, :449).
    ``owners[j] = (p_idx, g)`` and ``cu_lens[j] : cu_lens[j + 1]`` locate completion ``j``'s log-probs in the
    flat array of valid positions taken in row-major order; empty completions own an empty slice.
    """
    ids: np.ndarray
    targets: np.ndarray
    valid: np.ndarray
    owners: List[Tuple[int, int]]
    cu_lens: np.ndarray

    @property
    def n_scored(self) -> int:
        return int(self.cu_lens[-1])

    @property
    def scored_rows(self) -> np.ndarray:
        """Rows of the flattened [B * max_len] batch that are scored, ascending (int32): the packed row list."""
        return np.flatnonzero(self.valid.reshape(-1)).astype(np.int32)

    @property
    def scored_targets(self) -> np.ndarray:
        """The targets of ``scored_rows``, in the same order (int32 [n_scored])."""
        return self.targets.reshape(-1)[self.scored_rows]


def pack_ref_work(prompts: Sequence, results: Sequence, G: int, max_ref_batch_size: int = 32) -> List[PackedRefChunk]:
    """The work list and chunking of mlx-impl/node.py:409-441 as packed arrays, one entry per chunk."""
    work = []
    for p_idx, p in enumerate(prompts):                                   # node.py:409-414
        p_toks = list(p.tokens)
        for g in range(G):
            work.append((p_idx, g, p_toks, list(results[p_idx].completions[g].tokens)))
    chunks = []
    for c0 in range(0, len(work), max_ref_batch_size):                    # node.py:419-421
        chunk = work[c0:c0 + max_ref_batch_size]
        seqs = [p + c[:-1] if c else p for _, _, p, c in chunk]           # node.py:427-437
        max_len = max(len(s) for s in seqs)
        ids = np.zeros((len(chunk), max_len), dtype=np.int64)
        targets = np.zeros((len(chunk), max_len), dtype=np.int32)
        valid = np.zeros((len(chunk), max_len), dtype=np.int32)
        lens = []
        for i, (s, (_, _, p_toks, c_toks)) in enumerate(zip(seqs, chunk)):
            ids[i, :len(s)] = s
            if c_toks:
                lo = len(p_toks) - 1
                if lo < 0:
                    raise ValueError("a prompt needs at least one token to score its completion")
                targets[i, lo:lo + len(c_toks)] = c_toks
                valid[i, lo:lo + len(c_toks)] = 1
            lens.append(len(c_toks))
        cu = np.zeros(len(chunk) + 1, dtype=np.int64)
        np.cumsum(lens, out=cu[1:])
        chunks.append(PackedRefChunk(ids, targets, valid, [(w[0], w[1]) for w in chunk], cu))
    return chunks


def scatter_ref_logprobs(chunk: PackedRefChunk, flat_lp: np.ndarray, results: Sequence) -> int:
    """Append each completion's slice of ``flat_lp`` (float32 [n_scored], valid positions in row-major
    order) to ``results[p_idx].completions[g].ref_log_probs`` (node.py:457-458).  Returns tokens written."""
    flat_lp = np.asarray(flat_lp)
    if flat_lp.shape != (chunk.n_scored,):
        raise ValueError(f"expected {chunk.n_scored} log-probs, got {flat_lp.shape}")
    for j, (p_idx, g) in enumerate(chunk.owners):
        lo, hi = int(chunk.cu_lens[j]), int(chunk.cu_lens[j + 1])
        if hi > lo:
            results[p_idx].completions[g].ref_log_probs.extend(flat_lp[lo:hi].tolist())
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
