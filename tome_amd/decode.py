"""The policy-side extraction sites of Tome's decode loops, on the batched sampler.

``Rollout`` (mlx-impl/node.py:556-612) and ``Judge`` (node.py:325-374) both run, per generated
token, a full ``fused_log_softmax`` over the batch followed by a Python loop that samples every row
(``_sample_token``, node.py:894-907) and reads its log-prob back with ``float(...)`` - 2·B host round
trips per step.  Here a step is one ``sample_tokens`` call for the whole batch (finished rows are
masked and not read) and ONE device-to-host copy of the tokens and log-probs; the bookkeeping
around it follows the reference line by line, including the two loops' different treatment of EOS.

The model itself (KV cache, attention) is not part of this path: ``model_step(tokens)`` stands for
``self.model(current_tokens, cache=batched_cache)[0][:, 0, :]`` plus ``cache.advance(1)``.
"""
from __future__ import annotations

from typing import Callable, List, Optional

import numpy as np
import torch

from .logprob import sample_tokens

UniformSource = Callable[[int, int], torch.Tensor]


def _uniforms(source, step: int, rows: int, dev: torch.device, generator) -> Optional[torch.Tensor]:
    if source is None:
        return torch.rand(rows, dtype=torch.float32, device=dev, generator=generator)
    u = source(step, rows)
    return torch.as_tensor(u, dtype=torch.float32, device=dev).reshape(rows)


def _step(logits: torch.Tensor, temperature: float, top_k: int, uniforms, row_valid: Optional[torch.Tensor],
          active: Optional[np.ndarray] = None):
    """Sample every active row; returns the device token ids and, after ONE copy, the host (token, lp) arrays.

    ``active`` is the host copy of ``row_valid`` (None = every row).  The sampler answers -1 for a row it was asked
    to draw from that holds no logit above -inf (a model that has diverged); such an id must not reach the next
    ``model_step`` as an embedding index, so it is an error here, naming the rows."""
    out = sample_tokens(logits, temperature, top_k, uniforms=uniforms if temperature > 0 else None, row_valid=row_valid)
    n = out.token.numel()
    tok, lp = out.token.reshape(-1), out.lp.reshape(-1)
    if lp.data_ptr() == tok.data_ptr() + 4 * n:        # the sampler's outputs sit back to back: no gather needed
        both = torch.as_strided(tok, (2 * n,), (1,))
    else:
        both = torch.cat([tok, lp.view(torch.int32)])
    host = both.cpu().numpy()                                                  # one sync, one copy
    tok_h = host[:n].astype(np.int64)
    bad = tok_h < 0 if active is None else (tok_h < 0) & active
    if bad.any():
        raise RuntimeError(f"decode step: no token could be drawn for rows {np.flatnonzero(bad).tolist()} "
                           "(no logit above -inf); the model's logits are degenerate")
    return out.token, tok_h, host[n:].view(np.float32)


def _mask_to_device(active: np.ndarray, dev: torch.device) -> torch.Tensor:
    return torch.from_numpy(active.astype(np.int32)).to(dev)


def _results(toks: np.ndarray, lps: np.ndarray, lens: np.ndarray) -> List[dict]:
    return [{"tokens": toks[i, :lens[i]].tolist(), "log_probs": [float(v) for v in lps[i, :lens[i]]]}
            for i in range(toks.shape[0])]


def rollout_decode(model_step: Callable[[torch.Tensor], torch.Tensor], last_logits: torch.Tensor, G: int,
                   temperature: float, max_tokens: int, eos_token_id: int, *, top_k: int = 20,
                   uniform_source: Optional[UniformSource] = None,
                   generator: Optional[torch.Generator] = None) -> List[dict]:
    """The sampling half of ``_rollout_batched`` (mlx-impl/node.py:556-612).

    ``last_logits`` [num_prompts, V]: the last prompt position's logits; every prompt gets ``G``
    independent first tokens from its row (node.py:556-571).  Then up to ``max_tokens - 1`` steps
    (node.py:578): ``model_step(tokens int64 [num_prompts * G]) -> logits [num_prompts * G, V]``; a
    finished sequence is fed ``eos_token_id`` (node.py:593-595) and is neither sampled nor read.
    A sequence finishes when it draws EOS - which is kept, with its log-prob (node.py:604-608) - or
    reaches ``max_tokens``.  Returns ``[{"tokens": [...], "log_probs": [...]}]`` in sequence order
    ``p_idx * G + g_idx`` (node.py:574).  ``uniform_source(step, rows)`` supplies the draws' uniforms
    (step 0 = first tokens); by default they come from ``torch.rand`` with ``generator``.

    Per generated token the host does one device-to-host copy (tokens and log-probs of the batch) and array
    bookkeeping; the next step's input ids are formed on the device from the sampled ids, and the row mask is
    uploaded only when a sequence finishes.
    """
    dev = last_logits.device
    total = last_logits.shape[0] * G
    first = last_logits.repeat_interleave(G, dim=0)                            # same row, G independent draws
    dev_tok, tok, lp = _step(first, temperature, top_k, _uniforms(uniform_source, 0, total, dev, generator), None)
    width = max(int(max_tokens), 1)
    toks = np.zeros((total, width), dtype=np.int64)
    lps = np.zeros((total, width), dtype=np.float32)
    lens = np.ones(total, dtype=np.int64)
    toks[:, 0], lps[:, 0] = tok, lp                                            # node.py:574
    finished = np.zeros(total, dtype=bool)                                     # node.py:575: the first token is not checked
    rv_dev = None                                                              # None = every row active
    eos_dev = torch.full((total,), int(eos_token_id), dtype=torch.int64, device=dev)
    for step in range(max_tokens - 1):                                         # node.py:578
        if finished.all():
            break
        inputs = dev_tok.to(torch.int64)
        if rv_dev is not None:
            inputs = torch.where(rv_dev != 0, inputs, eos_dev)                 # node.py:593-595
        logits = model_step(inputs)
        dev_tok, tok, lp = _step(logits, temperature, top_k, _uniforms(uniform_source, step + 1, total, dev, generator),
                                 rv_dev, ~finished)
        act = ~finished
        rows = np.nonzero(act)[0]
        toks[rows, lens[rows]] = tok[rows]                                     # node.py:604-605
        lps[rows, lens[rows]] = lp[rows]
        lens[rows] += 1
        newly = act & ((tok == eos_token_id) | (lens >= max_tokens))           # node.py:607-608
        if newly.any():
            finished |= newly
            rv_dev = _mask_to_device(~finished, dev)
    return _results(toks, lps, lens)


def judge_decode(model_step: Callable[[torch.Tensor], torch.Tensor], first_logits: torch.Tensor,
                 temperature: float, max_tokens: int, eos_token_id: int, *, top_k: int = 20,
                 uniform_source: Optional[UniformSource] = None,
                 generator: Optional[torch.Generator] = None) -> List[dict]:
    """The sampling half of a ``Judge`` chunk (mlx-impl/node.py:325-374).

    ``first_logits`` [B, V]; the first token of every item is always kept (node.py:334-342).
    In the loop (node.py:346-374) an item that draws EOS becomes inactive and the EOS token is NOT
    recorded (node.py:369-370) - unlike ``rollout_decode`` - and inactive items are fed token 0
    (node.py:350).  Returns ``[{"tokens": [...], "log_probs": [...]}]`` per item.
    """
    dev = first_logits.device
    B = first_logits.shape[0]
    dev_tok, tok, lp = _step(first_logits, temperature, top_k, _uniforms(uniform_source, 0, B, dev, generator), None)
    width = max(int(max_tokens), 1)
    toks = np.zeros((B, width), dtype=np.int64)
    lps = np.zeros((B, width), dtype=np.float32)
    lens = np.ones(B, dtype=np.int64)
    toks[:, 0], lps[:, 0] = tok, lp
    active = np.ones(B, dtype=bool)                                            # node.py:344
    rv_dev = None
    zero_dev = torch.zeros(B, dtype=torch.int64, device=dev)
    for step in range(max_tokens - 1):                                         # node.py:346
        if not active.any():
            break
        inputs = dev_tok.to(torch.int64)
        if rv_dev is not None:
            inputs = torch.where(rv_dev != 0, inputs, zero_dev)                # node.py:350
        logits = model_step(inputs)
        dev_tok, tok, lp = _step(logits, temperature, top_k, _uniforms(uniform_source, step + 1, B, dev, generator), rv_dev,
                                 active)
        ended = active & (tok == eos_token_id)                                 # node.py:369-370: EOS is not recorded
        rows = np.nonzero(active & ~ended)[0]
        toks[rows, lens[rows]] = tok[rows]                                     # node.py:371-373
        lps[rows, lens[rows]] = lp[rows]
        lens[rows] += 1
        if ended.any():
            active &= ~ended
            rv_dev = _mask_to_device(active, dev)
    return _results(toks, lps, lens)
