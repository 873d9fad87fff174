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

from typing import Callable, List, Optional, Sequence

import numpy as np
import torch

from .logprob import sample_tokens

UniformSource = Callable[[int, int], torch.Tensor]


def _uniforms(source, step: int, rows: int, dev: torch.device, generator) -> Optional[torch.Tensor]:
    if source is None:
        return torch.rand(rows, dtype=torch.float32, device=dev, generator=generator)
    u = source(step, rows)
    return torch.as_tensor(u, dtype=torch.float32, device=dev).reshape(rows)


def _step(logits: torch.Tensor, temperature: float, top_k: int, uniforms, active: Optional[Sequence[bool]]):
    """Sample every active row and fetch (token, lp) with one copy."""
    dev = logits.device
    rv = None if active is None else torch.tensor([1 if a else 0 for a in active], dtype=torch.int32, device=dev)
    out = sample_tokens(logits, temperature, top_k, uniforms=uniforms if temperature > 0 else None, row_valid=rv)
    host = torch.cat([out.token, out.lp.view(torch.int32)]).cpu().numpy()      # one sync, one copy
    n = out.token.numel()
    return host[:n].astype(np.int64), host[n:].view(np.float32)


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
    """
    dev = last_logits.device
    total = last_logits.shape[0] * G
    first = last_logits.repeat_interleave(G, dim=0)                            # same row, G independent draws
    tok, lp = _step(first, temperature, top_k, _uniforms(uniform_source, 0, total, dev, generator), None)
    results = [{"tokens": [int(tok[i])], "log_probs": [float(lp[i])]} for i in range(total)]    # node.py:574
    active_tokens = [int(t) for t in tok]
    finished = [False] * total                                                 # node.py:575: the first token is not checked
    for step in range(max_tokens - 1):                                         # node.py:578
        if all(finished):
            break
        logits = model_step(torch.tensor(active_tokens, dtype=torch.int64, device=dev))
        tok, lp = _step(logits, temperature, top_k, _uniforms(uniform_source, step + 1, total, dev, generator),
                        [not f for f in finished])
        new_active = []
        for b in range(total):
            if finished[b]:
                new_active.append(eos_token_id)                                # node.py:593-595
                continue
            token = int(tok[b])
            results[b]["tokens"].append(token)                                 # node.py:604-605
            results[b]["log_probs"].append(float(lp[b]))
            if token == eos_token_id or len(results[b]["tokens"]) >= max_tokens:
                finished[b] = True                                             # node.py:607-608
            new_active.append(token)
        active_tokens = new_active
    return results


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
    tok, lp = _step(first_logits, temperature, top_k, _uniforms(uniform_source, 0, B, dev, generator), None)
    results = [{"tokens": [int(tok[i])], "log_probs": [float(lp[i])]} for i in range(B)]
    active_tokens = [int(t) for t in tok]
    active = [True] * B                                                        # node.py:344
    for step in range(max_tokens - 1):                                         # node.py:346
        if not any(active):
            break
        inputs = [t if active[i] else 0 for i, t in enumerate(active_tokens)]  # node.py:350
        logits = model_step(torch.tensor(inputs, dtype=torch.int64, device=dev))
        tok, lp = _step(logits, temperature, top_k, _uniforms(uniform_source, step + 1, B, dev, generator), active)
        for i in range(B):
            if not active[i]:
                continue
            token = int(tok[i])
            active_tokens[i] = token
            if token == eos_token_id:
                active[i] = False                                              # node.py:369-370
            else:
                results[i]["tokens"].append(token)                             # node.py:371-373
                results[i]["log_probs"].append(float(lp[i]))
    return results
