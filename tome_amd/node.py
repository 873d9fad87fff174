"""The reference-logprob entry of Tome's inference node, on the HIP kernels.

Mirrors ``InferenceNodeServicer._process_ref_logprobs_batched``
(mlx-impl/node.py:391-461): same name, arguments, in-place mutation of
``results[p].completions[g].ref_log_probs`` and chunking by ``max_ref_batch_size``.
The gRPC messages it walks (scheduler/proto/inference.proto:85-112) are mirrored
as plain dataclasses; anything with the same attributes (``.tokens``,
``.completions``, ``.ref_log_probs``) works, including the protobuf classes.
"""
from __future__ import annotations

import logging
import time
from dataclasses import dataclass, field
from typing import Any, Callable, List, Optional, Sequence

import numpy as np
import torch

from .wire import pack_ref_work, scatter_ref_logprobs
from .logprob import fused_lmhead_logprobs, token_logprobs_rows

logger = logging.getLogger(__name__)


@dataclass
class Prompt:
    """inference.proto:85-88"""
    prompt_id: str = ""
    tokens: List[int] = field(default_factory=list)


@dataclass
class Completion:
    """inference.proto:108-112: one float per completion token in both lists."""
    tokens: List[int] = field(default_factory=list)
    log_probs: List[float] = field(default_factory=list)
    ref_log_probs: List[float] = field(default_factory=list)


@dataclass
class PromptRollout:
    """inference.proto:103-106"""
    prompt_id: str = ""
    completions: List[Completion] = field(default_factory=list)


class RefLogprobServicer:
    """The slice of InferenceNodeServicer (mlx-impl/node.py:49-100) that the ref-logprob path uses.

    ``reference_model(full_ids, cache=None)`` follows Qwen3.__call__ (mlx-impl/model.py:522-540):
    it takes int64 token ids [B, L] on ``device`` and returns ``(logits [B, L, V], cache)``.

    If ``lm_head_weight`` ([V, H] bf16) is given, ``reference_model`` must instead return the
    final, normalised hidden states ``(hidden [B, L, H] bf16, cache)``; only the completion rows
    are then pushed through the fused lm_head + log-softmax kernel, so logits for prompt and
    padding rows (which the reference computes at node.py:443 and discards at :449) are never
    formed.  With ``final_norm_weight`` ([H] bf16) as well, ``reference_model`` returns the states
    BEFORE the last RMSNorm (model.py:536) and that norm, too, is applied to completion rows only.
    """

    def __init__(self, reference_model: Callable[..., Any], device: torch.device | str = "cuda:0",
                 max_ref_batch_size: int = 32, lm_head_weight: Optional[torch.Tensor] = None,
                 final_norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 1e-6):
        if final_norm_weight is not None and lm_head_weight is None:
            raise ValueError("final_norm_weight needs lm_head_weight (hidden-state mode)")
        self.reference_model = reference_model
        self.device = torch.device(device)
        self.max_ref_batch_size = max_ref_batch_size     # node.py:58
        self.lm_head_weight = lm_head_weight
        self.final_norm_weight = final_norm_weight
        self.norm_eps = norm_eps                          # RMSNorm default, model.py:337
        self.last_ref_tokens = 0
        self.last_ref_seconds = 0.0

    async def _process_ref_logprobs_batched(self, prompts: Sequence, results: Sequence, G: int,
                                            temperature: float = 1.0) -> None:
        """Compute reference-model log-probs of every completion token, batched, without KV cache."""
        self.process_ref_logprobs_batched(prompts, results, G, temperature)

    def process_ref_logprobs_batched(self, prompts: Sequence, results: Sequence, G: int,
                                     temperature: float = 1.0) -> None:
        """Synchronous body of ``_process_ref_logprobs_batched`` (the reference's coroutine has no awaits)."""
        t0 = time.perf_counter()
        num_toks = 0
        temp = temperature or 1.0                                         # node.py:451
        # work list, chunks of max_ref_batch_size, right-padding with id 0: node.py:409-441
        for chunk in pack_ref_work(prompts, results, G, self.max_ref_batch_size):
            if chunk.n_scored == 0:                                      # only empty completions (node.py:428-432)
                continue
            full_ids = torch.from_numpy(chunk.ids).to(self.device)
            out, _ = self.reference_model(full_ids, cache=None)           # node.py:443
            # The scored positions - rows p_len-1 .. p_len-2+len(c) of each sequence (node.py:449) - packed in
            # row-major order; one sync + one copy per chunk (node.py:456), of those positions only.
            if self.lm_head_weight is None:
                rows = torch.from_numpy(chunk.scored_rows).to(self.device)
                tg = torch.from_numpy(chunk.scored_targets).to(self.device)
                flat = token_logprobs_rows(out, rows, tg, temp).lp.cpu().numpy()   # only the listed rows are launched
            else:
                tg = torch.from_numpy(chunk.targets).to(self.device)
                rv = torch.from_numpy(chunk.valid).to(self.device)
                lps = fused_lmhead_logprobs(out, self.lm_head_weight, tg, temp, row_valid=rv,
                                            norm_weight=self.final_norm_weight, norm_eps=self.norm_eps).lp
                flat = lps[rv.bool()].cpu().numpy()
            num_toks += scatter_ref_logprobs(chunk, flat, results)        # node.py:457-458

        elapsed = time.perf_counter() - t0
        self.last_ref_tokens, self.last_ref_seconds = num_toks, elapsed
        logger.info("Ref log-probs non-KV batched completed: %d tokens in %.2fs (%.1f tok/s)",
                    num_toks, elapsed, num_toks / elapsed if elapsed > 0 else 0.0)
