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

from .wire import PackedRefChunk, iter_ref_work, scatter_ref_logprobs
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
        self._slots = None                                # created on first use (needs the GPU)

    async def _process_ref_logprobs_batched(self, prompts: Sequence, results: Sequence, G: int,
                                            temperature: float = 1.0) -> None:
        """Compute reference-model log-probs of every completion token, batched, without KV cache."""
        self.process_ref_logprobs_batched(prompts, results, G, temperature)

    # ---- staging: one pinned host buffer and one device buffer per pipeline slot, grown on demand ----------
    def _slot(self, i: int, in_bytes: int, out_floats: int) -> "_Slot":
        if self._slots is None:
            self._slots = [_Slot(), _Slot()]
        slot = self._slots[i]
        if slot.host_in is None or slot.host_in.numel() < in_bytes:
            cap = max(in_bytes, 1 << 16) * 3 // 2
            slot.host_in = torch.empty(cap, dtype=torch.uint8, pin_memory=True)
            slot.dev_in = torch.empty(cap, dtype=torch.uint8, device=self.device)
        if slot.host_out is None or slot.host_out.numel() < out_floats:
            slot.host_out = torch.empty(max(out_floats, 1 << 12) * 3 // 2, dtype=torch.float32, pin_memory=True)
        return slot

    def _launch(self, chunk: PackedRefChunk, slot_index: int, temp: float) -> "_Slot":
        """Everything one chunk puts on the stream: ONE upload (ids, scored rows, targets), the model's forward,
        the log-prob kernel over the scored rows only, and the download of the packed result.  Nothing here waits
        for the GPU."""
        nb, max_len = chunk.ids.shape
        n = chunk.n_scored
        id_bytes, n_bytes = nb * max_len * 8, n * 4
        slot = self._slot(slot_index, id_bytes + 2 * n_bytes, n)
        host = slot.host_in.numpy()
        host[:id_bytes].view(np.int64)[:] = chunk.ids.reshape(-1)
        host[id_bytes:id_bytes + n_bytes].view(np.int32)[:] = chunk.scored_rows
        host[id_bytes + n_bytes:id_bytes + 2 * n_bytes].view(np.int32)[:] = chunk.scored_targets
        total = id_bytes + 2 * n_bytes
        slot.dev_in[:total].copy_(slot.host_in[:total], non_blocking=True)
        full_ids = slot.dev_in[:id_bytes].view(torch.int64).view(nb, max_len)
        rows = slot.dev_in[id_bytes:id_bytes + n_bytes].view(torch.int32)
        tg = slot.dev_in[id_bytes + n_bytes:total].view(torch.int32)
        out, _ = self.reference_model(full_ids, cache=None)               # node.py:443
        # The scored positions - rows p_len-1 .. p_len-2+len(c) of each sequence (node.py:449) - in row-major order.
        if self.lm_head_weight is None:
            lps = token_logprobs_rows(out, rows, tg, temp).lp             # only the listed rows are launched
        else:
            picked = out.reshape(nb * max_len, out.shape[-1]).index_select(0, rows.long())   # completion rows only
            lps = fused_lmhead_logprobs(picked, self.lm_head_weight, tg, temp,
                                        norm_weight=self.final_norm_weight, norm_eps=self.norm_eps).lp
        slot.host_out[:n].copy_(lps, non_blocking=True)                   # node.py:456: the one copy back, of n floats
        slot.done.record(torch.cuda.current_stream(self.device))
        slot.chunk, slot.keep = chunk, (out, lps)                         # outputs stay alive until they have been read
        return slot

    def _finish(self, slot: "_Slot", results: Sequence) -> int:
        slot.done.synchronize()
        n = slot.chunk.n_scored
        written = scatter_ref_logprobs(slot.chunk, slot.host_out.numpy()[:n], results)   # node.py:457-458
        slot.chunk = slot.keep = None
        return written

    def process_ref_logprobs_batched(self, prompts: Sequence, results: Sequence, G: int,
                                     temperature: float = 1.0) -> None:
        """Synchronous body of ``_process_ref_logprobs_batched`` (the reference's coroutine has no awaits).

        Chunks run one deep in a pipeline: chunk i + 1 is packed on the host and put on the stream before the
        result of chunk i is waited for, so host bookkeeping and GPU work overlap.  Results are appended in chunk
        order, as the reference does.  (Two chunks' model outputs are alive at a time.)"""
        t0 = time.perf_counter()
        num_toks = 0
        temp = temperature or 1.0                                         # node.py:451
        pending = None
        turn = 0
        # work list, chunks of max_ref_batch_size, right-padding with id 0: node.py:409-441
        for chunk in iter_ref_work(prompts, results, G, self.max_ref_batch_size):
            if chunk.n_scored == 0:                                      # only empty completions (node.py:428-432)
                continue
            with torch.cuda.device(self.device):
                slot = self._launch(chunk, turn & 1, temp)
            turn += 1
            if pending is not None:
                num_toks += self._finish(pending, results)
            pending = slot
        if pending is not None:
            num_toks += self._finish(pending, results)

        elapsed = time.perf_counter() - t0
        self.last_ref_tokens, self.last_ref_seconds = num_toks, elapsed
        logger.info("Ref log-probs non-KV batched completed: %d tokens in %.2fs (%.1f tok/s)",
                    num_toks, elapsed, num_toks / elapsed if elapsed > 0 else 0.0)


class _Slot:
    """Staging buffers and the completion event of one chunk in flight."""

    def __init__(self):
        self.host_in = self.dev_in = self.host_out = None
        self.done = torch.cuda.Event()
        self.chunk = self.keep = None
