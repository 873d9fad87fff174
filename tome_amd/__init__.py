"""tome_amd: Tome's token-log-prob path on AMD Instinct MI355X (gfx950).

Host-side mirror of the reference's operator interface for this path
(``fused_log_softmax`` in mlx-impl/model.py:77-89, ``local_compute_logprobs`` and
``_process_ref_logprobs_batched`` in mlx-impl/node.py:391-461) on PyTorch-ROCm
tensors, calling hand-written HIP kernels through the C ABI of
``libtome_logprob.so``.  There is no CPU or eager-PyTorch fallback: every op
raises if the HIP library is missing or the tensors are not on a GPU.
"""
from .logprob import (  # noqa: F401
    fused_log_softmax,
    local_compute_logprobs,
    token_logprobs,
    token_logprobs_rows,
    sample_tokens,
    DecodeStepGraph,
    fused_lmhead_logprobs,
    grpo_dual_logprobs,
    grpo_pair_logprobs,
    TokenLogprobs,
    SampledTokens,
    DualLogprobs,
)
from .decode import rollout_decode, judge_decode  # noqa: F401
from .weights import LayerUpdate, WeightUpdateResponse, WeightUpdateServicer, apply_weight_update, lora_merge  # noqa: F401
from .node import Prompt, Completion, PromptRollout, RefLogprobServicer  # noqa: F401
from .wire import (  # noqa: F401
    PackedRefChunk, pack_ref_work, scatter_ref_logprobs, rollout_response_to_json, rollout_response_from_json,
)
from ._lib import TomeError, lib_path, load_library  # noqa: F401

__all__ = [
    "fused_log_softmax", "local_compute_logprobs", "token_logprobs", "token_logprobs_rows", "sample_tokens", "DecodeStepGraph", "fused_lmhead_logprobs",
    "grpo_dual_logprobs", "grpo_pair_logprobs", "LayerUpdate", "WeightUpdateResponse", "WeightUpdateServicer",
    "apply_weight_update", "lora_merge", "TokenLogprobs", "SampledTokens", "DualLogprobs", "Prompt", "Completion", "PromptRollout",
    "RefLogprobServicer", "rollout_decode", "judge_decode", "PackedRefChunk", "pack_ref_work", "scatter_ref_logprobs",
    "rollout_response_to_json", "rollout_response_from_json", "TomeError", "lib_path", "load_library",
]
