"""``UpdateWeights`` of Tome's inference node (mlx-impl/node.py:102-164) on the batched merge kernel.

The reference forms ``delta_W = scale * (lora_B @ lora_A)`` per update as a full bf16 matrix and then
assigns ``policy_W = base_W + delta_W`` per parameter: three passes over every weight plus the delta's
own storage.  Here every touched parameter is one job of a single ``tome_lora_merge`` launch that reads
the reference model's weight once and writes the policy's weight once, in place.

The bookkeeping follows the reference line by line: updates grouped by layer with the last update of a
``(layer, param)`` winning (node.py:130), ``lora_scale == 0`` meaning 1.0 (node.py:127), empty updates
skipped with a warning (node.py:119-121), a whole ``qkv_proj`` delta taking precedence over per-projection
ones and missing q/k/v slices reverting to the base (node.py:136-146), unknown parameter names ignored,
and the result being non-cumulative: base weights always come from the frozen reference model.
"""
from __future__ import annotations

import ctypes
import logging
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib

logger = logging.getLogger(__name__)


@dataclass
class LayerUpdate:
    """scheduler/proto/inference.proto:68-76; ``lora_A`` / ``lora_B`` are raw bf16 bytes."""
    layer_idx: int = 0
    param_name: str = ""
    lora_A: bytes = b""
    lora_B: bytes = b""
    shape_A: List[int] = field(default_factory=list)
    shape_B: List[int] = field(default_factory=list)
    lora_scale: float = 0.0


@dataclass
class WeightUpdateResponse:
    """scheduler/proto/inference.proto:78-81"""
    success: bool = False
    policy_version: int = 0


# (base, out, lora_A or None, lora_B or None, scale): one weight matrix (or row slice of one) to rebuild
MergeJob = Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor], float]


def lora_merge(jobs: Sequence[MergeJob]) -> None:
    """``out = base + scale * (lora_B @ lora_A)`` for every job, in one launch on the current stream.

    bf16 throughout, rounded where the reference's expressions round (node.py:128,137): the product to
    bf16, the scaling by the bf16-rounded scalar to bf16, the sum to bf16.  ``lora_A`` [rank, cols] and
    ``lora_B`` [rows, rank] may both be None (``out = base + 0``).  ``out`` may be ``base`` itself.
    """
    if not jobs:
        return
    lib = _lib.load_library()
    arr = (_lib.TomeLoraJob * len(jobs))()
    keep = []
    dev = jobs[0][0].device
    for i, (base, out, a, b, scale) in enumerate(jobs):
        for t in (base, out, a, b):
            if t is None:
                continue
            if not t.is_cuda:
                raise RuntimeError("tome_amd operators run on a ROCm GPU only (there is no CPU fallback); "
                                   f"got a tensor on {t.device}")
            if t.device != dev:
                raise ValueError("all tensors of a merge must be on the same device")
            if t.dtype != torch.bfloat16 or t.dim() != 2:
                raise TypeError("LoRA merges work on 2-D bfloat16 tensors (inference.proto:71-72)")
        if out.shape != base.shape or base.stride(1) != 1 or out.stride(1) != 1:
            raise ValueError("base and out must have the same shape and unit stride along the input dimension")
        rows, cols = base.shape
        rank = 0
        if (a is None) != (b is None):
            raise ValueError("lora_A and lora_B come together")
        if a is not None:
            rank = a.shape[0]
            if a.shape != (rank, cols) or b.shape != (rows, rank):
                raise ValueError(f"lora_A must be [rank, {cols}] and lora_B [{rows}, rank]; got {tuple(a.shape)}, {tuple(b.shape)}")
            a, b = a.contiguous(), b.contiguous()
            if rank % 8 != 0:                       # zero-pad the rank: extra terms of the product are exact zeros
                pad = 8 - rank % 8
                a = torch.cat([a, a.new_zeros(pad, cols)], 0)
                b = torch.cat([b, b.new_zeros(rows, pad)], 1).contiguous()
                rank += pad
            keep += [a, b]
        j = arr[i]
        j.base, j.out = base.data_ptr(), out.data_ptr()
        j.lora_a, j.lora_b = (a.data_ptr(), b.data_ptr()) if a is not None else (None, None)
        j.rows, j.cols, j.rank = rows, cols, rank
        j.base_stride = base.stride(0) if rows > 1 else cols
        j.out_stride = out.stride(0) if rows > 1 else cols
        j.scale = float(scale)
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        jobs_ptr = ctypes.cast(arr, ctypes.c_void_p)
        ws_bytes = lib.tome_lora_merge_workspace(jobs_ptr, len(jobs))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
        _lib.check(lib.tome_lora_merge(jobs_ptr, len(jobs), None if ws is None else ws.data_ptr(), ws_bytes, stream))
    del keep, ws                                   # launches are stream-ordered; torch frees on the same stream


def _upload_lora(entries: Sequence[Tuple[object, float]], dev: torch.device) -> dict:
    """All adapters of a request in ONE host-to-device copy.

    Each ``LayerUpdate`` is decoded as the reference does - ``np.frombuffer(raw, uint16).reshape(shape)`` viewed
    as bf16 (node.py:123-126) - with the rank zero-padded to a multiple of 8 (extra terms of the product are exact
    zeros) and every matrix starting on a 16-byte boundary of one staging array.  Returns
    ``{id(update): (lora_A [rank, in], lora_B [out, rank])}`` as views of the uploaded buffer.
    """
    parts, layout, total = [], {}, 0
    for up, _ in entries:
        a = np.frombuffer(up.lora_A, dtype=np.uint16).reshape([int(v) for v in up.shape_A])
        b = np.frombuffer(up.lora_B, dtype=np.uint16).reshape([int(v) for v in up.shape_B])
        if a.ndim != 2 or b.ndim != 2 or a.shape[0] != b.shape[1]:
            raise ValueError(f"lora_A {a.shape} and lora_B {b.shape} do not form a rank decomposition")
        pad = -a.shape[0] % 8
        if pad:
            a = np.concatenate([a, np.zeros((pad, a.shape[1]), np.uint16)], 0)
            b = np.concatenate([b, np.zeros((b.shape[0], pad), np.uint16)], 1)
        offs = []
        for m in (a, b):
            offs.append((total, m.shape))
            parts.append((total, m))
            total += -(-m.size // 8) * 8
        layout[id(up)] = offs
    stage = np.zeros(total, dtype=np.uint16)
    for off, m in parts:
        stage[off:off + m.size] = m.reshape(-1)
    buf = torch.from_numpy(stage.view(np.int16)).to(dev).view(torch.bfloat16)
    return {key: tuple(buf[off:off + sh[0] * sh[1]].view(sh) for off, sh in offs) for key, offs in layout.items()}


def apply_weight_update(policy_layers: Sequence, reference_layers: Sequence, updates: Sequence, *,
                        num_heads: int, num_kv_heads: int, head_dim: int) -> int:
    """The try-block of ``UpdateWeights`` (node.py:114-151): rebuild the touched policy weights.

    ``policy_layers[i]`` / ``reference_layers[i]`` expose ``self_attn.qkv_proj.weight``,
    ``mlp.gate_up_proj.weight`` and ``mlp.down_proj.weight`` as bf16 [out, in] tensors on the GPU
    (mlx-impl/model.py's module layout); the policy's are overwritten in place.  Returns the number of
    weight matrices rebuilt.
    """
    layer_deltas: dict = {}
    for up in updates:                                               # node.py:117-130
        if not up.lora_A or not up.lora_B:
            logger.warning("Empty LoRA update for layer %d", up.layer_idx)
            continue
        scale = up.lora_scale if up.lora_scale != 0.0 else 1.0       # node.py:127
        layer_deltas.setdefault(int(up.layer_idx), {})[up.param_name] = (up, scale)

    jobs: List[MergeJob] = []
    rebuilt = 0
    uploaded: dict = {}                                              # device -> adapters of that device's layers

    def lora(entry, dev):
        if dev not in uploaded:
            mine = [e for li, d in layer_deltas.items() for e in d.values()
                    if reference_layers[li].self_attn.qkv_proj.weight.device == dev]
            uploaded[dev] = _upload_lora(mine, dev)
        up, scale = entry
        a, b = uploaded[dev][id(up)]
        return a, b, scale

    for layer_idx, deltas in layer_deltas.items():                   # node.py:132-151
        ref_layer, target = reference_layers[layer_idx], policy_layers[layer_idx]
        qkv_base, qkv_out = ref_layer.self_attn.qkv_proj.weight, target.self_attn.qkv_proj.weight
        dev = qkv_base.device
        if "self_attn.qkv_proj" in deltas:                           # node.py:136-138
            a, b, s = lora(deltas["self_attn.qkv_proj"], dev)
            jobs.append((qkv_base, qkv_out, a, b, s))
            rebuilt += 1
        elif any(k in deltas for k in ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj")):
            q_size, k_size = num_heads * head_dim, num_kv_heads * head_dim        # node.py:140-142
            bounds = {"self_attn.q_proj": (0, q_size), "self_attn.k_proj": (q_size, q_size + k_size),
                      "self_attn.v_proj": (q_size + k_size, qkv_base.shape[0])}
            for name, (lo, hi) in bounds.items():                    # node.py:143-146
                if name in deltas:
                    a, b, s = lora(deltas[name], dev)
                    jobs.append((qkv_base[lo:hi], qkv_out[lo:hi], a, b, s))
                else:                                                # zeros_like delta: the slice reverts to the base
                    jobs.append((qkv_base[lo:hi], qkv_out[lo:hi], None, None, 1.0))
            rebuilt += 1
        for name, mod in (("mlp.gate_up_proj", "gate_up_proj"), ("mlp.down_proj", "down_proj")):   # node.py:148-151
            if name in deltas:
                a, b, s = lora(deltas[name], dev)
                jobs.append((getattr(ref_layer.mlp, mod).weight, getattr(target.mlp, mod).weight, a, b, s))
                rebuilt += 1
    for base, out, *_ in jobs:
        if base.data_ptr() == out.data_ptr():
            raise ValueError("policy and reference models share weight storage: the merge would overwrite the frozen base")
    lora_merge(jobs)
    return rebuilt


class WeightUpdateServicer:
    """The ``UpdateWeights`` slice of InferenceNodeServicer (mlx-impl/node.py:49-164).

    ``model`` / ``reference_model`` expose ``.layers``; ``num_heads`` is read from the first layer's
    ``self_attn.num_heads`` (node.py:100).  The prefix cache the reference clears after an update
    (node.py:155-157) belongs to the serving engine and is represented by the ``on_update`` hook.
    """

    def __init__(self, model, reference_model, head_dim: int, num_kv_heads: int, on_update=None):
        self.model = model                                           # node.py:65
        self.reference_model = reference_model                       # node.py:66
        self.head_dim = head_dim
        self.num_kv_heads = num_kv_heads
        self.num_heads = model.layers[0].self_attn.num_heads         # node.py:100
        self.policy_version = 0
        self.on_update = on_update

    async def UpdateWeights(self, request, context=None) -> WeightUpdateResponse:  # noqa: N802
        return self.update_weights(request)

    def update_weights(self, request) -> WeightUpdateResponse:
        """Synchronous body of ``UpdateWeights``; failures are reported, not raised (node.py:162-164)."""
        logger.info("Weight update request: %d layers", len(request.updates))
        try:
            apply_weight_update(self.model.layers, self.reference_model.layers, request.updates,
                                num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, head_dim=self.head_dim)
            torch.cuda.current_stream().synchronize()                # mx.eval(self.model.parameters()), node.py:153
            self.policy_version += 1                                 # node.py:154
            if self.on_update is not None:
                self.on_update()                                     # node.py:155-157
            logger.info("Weight update applied: policy_version=%d", self.policy_version)
            return WeightUpdateResponse(success=True, policy_version=self.policy_version)
        except Exception as e:                                       # node.py:162-164
            logger.error("Weight update error: %s", e)
            return WeightUpdateResponse(success=False)
