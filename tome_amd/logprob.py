"""Token-log-prob operators on torch (ROCm) tensors, backed by libtome_logprob.so.

The first two functions keep the reference's names, argument order and meaning:

* ``fused_log_softmax(logits, temperature=1.0)``     mlx-impl/model.py:77-89
* ``local_compute_logprobs(logits, ids, temp)``      mlx-impl/node.py:400-404

The others are the additive, fused forms of the same path: one scalar per row
instead of a [rows, V] matrix (``token_logprobs``), the lm_head matmul of
mlx-impl/model.py:538 folded in (``fused_lmhead_logprobs``), and the GRPO
policy + reference pair with k3 KL and entropy (``grpo_dual_logprobs``).

Launches are asynchronous on the current torch stream, like MLX's lazy graph
(forced by ``mx.eval`` at node.py:456); reading a result on the host synchronises.
"""
from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from . import _lib
from ._lib import TOME_BF16, TOME_F32


class TokenLogprobs(NamedTuple):
    lp: torch.Tensor                    # float32, log-prob of the target id
    lse: Optional[torch.Tensor]         # float32, logsumexp of x / temperature
    entropy: Optional[torch.Tensor]     # float32, entropy of softmax(x / temperature), nats
    argmax: Optional[torch.Tensor]      # int32, first maximum of the row


class SampledTokens(NamedTuple):
    token: torch.Tensor                 # int32, the drawn (or greedy) token id; -1 for masked rows
    lp: torch.Tensor                    # float32, its log-prob under the full softmax
    argmax: torch.Tensor                # int32, first maximum of the row
    topk_idx: Optional[torch.Tensor]    # int32 [..., top_k], candidates by descending logit
    topk_logit: Optional[torch.Tensor]  # float32 [..., top_k], their raw logits


class DualLogprobs(NamedTuple):
    lp: torch.Tensor        # policy log-prob of the target id
    ref_lp: torch.Tensor    # reference-model log-prob of the target id
    k3: torch.Tensor        # exp(ref_lp - lp) - (ref_lp - lp) - 1
    entropy: torch.Tensor   # entropy of the policy distribution


def _require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("tome_amd operators run on a ROCm GPU only (there is no CPU fallback); "
                               f"got a tensor on {t.device}")
        if t.device != dev:
            raise ValueError("all tensors must be on the same device")
    return dev


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return TOME_F32
    if t.dtype == torch.bfloat16:
        return TOME_BF16
    raise TypeError(f"logits must be float32 or bfloat16, got {t.dtype}")


def _check_temperature(temperature: float) -> float:
    temperature = float(temperature)
    if not (temperature > 0.0) or temperature == float("inf"):
        # the reference maps 0 to 1.0 at its call sites (`temperature or 1.0`, node.py:451)
        raise ValueError(f"temperature must be finite and > 0, got {temperature}")
    return temperature


def _rows_view(x: torch.Tensor) -> torch.Tensor:
    """[..., V] -> [rows, V] with unit stride along V, copying only when no such view exists."""
    if x.dim() == 0:
        raise ValueError("expected a tensor with a vocabulary axis")
    V = x.shape[-1]
    if x.dim() == 1:
        x = x.unsqueeze(0)
    if x.stride(-1) != 1 and V > 1:
        x = x.contiguous()
    if x.dim() == 2:
        return x
    try:
        return x.view(-1, V)
    except RuntimeError:
        return x.reshape(-1, V)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(dev: torch.device) -> int:
    """Raw hipStream_t of torch's current stream on ``dev`` (the launch stream of every call)."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # a fraction of the cost of the Stream object
    if raw is not None and dev.index is not None:
        return raw(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


class _on_device:
    """``torch.cuda.device(dev)`` that does nothing when ``dev`` is already current (the usual case):
    the HIP launches of the library go to the current device, so it has to be the tensors' one."""

    def __init__(self, dev: torch.device):
        idx = dev.index if dev.index is not None else torch.cuda.current_device()
        self._guard = None if idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            return self._guard.__exit__(*exc)
        return False


def _as_i32(t, n: int, dev: torch.device, what: str) -> torch.Tensor:
    t = torch.as_tensor(t, device=dev) if not isinstance(t, torch.Tensor) else t
    if t.device != dev:
        raise ValueError(f"{what} must be on {dev}")
    if t.numel() != n:
        raise ValueError(f"{what} has {t.numel()} entries, expected {n}")
    if t.dtype.is_floating_point or t.dtype == torch.bool:
        raise TypeError(f"{what} must be an integer tensor")
    return t.reshape(-1).to(torch.int32).contiguous()


def _row_valid(lead_shape, n_rows: int, lengths, row_valid, dev) -> Optional[torch.Tensor]:
    """Row mask from either an explicit mask or per-sequence lengths over a [B, L] leading shape."""
    if lengths is not None and row_valid is not None:
        raise ValueError("pass lengths or row_valid, not both")
    if row_valid is not None:
        rv = row_valid if isinstance(row_valid, torch.Tensor) else torch.as_tensor(row_valid, device=dev)
        if rv.numel() != n_rows:
            raise ValueError(f"row_valid has {rv.numel()} entries, expected {n_rows}")
        return rv.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
    if lengths is None:
        return None
    if len(lead_shape) != 2:
        raise ValueError("lengths needs inputs shaped [batch, seq, ...]")
    B, L = lead_shape
    ln = lengths if isinstance(lengths, torch.Tensor) else torch.as_tensor(lengths)
    if ln.numel() != B:
        raise ValueError(f"lengths has {ln.numel()} entries, expected {B}")
    ln = ln.to(device=dev, dtype=torch.int64).reshape(B, 1)
    return (torch.arange(L, device=dev).reshape(1, L) < ln).to(torch.int32).reshape(-1).contiguous()


def _workspace(nbytes: int, dev: torch.device) -> Optional[torch.Tensor]:
    return torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes > 0 else None


def token_logprobs(logits: torch.Tensor, targets, temperature: float = 1.0, lengths=None, *,
                   row_valid=None, want_lse: bool = False, want_entropy: bool = False,
                   want_argmax: bool = False) -> TokenLogprobs:
    """Log-prob of ``targets`` under softmax(logits / temperature), one scalar per row.

    ``logits`` is [..., V] float32 or bfloat16; ``targets`` has the leading shape.
    Rows masked out by ``lengths`` (per sequence, for [B, L, V] inputs) or
    ``row_valid`` are not read; their outputs are 0 (argmax -1).  Outputs are float32
    with the leading shape.
    """
    lib = _lib.load_library()
    dev = _require_gpu(logits)
    temperature = _check_temperature(temperature)
    dtype = _dtype_code(logits)
    lead = tuple(logits.shape[:-1])
    x = _rows_view(logits)
    rows, V = x.shape
    tg = _as_i32(targets, rows, dev, "targets")
    rv = _row_valid(lead, rows, lengths, row_valid, dev)
    with _on_device(dev):
        lp = torch.empty(rows, dtype=torch.float32, device=dev)
        lse = torch.empty(rows, dtype=torch.float32, device=dev) if want_lse else None
        ent = torch.empty(rows, dtype=torch.float32, device=dev) if want_entropy else None
        amax = torch.empty(rows, dtype=torch.int32, device=dev) if want_argmax else None
        ws_bytes = lib.tome_row_logprob_workspace(rows, V)
        ws = _workspace(ws_bytes, dev)
        _lib.check(lib.tome_row_logprob(x.data_ptr(), dtype, rows, V, x.stride(0) if rows > 1 else V,
                                        tg.data_ptr(), _ptr(rv), temperature, lp.data_ptr(), _ptr(lse),
                                        _ptr(ent), _ptr(amax), _ptr(ws), ws_bytes, _stream(dev)))

    def _shaped(t):
        return None if t is None else t.reshape(lead)
    return TokenLogprobs(_shaped(lp), _shaped(lse), _shaped(ent), _shaped(amax))


def token_logprobs_rows(logits: torch.Tensor, row_index, targets, temperature: float = 1.0, *,
                        want_lse: bool = False, want_entropy: bool = False, want_argmax: bool = False) -> TokenLogprobs:
    """``token_logprobs`` for a list of rows, packed: entry i scores row ``row_index[i]`` of the flattened
    ``logits`` ([..., V] -> [rows, V]) against ``targets[i]``; every output has ``len(row_index)`` entries.

    This is the slicing of mlx-impl/node.py:449 (the completion rows of each sequence of a padded chunk) and
    local_compute_logprobs on the slices (node.py:400-404) for the whole chunk in one launch; rows that are not
    listed are neither read nor launched.  An index outside the matrix scores NaN (argmax -1).
    """
    lib = _lib.load_library()
    dev = _require_gpu(logits)
    temperature = _check_temperature(temperature)
    dtype = _dtype_code(logits)
    x = _rows_view(logits)
    rows, V = x.shape
    idx = torch.as_tensor(row_index, device=dev) if not isinstance(row_index, torch.Tensor) else row_index
    n = idx.numel()
    idx = _as_i32(idx, n, dev, "row_index")
    tg = _as_i32(targets, n, dev, "targets")
    with _on_device(dev):
        lp = torch.empty(n, dtype=torch.float32, device=dev)
        lse = torch.empty(n, dtype=torch.float32, device=dev) if want_lse else None
        ent = torch.empty(n, dtype=torch.float32, device=dev) if want_entropy else None
        amax = torch.empty(n, dtype=torch.int32, device=dev) if want_argmax else None
        ws_bytes = lib.tome_row_logprob_workspace(n, V)
        ws = _workspace(ws_bytes, dev)
        _lib.check(lib.tome_row_logprob_rows(x.data_ptr(), dtype, rows, V, x.stride(0) if rows > 1 else V, idx.data_ptr(), n,
                                             tg.data_ptr(), temperature, lp.data_ptr(), _ptr(lse), _ptr(ent), _ptr(amax),
                                             _ptr(ws), ws_bytes, _stream(dev)))
    return TokenLogprobs(lp, lse, ent, amax)


def sample_tokens(logits: torch.Tensor, temperature: float, top_k: int = 20, *, uniforms=None,
                  generator: Optional[torch.Generator] = None, row_valid=None, lengths=None,
                  want_topk: bool = False) -> SampledTokens:
    """One decode step for a batch of rows: ``_sample_token(logits, temperature, top_k)``
    (mlx-impl/node.py:894-907) for every row at once, with the log-prob of the chosen token that
    the decode loops look up afterwards (node.py:590,605) from the same pass.

    ``temperature == 0`` is greedy (node.py:896-897) and the log-prob then uses temperature 1.0, as
    ``temperature or 1.0`` does at node.py:590.  Otherwise the token is drawn from
    softmax(top-k logits / temperature) by inverse CDF at ``uniforms`` (float32 in [0, 1), one per
    row; drawn with ``torch.rand`` from ``generator`` when omitted) - candidates ordered by
    logit descending, equal logits by ascending id.  MLX's random stream is not reproduced.
    """
    lib = _lib.load_library()
    dev = _require_gpu(logits)
    greedy = float(temperature) == 0.0
    temperature = _check_temperature(1.0 if greedy else temperature)
    dtype = _dtype_code(logits)
    lead = tuple(logits.shape[:-1])
    x = _rows_view(logits)
    rows, V = x.shape
    if not 1 <= int(top_k) <= 32:
        raise ValueError("top_k must be in 1..32")
    rv = _row_valid(lead, rows, lengths, row_valid, dev)
    with _on_device(dev):
        u = None
        if not greedy:
            if uniforms is None:
                u = torch.rand(rows, dtype=torch.float32, device=dev, generator=generator)
            else:
                u = torch.as_tensor(uniforms, dtype=torch.float32, device=dev).reshape(-1).contiguous()
                if u.numel() != rows:
                    raise ValueError(f"uniforms must have one value per row ({rows}), got {u.numel()}")
        packed = torch.empty((3, rows), dtype=torch.int32, device=dev)   # token | lp bits | argmax: one allocation,
        tok, lp, amax = packed[0], packed[1].view(torch.float32), packed[2]  # and (token, lp) leave in one copy
        tki = torch.empty((rows, top_k), dtype=torch.int32, device=dev) if want_topk else None
        tkl = torch.empty((rows, top_k), dtype=torch.float32, device=dev) if want_topk else None
        ws_bytes = lib.tome_row_sample_workspace(dtype, rows, V, int(top_k))
        ws = _workspace(ws_bytes, dev)
        _lib.check(lib.tome_row_sample(x.data_ptr(), dtype, rows, V, x.stride(0) if rows > 1 else V, _ptr(u), _ptr(rv),
                                       temperature, int(top_k), tok.data_ptr(), lp.data_ptr(), None, amax.data_ptr(),
                                       _ptr(tki), _ptr(tkl), _ptr(ws), ws_bytes, _stream(dev)))
    return SampledTokens(tok.reshape(lead), lp.reshape(lead), amax.reshape(lead),
                         None if tki is None else tki.reshape(*lead, top_k),
                         None if tkl is None else tkl.reshape(*lead, top_k))


class DecodeStepGraph:
    """``sample_tokens`` for one fixed decode-batch shape, captured once as a HIP graph and replayed.

    A decode loop (mlx-impl/node.py:575-612) calls the sampler once per generated token with the
    same shapes; replaying a captured graph removes the per-call host work (argument checks, output
    allocation, two kernel launches).  ``logits`` and ``uniforms`` are the static input buffers: write
    the step's logits and fresh uniforms into them (``copy_``, ``uniform_``), call ``replay()``, read
    ``token`` / ``lp`` / ``argmax``.  The kernels allocate nothing and clear nothing with memsets,
    so every replay computes exactly what the eager call does.
    """

    def __init__(self, logits: torch.Tensor, temperature: float, top_k: int = 20, *, uniforms: Optional[torch.Tensor] = None):
        dev = _require_gpu(logits)
        self.logits = logits
        rows = logits.numel() // logits.shape[-1]
        self.uniforms = uniforms if uniforms is not None else torch.rand(rows, dtype=torch.float32, device=dev)
        self.temperature, self.top_k = float(temperature), int(top_k)
        self._stream = torch.cuda.Stream(device=dev)       # default priority
        self._graph = torch.cuda.CUDAGraph()
        self._stream.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(self._stream):
            sample_tokens(self.logits, self.temperature, self.top_k, uniforms=self.uniforms)   # warm-up outside capture
        self._stream.synchronize()
        with torch.cuda.graph(self._graph, stream=self._stream):
            out = sample_tokens(self.logits, self.temperature, self.top_k, uniforms=self.uniforms)
        self.token, self.lp, self.argmax = out.token, out.lp, out.argmax

    def replay(self) -> SampledTokens:
        self._graph.replay()
        return SampledTokens(self.token, self.lp, self.argmax, None, None)


def local_compute_logprobs(logits: torch.Tensor, ids: torch.Tensor, temp: float) -> torch.Tensor:
    """Drop-in for the closure at mlx-impl/node.py:400-404.

    ``logits`` [Lc, V] (bf16 or f32), ``ids`` [Lc] token ids, ``temp`` > 0.  Returns
    float32 [Lc]: ``logits[ids]/temp - logsumexp(logits/temp)`` computed in fp32 in one
    pass over the row.
    """
    return token_logprobs(logits, ids, temp).lp


def fused_log_softmax(logits: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """Drop-in for mlx-impl/model.py:77-89: full log-softmax with temperature, same shape and dtype."""
    lib = _lib.load_library()
    dev = _require_gpu(logits)
    temperature = _check_temperature(temperature)
    dtype = _dtype_code(logits)
    x = _rows_view(logits)
    rows, V = x.shape
    with _on_device(dev):
        out = torch.empty((rows, V), dtype=logits.dtype, device=dev)
        row_lse = torch.empty(rows, dtype=torch.float32, device=dev)
        ws_bytes = lib.tome_row_logprob_workspace(rows, V)
        ws = _workspace(ws_bytes, dev)
        _lib.check(lib.tome_full_log_softmax(x.data_ptr(), out.data_ptr(), dtype, rows, V,
                                             x.stride(0) if rows > 1 else V, V, temperature,
                                             row_lse.data_ptr(), _ptr(ws), ws_bytes, _stream(dev)))
    return out.reshape(logits.shape)


def _check_fused_inputs(hidden: torch.Tensor, *weights: torch.Tensor):
    dev = _require_gpu(hidden, *weights)
    if hidden.dtype != torch.bfloat16 or any(w.dtype != torch.bfloat16 for w in weights):
        raise TypeError("hidden and lm_head weights must be bfloat16 "
                        "(the reference loads bf16 weights, mlx-impl/load_weights.py:20-22)")
    H = hidden.shape[-1]
    for w in weights:
        if w.dim() != 2 or w.shape[1] != H:
            raise ValueError(f"weight must be [V, {H}] (rows = vocabulary, as embed_tokens.weight), got {tuple(w.shape)}")
        if w.shape != weights[0].shape:
            raise ValueError("policy and reference weights must have the same shape")
    lead = tuple(hidden.shape[:-1])
    h2 = _rows_view(hidden)
    ws_ = [w if w.stride(1) == 1 else w.contiguous() for w in weights]
    return dev, lead, h2, ws_


def fused_lmhead_logprobs(hidden: torch.Tensor, weight: torch.Tensor, targets, temperature: float = 1.0,
                          lengths=None, *, row_valid=None, want_lse: bool = False,
                          want_entropy: bool = False, want_argmax: bool = False,
                          norm_weight: torch.Tensor | None = None, norm_eps: float = 1e-6) -> TokenLogprobs:
    """Log-probs of ``targets`` under softmax((hidden @ weight.T) / temperature) without the logits.

    ``hidden`` [..., H] bf16 (already through the final norm, mlx-impl/model.py:536),
    ``weight`` [V, H] bf16 (the tied embedding matrix, model.py:538).  bf16 products are
    accumulated in fp32; unlike the reference the logits are not rounded to bf16.
    ``want_argmax`` adds the greedy token id (first maximum, as ``int(mx.argmax(logits))`` at
    mlx-impl/node.py:897); logits closer than fp32 accumulation noise may swap.
    With ``norm_weight`` (bf16 [H]) ``hidden`` holds the PRE-norm states and the model's final
    RMSNorm (``mx.fast.rms_norm(x, weight, eps)``, model.py:336-343, :536) is applied to the valid
    rows first.
    """
    lib = _lib.load_library()
    dev, lead, h2, (w,) = _check_fused_inputs(hidden, weight)
    temperature = _check_temperature(temperature)
    n, H = h2.shape
    V = w.shape[0]
    tg = _as_i32(targets, n, dev, "targets")
    rv = _row_valid(lead, n, lengths, row_valid, dev)
    with _on_device(dev):
        lp = torch.empty(n, dtype=torch.float32, device=dev)
        lse = torch.empty(n, dtype=torch.float32, device=dev) if want_lse else None
        ent = torch.empty(n, dtype=torch.float32, device=dev) if want_entropy else None
        amax = torch.empty(n, dtype=torch.int32, device=dev) if want_argmax else None
        if norm_weight is None:
            ws_bytes = lib.tome_fused_lmhead_logprob_workspace(n, H, V)
            ws = _workspace(ws_bytes, dev)
            _lib.check(lib.tome_fused_lmhead_logprob(h2.data_ptr(), w.data_ptr(), n, H, V,
                                                     h2.stride(0) if n > 1 else H, w.stride(0),
                                                     tg.data_ptr(), _ptr(rv), temperature, lp.data_ptr(), _ptr(lse),
                                                     _ptr(ent), _ptr(amax), _ptr(ws), ws_bytes, _stream(dev)))
        else:
            if norm_weight.dtype != torch.bfloat16 or norm_weight.shape != (H,) or norm_weight.device != dev:
                raise ValueError(f"norm_weight must be a bfloat16 [{H}] tensor on {dev}")
            nw = norm_weight.contiguous()
            ws_bytes = lib.tome_norm_lmhead_logprob_workspace(n, H, V)
            ws = _workspace(ws_bytes, dev)
            _lib.check(lib.tome_norm_lmhead_logprob(h2.data_ptr(), nw.data_ptr(), float(norm_eps), w.data_ptr(), n, H, V,
                                                    h2.stride(0) if n > 1 else H, w.stride(0),
                                                    tg.data_ptr(), _ptr(rv), temperature, lp.data_ptr(), _ptr(lse),
                                                    _ptr(ent), _ptr(amax), _ptr(ws), ws_bytes, _stream(dev)))

    def _shaped(t):
        return None if t is None else t.reshape(lead)
    return TokenLogprobs(_shaped(lp), _shaped(lse), _shaped(ent), _shaped(amax))


def grpo_dual_logprobs(hidden: torch.Tensor, w_policy: torch.Tensor, w_ref: torch.Tensor, targets,
                       temperature: float = 1.0, lengths=None, *, row_valid=None) -> DualLogprobs:
    """Policy and reference log-probs of ``targets`` plus k3 KL and policy entropy, per token.

    The two weight sets share ``hidden`` (in Tome the policy is the reference plus a merged
    LoRA delta, mlx-impl/node.py:102-164).  k3 and entropy have no counterpart in the
    reference node; they are defined by their closed forms.
    """
    lib = _lib.load_library()
    dev, lead, h2, (wp, wr) = _check_fused_inputs(hidden, w_policy, w_ref)
    if wp.stride(0) != wr.stride(0):
        wr = wr.contiguous()
        wp = wp.contiguous()
    temperature = _check_temperature(temperature)
    n, H = h2.shape
    V = wp.shape[0]
    tg = _as_i32(targets, n, dev, "targets")
    rv = _row_valid(lead, n, lengths, row_valid, dev)
    with _on_device(dev):
        outs = [torch.empty(n, dtype=torch.float32, device=dev) for _ in range(4)]
        ws_bytes = lib.tome_grpo_dual_workspace(n, H, V)
        ws = _workspace(ws_bytes, dev)
        _lib.check(lib.tome_grpo_dual(h2.data_ptr(), wp.data_ptr(), wr.data_ptr(), n, H, V,
                                      h2.stride(0) if n > 1 else H, wp.stride(0), tg.data_ptr(), _ptr(rv),
                                      temperature, outs[0].data_ptr(), outs[1].data_ptr(), outs[2].data_ptr(),
                                      outs[3].data_ptr(), _ptr(ws), ws_bytes, _stream(dev)))
    return DualLogprobs(*(o.reshape(lead) for o in outs))


def grpo_pair_logprobs(hidden_policy: torch.Tensor, hidden_ref: torch.Tensor, w_policy: torch.Tensor, targets,
                       temperature: float = 1.0, lengths=None, *, w_ref: torch.Tensor | None = None,
                       row_valid=None, norm_weight: torch.Tensor | None = None,
                       norm_eps: float = 1e-6) -> DualLogprobs:
    """``grpo_dual_logprobs`` for the reference's two-model layout: one hidden-state matrix per model.

    Tome's ``UpdateWeights`` merges LoRA deltas into attention and MLP weights only
    (mlx-impl/node.py:134-151), so policy and reference models differ in their final hidden
    states and share the final norm and the lm_head (mlx-impl/model.py:536-538): ``w_ref``
    defaults to ``w_policy``.  ``norm_weight`` as in ``fused_lmhead_logprobs``, applied to both.
    """
    lib = _lib.load_library()
    ws_in = (w_policy,) if w_ref is None else (w_policy, w_ref)
    dev, lead, h2, ws_ = _check_fused_inputs(hidden_policy, *ws_in)
    _require_gpu(hidden_policy, hidden_ref)
    if hidden_ref.dtype != torch.bfloat16 or hidden_ref.shape != hidden_policy.shape:
        raise ValueError("hidden_ref must be bfloat16 with hidden_policy's shape")
    r2 = _rows_view(hidden_ref)
    wp = ws_[0]
    wr = ws_[1] if w_ref is not None else wp
    if wp.stride(0) != wr.stride(0):
        wp, wr = wp.contiguous(), wr.contiguous()
    n, H = h2.shape
    if n > 1 and h2.stride(0) != r2.stride(0):
        h2, r2 = h2.contiguous(), r2.contiguous()
    temperature = _check_temperature(temperature)
    V = wp.shape[0]
    tg = _as_i32(targets, n, dev, "targets")
    rv = _row_valid(lead, n, lengths, row_valid, dev)
    nw = None
    if norm_weight is not None:
        _require_gpu(hidden_policy, norm_weight)
        if norm_weight.dtype != torch.bfloat16 or norm_weight.shape != (H,):
            raise ValueError(f"norm_weight must be bfloat16 [{H}]")
        nw = norm_weight.contiguous()
    with _on_device(dev):
        outs = [torch.empty(n, dtype=torch.float32, device=dev) for _ in range(4)]
        ws_bytes = lib.tome_grpo_pair_workspace(n, H, V, 1 if nw is not None else 0)
        ws = _workspace(ws_bytes, dev)
        _lib.check(lib.tome_grpo_pair(h2.data_ptr(), r2.data_ptr(), _ptr(nw), float(norm_eps), wp.data_ptr(),
                                      wr.data_ptr(), n, H, V, h2.stride(0) if n > 1 else H, wp.stride(0),
                                      tg.data_ptr(), _ptr(rv), temperature, outs[0].data_ptr(), outs[1].data_ptr(),
                                      outs[2].data_ptr(), outs[3].data_ptr(), _ptr(ws), ws_bytes, _stream(dev)))
    return DualLogprobs(*(o.reshape(lead) for o in outs))
