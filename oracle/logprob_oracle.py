"""CPU restatement of Tome's token-log-prob path.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels in ``tome_amd``; it is never on
the product path.  Every function cites the reference lines it follows
(paths relative to the reference repository root).

Two families live here:

* fp64 closed forms (``lse_rows``, ``logprob_rows``, ``entropy_rows``,
  ``k3``, ``lmhead_logits64`` ...) - the mathematical statement of what
  ``mlx-impl/node.py:400-404`` and ``mlx-impl/model.py:16-66`` compute,
  evaluated on exactly-upcast inputs.  These are what parity is judged against.
* fp32 restatements that keep the reference's own arithmetic
  (``local_compute_logprobs_f32``, ``fused_log_softmax_f32``,
  ``process_ref_logprobs_batched``) - used for the CPU baseline timing and
  for the entry-point bookkeeping tests.

The reference's arithmetic lives partly in MLX (``mlx>=0.30.6``,
``pyproject.toml:17``; not vendored, not installable here): ``mx.logsumexp``,
``mx.take_along_axis``, ``mx.argmax`` and the bf16 matmul.  Their published
definitions are restated; what pins each function is listed below.

Pinning (tests/test_oracle.py):
  lse_rows / logprob_rows   closed forms (all-equal row -> -ln V, one spike
                            over zeros -> -log1p((V-1)e^-c)), shift invariance,
                            temperature identity, brute force with math.fsum on
                            V <= 16, scipy.special.logsumexp / log_softmax and
                            torch.float64 log_softmax as independent library
                            routines, committed golden vectors.
  entropy_rows              H(all-equal) = ln V, 0 <= H <= ln V, brute force,
                            scipy.stats.entropy.
  k3                        k3 >= 0, k3 = 0 iff lp == ref_lp, series expansion
                            d^2/2 for small d, brute force.  NOT in the
                            reference: pinned by closed form only.
  argmax_rows               planted ties (lowest index wins, NumPy convention).
                            MLX's own tie/NaN rule: parity unpinned.
  lmhead_logits64           brute-force triple loop on tiny shapes, numpy
                            float64 matmul.  MLX bf16 rounding of the
                            materialised logits: parity unpinned (the fused
                            path is specified as bf16 inputs, fp32 accumulate).
  fused_log_softmax_f32     the reference's own check restated
                            (tests/test_logprob_comparison.py:84-102, < 5e-3
                            vs logits - logsumexp on bf16 [1,151936]) and the
                            tail cases of model.py:17-20,34-36.
  local_compute_logprobs_f32  agreement with logprob_rows within 1e-5.
  rms_norm64 / rms_norm_bf16  the published definition of mx.fast.rms_norm
                            (MLX, not vendored): closed forms (w = 1 -> unit RMS,
                            x -> c x leaves y unchanged as eps -> 0, constant row
                            -> sign(x) w), torch.nn.functional.rms_norm in float64
                            as an independent library routine, brute force with
                            math.fsum.  The order of MLX's two bf16 roundings
                            (normalise, round, scale, round): parity unpinned.
  top_k_rows / sample_top_k  np.argpartition + sort as an independent library
                            route to the same candidate set, brute force on tiny
                            rows, planted ties, and the law of the draw: over a
                            fine grid of uniforms the token frequencies equal
                            softmax(top-k logits / T) (what mx.random.categorical
                            samples, node.py:906).  MLX's random stream itself and
                            argpartition's order among equal logits: parity unpinned.
  rollout_decode / judge_decode  known-answer tests on a scripted transition-table
                            model at temperature 0 (hand-derived token lists): EOS
                            kept with its log-prob in Rollout and dropped in Judge,
                            the first token never checked in Rollout, the
                            max_tokens cut, eos / 0 fed to finished rows.
  lora_merge_bf16 / update_weights  node.py:102-164.  The mathematics base + scale * B @ A
                            is pinned by closed forms (zero A -> the base bit for bit,
                            rank-1 outer product, B selecting rows of A, linearity in
                            scale on exactly representable inputs), brute-force loops
                            with math.fsum, numpy's float64 matmul and committed golden
                            vectors from exact rational arithmetic
                            (tests/golden/make_lora_golden.py); the
                            bookkeeping (last update wins, scale 0 -> 1.0, qkv_proj
                            over q/k/v, missing q/k/v slices revert to the base,
                            non-cumulative, untouched layers kept) by known-answer
                            tests on a two-layer toy model.  WHERE MLX rounds to bf16
                            (matmul output, scalar cast to bf16 before the multiply,
                            the sum) is restated from MLX's published semantics:
                            parity unpinned by the reference's tests.
  process_ref_logprobs_batched  known-answer tests on a stub model
                            (alignment, empty completion, temperature 0,
                            chunking, padding id 0) and the length contract of
                            tests/test_grpo.py:78-80.
"""
from __future__ import annotations

import math
from typing import Callable, Sequence

import numpy as np

__all__ = [
    "bf16_round", "bf16_to_f32", "to_f64", "lse_rows", "logprob_rows", "entropy_rows",
    "argmax_rows", "k3", "lmhead_logits64", "lmhead_stats", "full_log_softmax64",
    "local_compute_logprobs_f32", "fused_log_softmax_f32", "process_ref_logprobs_batched",
    "rms_norm64", "rms_norm_bf16", "top_k_rows", "sample_top_k", "rollout_decode", "judge_decode",
    "lora_merge64", "lora_merge_bf16", "update_weights",
]


# --------------------------------------------------------------------------
# bf16 <-> f32 (bit patterns held as uint16; weights are bf16 in the reference,
# mlx-impl/load_weights.py:20-22)
# --------------------------------------------------------------------------
def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit pattern (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    """bf16 bit pattern (uint16) -> float32, exact."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def to_f64(x: np.ndarray) -> np.ndarray:
    """Exact upcast.  uint16 arrays are read as bf16 bit patterns."""
    x = np.asarray(x)
    if x.dtype == np.uint16:
        return bf16_to_f32(x).astype(np.float64)
    return x.astype(np.float64)


# --------------------------------------------------------------------------
# fp64 closed forms
# --------------------------------------------------------------------------
def _scaled(x: np.ndarray, temperature: float) -> np.ndarray:
    # node.py:401 divides by temp; model.py:27 multiplies by 1/temp.  In fp64
    # the two agree to 1e-16 relative, far below the parity tolerance.
    return to_f64(x) / float(temperature)


def lse_rows(x: np.ndarray, temperature: float = 1.0) -> np.ndarray:
    """logsumexp over the last axis of x/T, fp64 (mx.logsumexp at node.py:402)."""
    z = _scaled(x, temperature)
    m = z.max(axis=-1, keepdims=True)
    return (m + np.log(np.exp(z - m).sum(axis=-1, keepdims=True)))[..., 0]


def logprob_rows(x: np.ndarray, targets: np.ndarray, temperature: float = 1.0) -> np.ndarray:
    """lp[r] = x[r, t_r]/T - logsumexp(x[r]/T), fp64 (node.py:400-404)."""
    z = _scaled(x, temperature)
    t = np.asarray(targets).astype(np.int64)
    picked = np.take_along_axis(z, t[..., None], axis=-1)[..., 0]
    m = z.max(axis=-1, keepdims=True)
    lse = (m + np.log(np.exp(z - m).sum(axis=-1, keepdims=True)))[..., 0]
    return picked - lse


def full_log_softmax64(x: np.ndarray, temperature: float = 1.0) -> np.ndarray:
    """out[r, j] = x[r, j]/T - logsumexp(x[r]/T): the matrix model.py:16-66 writes."""
    z = _scaled(x, temperature)
    m = z.max(axis=-1, keepdims=True)
    return z - (m + np.log(np.exp(z - m).sum(axis=-1, keepdims=True)))


def entropy_rows(x: np.ndarray, temperature: float = 1.0) -> np.ndarray:
    """H[r] = lse - sum_j p_j z_j with z = x/T, p = softmax(z).  Not in the reference.

    Entries of -inf (a masked vocabulary) have p_j = 0 and contribute nothing (0 log 0 = 0).
    """
    z = _scaled(x, temperature)
    m = z.max(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        e = np.exp(z - m)
        ez = np.where(np.isneginf(z), 0.0, e * z)
    s = e.sum(axis=-1)
    lse = m[..., 0] + np.log(s)
    return lse - ez.sum(axis=-1) / s


def argmax_rows(x: np.ndarray) -> np.ndarray:
    """Greedy token id, first maximum wins (int(mx.argmax(logits)), node.py:897)."""
    return np.argmax(to_f64(x), axis=-1).astype(np.int32)


def k3(lp: np.ndarray, ref_lp: np.ndarray) -> np.ndarray:
    """k3 = exp(d) - d - 1, d = ref_lp - lp: per-token estimator of KL(pi || pi_ref).

    Not in the reference (its wire format carries only log_probs and ref_log_probs,
    scheduler/proto/inference.proto:108-112); closed form only.
    """
    d = np.asarray(ref_lp, dtype=np.float64) - np.asarray(lp, dtype=np.float64)
    return np.expm1(d) - d


def lmhead_logits64(hidden: np.ndarray, weight: np.ndarray) -> np.ndarray:
    """logits = hidden @ weight.T in fp64 on exactly-upcast inputs.

    weight is [V, H] row-major as in model.py:538 (x @ embed_tokens.weight.T).
    """
    return to_f64(hidden) @ to_f64(weight).T


def rms_norm64(x: np.ndarray, weight: np.ndarray, eps: float = 1e-6) -> np.ndarray:
    """y = x * rsqrt(mean(x^2, -1) + eps) * w in fp64 on exactly-upcast inputs: RMSNorm.__call__ =
    mx.fast.rms_norm(x, self.weight, self.eps) (mlx-impl/model.py:336-343), applied to the last
    hidden states at model.py:536."""
    x64, w64 = to_f64(x), to_f64(weight)
    inv = 1.0 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + float(eps))
    return x64 * inv * w64


def rms_norm_bf16(x: np.ndarray, weight: np.ndarray, eps: float = 1e-6) -> np.ndarray:
    """The same with MLX's storage roundings, bf16 bit patterns in and out: statistics in fp32, the
    normalised value rounded to bf16, then multiplied by the bf16 weight and rounded again (the
    published rms_norm kernel of MLX; model.py:343 passes bf16 activations and weights)."""
    x32, w32 = bf16_to_f32(x), bf16_to_f32(weight)
    ms = (x32.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    inv = (1.0 / np.sqrt(ms + float(eps))).astype(np.float32)
    t = bf16_to_f32(bf16_round(x32 * inv))
    return bf16_round(w32 * t)


def top_k_rows(x: np.ndarray, top_k: int = 20):
    """The ``top_k`` largest entries of each row: ``mx.argpartition(scaled_logits, size - top_k)[-top_k:]``
    (mlx-impl/node.py:902; temperature > 0 does not change the set), returned ordered by value
    descending, equal values by ascending index.  NaN and -inf entries are never candidates (a -inf
    logit has probability zero under the categorical of node.py:906, so leaving it out changes no draw);
    a row with fewer than ``top_k`` candidates is padded with index -1.
    Returns (idx int32 [rows, top_k], val float64)."""
    x64 = to_f64(x)
    rows, V = x64.shape
    idx = np.full((rows, top_k), -1, dtype=np.int32)
    val = np.zeros((rows, top_k), dtype=np.float64)
    for r in range(rows):
        cand = np.flatnonzero(x64[r] > -np.inf)                      # drops NaN too
        order = cand[np.lexsort((cand, -x64[r, cand]))][:top_k]     # value descending, then index ascending
        idx[r, :len(order)] = order
        val[r, :len(order)] = x64[r, order]
    return idx, val


def sample_top_k(x: np.ndarray, uniforms, temperature: float, top_k: int = 20):
    """_sample_token (mlx-impl/node.py:894-907) with the randomness made explicit.

    temperature == 0: ``int(mx.argmax(logits))`` (node.py:896-897).  Otherwise the categorical draw
    over ``top_logits = (logits / temperature)[top_indices]`` (node.py:899-907) taken as the inverse
    CDF of softmax(top_logits) at ``uniforms[r]`` in [0, 1), candidates in the order of
    ``top_k_rows``.  Returns (token int32 [rows], lp float64 [rows]) where lp is the log-prob of the
    token under the full softmax at ``temperature or 1.0`` (node.py:590,605).  A row without any
    candidate (all -inf / NaN) yields token -1 and lp NaN."""
    x64 = to_f64(x)
    rows = x64.shape[0]
    idx, val = top_k_rows(x, top_k)
    tok = np.empty(rows, dtype=np.int32)
    for r in range(rows):
        n = int((idx[r] >= 0).sum())
        if n == 0 or temperature == 0 or uniforms is None:
            tok[r] = idx[r, 0]
            continue
        z = val[r, :n] / float(temperature)
        p = np.exp(z - z[0])
        cdf = np.cumsum(p)
        j = int(np.searchsorted(cdf, float(uniforms[r]) * cdf[-1], side="right"))
        tok[r] = idx[r, min(j, n - 1)]
    with np.errstate(invalid="ignore"):
        lp = logprob_rows(x64, np.maximum(tok, 0), float(temperature) or 1.0)
    lp = np.where(tok < 0, np.nan, lp)
    return tok, lp


def lmhead_stats(hidden: np.ndarray, weight: np.ndarray, targets: np.ndarray,
                 temperature: float = 1.0, row_chunk: int = 64) -> dict:
    """Row statistics of the lm_head logits without keeping the full matrix.

    Returns fp64 ``lp``, ``lse``, ``entropy`` and int32 ``argmax`` plus the two
    largest scaled logits per row (``top1``, ``top2``; tests use the gap to
    decide whether an argmax comparison is meaningful).
    """
    h = to_f64(hidden)
    w = to_f64(weight)
    t = np.asarray(targets).astype(np.int64)
    n = h.shape[0]
    out = {k: np.empty(n, dtype=np.float64) for k in ("lp", "lse", "entropy", "top1", "top2")}
    out["argmax"] = np.empty(n, dtype=np.int32)
    for r0 in range(0, n, row_chunk):
        r1 = min(n, r0 + row_chunk)
        z = (h[r0:r1] @ w.T) / float(temperature)
        m = z.max(axis=-1, keepdims=True)
        e = np.exp(z - m)
        s = e.sum(axis=-1)
        lse = m[:, 0] + np.log(s)
        out["lse"][r0:r1] = lse
        out["lp"][r0:r1] = np.take_along_axis(z, t[r0:r1, None], axis=-1)[:, 0] - lse
        out["entropy"][r0:r1] = lse - (e * z).sum(axis=-1) / s
        out["argmax"][r0:r1] = np.argmax(z, axis=-1)
        part = np.partition(z, -2, axis=-1)[:, -2:]
        out["top1"][r0:r1] = part[:, 1]
        out["top2"][r0:r1] = part[:, 0]
    return out


# --------------------------------------------------------------------------
# fp32 restatements that keep the reference's arithmetic
# --------------------------------------------------------------------------
def local_compute_logprobs_f32(logits: np.ndarray, ids: np.ndarray, temp: float) -> np.ndarray:
    """node.py:400-404 in NumPy fp32: upcast, DIVIDE by temp, logsumexp, gather, subtract."""
    x = (bf16_to_f32(logits) if logits.dtype == np.uint16 else logits.astype(np.float32, copy=False))
    x = x / np.float32(temp)
    m = x.max(axis=-1, keepdims=True)
    log_z = m + np.log(np.exp(x - m).sum(axis=-1, keepdims=True, dtype=np.float32))
    tok = np.take_along_axis(x, np.asarray(ids).astype(np.int64)[..., None], axis=-1)[..., 0]
    return (tok - log_z[..., 0]).astype(np.float32)


def fused_log_softmax_f32(logits: np.ndarray, temperature: float = 1.0) -> np.ndarray:
    """model.py:16-66 in NumPy fp32, output in the input's dtype.

    Keeps the kernel's arithmetic choices: multiply by inv_temp = 1/temp
    (model.py:27), running max floored at -1e30 (:28), fp32 sum of exp(x*inv_temp
    - row_max) (:43-50), lse cast to the I/O dtype T before the subtraction,
    which is itself done in T (:57,60).  The 1024-thread reduction ORDER is not
    reproduced here (oracle/metal_logsoftmax.c does that); fp32 sums are taken
    pairwise by NumPy.
    """
    is_bf16 = logits.dtype == np.uint16
    x = bf16_to_f32(logits) if is_bf16 else logits.astype(np.float32, copy=False)
    inv_temp = np.float32(1.0) / np.float32(temperature)
    z = x * inv_temp
    row_max = np.maximum(z.max(axis=-1, keepdims=True), np.float32(-1e30))
    s = np.exp(z - row_max).sum(axis=-1, keepdims=True, dtype=np.float32)
    lse = (row_max + np.log(s)).astype(np.float32)
    if is_bf16:
        lse_t = bf16_to_f32(bf16_round(lse))
        z_t = bf16_to_f32(bf16_round(z))
        return bf16_round(z_t - lse_t)
    return (z - lse).astype(np.float32)


def process_ref_logprobs_batched(prompts: Sequence, results: Sequence, G: int,
                                 temperature: float = 1.0, *,
                                 reference_model: Callable[[np.ndarray], np.ndarray],
                                 max_ref_batch_size: int = 32) -> int:
    """node.py:391-461 with NumPy in place of MLX.

    ``reference_model(full_ids uint32 [B, L]) -> logits [B, L, V]`` stands in for
    ``self.reference_model(full_ids, cache=None)[0]`` (node.py:443).  Mutates
    ``results[p].completions[g].ref_log_probs`` via ``extend`` (node.py:458) and
    returns the number of completion tokens scored (node.py:454).
    """
    all_work = []
    for p_idx, p in enumerate(prompts):                                   # node.py:409-414
        p_toks = list(p.tokens)
        for g in range(G):
            all_work.append((p_idx, g, p_toks, list(results[p_idx].completions[g].tokens)))
    num_toks = 0
    for c0 in range(0, len(all_work), max_ref_batch_size):               # node.py:419-421
        chunk = all_work[c0:c0 + max_ref_batch_size]
        seqs = [p + c[:-1] if c else p for _, _, p, c in chunk]          # node.py:427-437
        max_len = max(len(s) for s in seqs)
        full_ids = np.array([s + [0] * (max_len - len(s)) for s in seqs], dtype=np.uint32)  # :439-441
        logits = reference_model(full_ids)                               # node.py:443
        for i, (p_idx, g, p_toks, c_toks) in enumerate(chunk):           # node.py:446-454
            if not c_toks:
                continue
            lo = len(p_toks) - 1
            c_logits = logits[i, lo:lo + len(c_toks)]
            lps = local_compute_logprobs_f32(c_logits, np.array(c_toks, dtype=np.uint32),
                                             temperature or 1.0)        # node.py:451
            results[p_idx].completions[g].ref_log_probs.extend(lps.tolist())  # node.py:458
            num_toks += len(c_toks)
    return num_toks


# --------------------------------------------------------------------------
# UpdateWeights (mlx-impl/node.py:102-164); weights are bf16 bit patterns (uint16)
# --------------------------------------------------------------------------
def lora_merge64(base: np.ndarray, lora_a: np.ndarray, lora_b: np.ndarray, scale: float) -> np.ndarray:
    """base_W + scale * (lora_B @ lora_A) in fp64 on exactly-upcast inputs, no intermediate rounding:
    the mathematical statement of node.py:128,137.  lora_a [rank, in], lora_b [out, rank]."""
    return to_f64(base) + float(scale) * (to_f64(lora_b) @ to_f64(lora_a))


def _bf16_of_f64(x: np.ndarray) -> np.ndarray:
    """float64 -> bf16 bit patterns, one correct rounding (ties to even).  Going through float32
    first would round twice; instead round the float64 significand directly."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    f32 = x.astype(np.float32)
    bits = bf16_round(f32)
    # repair double rounding: compare against both neighbours in exact float64 arithmetic
    up = bf16_to_f32(bits).astype(np.float64)
    lo_bits = np.where(up > x, _bf16_step(bits, -1), bits)
    hi_bits = _bf16_step(lo_bits, +1)
    lo = bf16_to_f32(lo_bits).astype(np.float64)
    hi = bf16_to_f32(hi_bits).astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        d_lo, d_hi = x - lo, hi - x
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & ((lo_bits & 1) == 1))
    out = np.where(pick_hi, hi_bits, lo_bits).astype(np.uint16)
    special = ~np.isfinite(x) | ~np.isfinite(hi) | ~np.isfinite(lo) | (x == 0)
    return np.where(special, bits, out).astype(np.uint16)


def _bf16_step(bits: np.ndarray, direction: int) -> np.ndarray:
    """Next bf16 value towards +inf (direction +1) or -inf (-1), on bit patterns of finite values."""
    b = bits.astype(np.int32)
    neg = (b & 0x8000) != 0
    mag = b & 0x7FFF
    if direction > 0:
        mag2 = np.where(neg, mag - 1, mag + 1)
        flip = neg & (mag == 0)
        out = np.where(flip, 0x0001, np.where(neg, 0x8000 | mag2, mag2))
    else:
        mag2 = np.where(neg, mag + 1, mag - 1)
        flip = (~neg) & (mag == 0)
        out = np.where(flip, 0x8001, np.where(neg, 0x8000 | mag2, mag2))
    return (out & 0xFFFF).astype(np.uint16)


def lora_merge_bf16(base: np.ndarray, lora_a, lora_b, scale: float) -> np.ndarray:
    """The same with the roundings of the reference's bf16 array expressions, bit patterns in and out:
    ``delta_W = scale * (lora_B @ lora_A)`` (node.py:128) is a bf16 matmul (exact products, wide
    accumulation, ONE rounding to bf16) times a Python scalar that MLX first casts to the array's
    dtype, the product rounded to bf16; ``base_W + delta_W`` (node.py:137) rounds once more.
    ``lora_a is None`` stands for the ``mx.zeros_like`` deltas of node.py:143-145."""
    b64 = to_f64(base)
    if lora_a is None:
        return _bf16_of_f64(b64 + 0.0)
    d = to_f64(_bf16_of_f64(to_f64(lora_b) @ to_f64(lora_a)))
    s = to_f64(bf16_round(np.float32(scale).reshape(1)))[0]
    d2 = to_f64(_bf16_of_f64(s * d))
    return _bf16_of_f64(b64 + d2)


def update_weights(policy: list, reference: list, updates: Sequence, *, num_heads: int, num_kv_heads: int,
                   head_dim: int) -> int:
    """node.py:114-151 on dict models: ``policy[i]`` / ``reference[i]`` map ``"self_attn.qkv_proj"``,
    ``"mlp.gate_up_proj"``, ``"mlp.down_proj"`` to bf16 bit patterns [out, in]; ``updates`` carry
    ``layer_idx, param_name, lora_A, lora_B`` (bytes), ``shape_A, shape_B, lora_scale``
    (scheduler/proto/inference.proto:68-76).  Mutates ``policy``; returns the matrices rebuilt."""
    layer_deltas: dict = {}
    for up in updates:                                                    # node.py:117-130
        if not up.lora_A or not up.lora_B:
            continue
        a = np.frombuffer(up.lora_A, dtype=np.uint16).reshape(list(up.shape_A))
        b = np.frombuffer(up.lora_B, dtype=np.uint16).reshape(list(up.shape_B))
        scale = up.lora_scale if up.lora_scale != 0.0 else 1.0
        layer_deltas.setdefault(up.layer_idx, {})[up.param_name] = (a, b, scale)
    rebuilt = 0
    for layer_idx, deltas in layer_deltas.items():                        # node.py:132-151
        ref, tgt = reference[layer_idx], policy[layer_idx]
        base = ref["self_attn.qkv_proj"]
        if "self_attn.qkv_proj" in deltas:
            tgt["self_attn.qkv_proj"] = lora_merge_bf16(base, *deltas["self_attn.qkv_proj"])
            rebuilt += 1
        elif any(k in deltas for k in ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj")):
            q_size, k_size = num_heads * head_dim, num_kv_heads * head_dim
            parts = []
            for name, lo, hi in (("self_attn.q_proj", 0, q_size), ("self_attn.k_proj", q_size, q_size + k_size),
                                 ("self_attn.v_proj", q_size + k_size, base.shape[0])):
                a, b, sc = deltas.get(name, (None, None, 1.0))
                parts.append(lora_merge_bf16(base[lo:hi], a, b, sc))
            tgt["self_attn.qkv_proj"] = np.concatenate(parts, axis=0)
            rebuilt += 1
        for name in ("mlp.gate_up_proj", "mlp.down_proj"):
            if name in deltas:
                tgt[name] = lora_merge_bf16(ref[name], *deltas[name])
                rebuilt += 1
    return rebuilt


def _draw(logits_row: np.ndarray, u, temperature: float, top_k: int):
    """One call of _sample_token or argmax (node.py:598-602) and the log-prob lookup (node.py:605)."""
    tok, lp = sample_top_k(logits_row[None, :], None if u is None else [u], temperature, top_k)
    return int(tok[0]), float(lp[0])


def rollout_decode(model_step: Callable[[np.ndarray], np.ndarray], last_logits: np.ndarray, G: int,
                   temperature: float, max_tokens: int, eos_token_id: int, uniforms, top_k: int = 20) -> list:
    """The sampling half of _rollout_batched, mlx-impl/node.py:556-612, row by row as the reference does.

    ``uniforms[step][row]`` replaces MLX's random stream (step 0 = first tokens).
    ``model_step(tokens int64 [N]) -> logits [N, V]`` stands for the model call of node.py:585."""
    num_prompts = last_logits.shape[0]
    active_tokens, active_lps = [], []
    for p_idx in range(num_prompts):                                       # node.py:556-571
        for g_idx in range(G):
            u = None if temperature == 0 else uniforms[0][p_idx * G + g_idx]
            token, lp = _draw(to_f64(last_logits[p_idx]), u, temperature, top_k)
            active_tokens.append(token)
            active_lps.append(lp)
    total = num_prompts * G
    seq = [{"tokens": [active_tokens[i]], "log_probs": [active_lps[i]]} for i in range(total)]   # node.py:574
    finished = [False] * total                                             # node.py:575
    for step in range(max_tokens - 1):                                     # node.py:578
        if all(finished):
            break
        logits = to_f64(model_step(np.array(active_tokens, dtype=np.int64)))   # node.py:583-585
        new_active = []
        for b in range(total):                                             # node.py:592-610
            if finished[b]:
                new_active.append(eos_token_id)
                continue
            u = None if temperature == 0 else uniforms[step + 1][b]
            token, lp = _draw(logits[b], u, temperature, top_k)
            seq[b]["tokens"].append(token)
            seq[b]["log_probs"].append(lp)
            if token == eos_token_id or len(seq[b]["tokens"]) >= max_tokens:
                finished[b] = True
            new_active.append(token)
        active_tokens = new_active
    return seq


def judge_decode(model_step: Callable[[np.ndarray], np.ndarray], first_logits: np.ndarray, temperature: float,
                 max_tokens: int, eos_token_id: int, uniforms, top_k: int = 20) -> list:
    """The sampling half of a Judge chunk, mlx-impl/node.py:325-374."""
    B = first_logits.shape[0]
    active_tokens, results = [], []
    for i in range(B):                                                     # node.py:334-342
        u = None if temperature == 0 else uniforms[0][i]
        token, lp = _draw(to_f64(first_logits[i]), u, temperature, top_k)
        active_tokens.append(token)
        results.append({"tokens": [token], "log_probs": [lp]})
    active = [True] * B                                                    # node.py:344
    for step in range(max_tokens - 1):                                     # node.py:346
        if not any(active):
            break
        inputs = np.array([t if active[i] else 0 for i, t in enumerate(active_tokens)], dtype=np.int64)  # :350
        logits = to_f64(model_step(inputs))
        for i in range(B):                                                 # node.py:357-374
            if not active[i]:
                continue
            u = None if temperature == 0 else uniforms[step + 1][i]
            token, lp = _draw(logits[i], u, temperature, top_k)
            active_tokens[i] = token
            if token == eos_token_id:
                active[i] = False
            else:
                results[i]["tokens"].append(token)
                results[i]["log_probs"].append(lp)
    return results


def _brute_logprob(row: Sequence[float], target: int, temperature: float = 1.0) -> float:
    """math.fsum brute force for tiny rows; used only by the oracle's own tests."""
    z = [float(v) / temperature for v in row]
    m = max(z)
    return z[target] - (m + math.log(math.fsum(math.exp(v - m) for v in z)))
