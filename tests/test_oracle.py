"""Pins the CPU oracle: golden vectors, closed forms, brute force, independent library routines.

Each check is chosen so that a plausible slip (dropped max shift, wrong sign, temperature applied
to one term only, transposed weight, off-by-one gather) fails it.
"""
import math

import numpy as np
import pytest
import scipy.special
import scipy.stats

import oracle
from oracle import cport
from oracle.logprob_oracle import _brute_logprob
from golden_util import V_QWEN3, load, seeded_case

G = load()


# ---- golden vectors ---------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["s0", "s1", "s2"])
def test_golden_small_bruteforce(name):
    x, t, T = G[f"{name}_x"], G[f"{name}_t"], float(G[f"{name}_T"])
    np.testing.assert_allclose(oracle.logprob_rows(x, t, T), G[f"{name}_lp"], atol=1e-12)
    np.testing.assert_allclose(oracle.lse_rows(x, T), G[f"{name}_lse"], atol=1e-12)
    np.testing.assert_allclose(oracle.entropy_rows(x, T), G[f"{name}_ent"], atol=1e-12)


def test_golden_bf16_spike_rows():
    b, t = G["b0_bits"], G["b0_t"]
    np.testing.assert_allclose(oracle.logprob_rows(b, t, 1.0), G["b0_lp"], atol=1e-12)
    np.testing.assert_allclose(oracle.entropy_rows(b, 1.0), G["b0_ent"], atol=1e-11)
    np.testing.assert_array_equal(oracle.argmax_rows(b), G["b0_argmax"])


@pytest.mark.parametrize("name", ["c1", "c2", "c2t"])
def test_golden_full_vocab(name):
    x, t, T, exp = seeded_case(G, name)
    np.testing.assert_allclose(oracle.logprob_rows(x, t, T), exp["lp"], atol=1e-11)
    np.testing.assert_allclose(oracle.lse_rows(x, T), exp["lse"], atol=1e-11)
    np.testing.assert_allclose(oracle.entropy_rows(x, T), exp["ent"], atol=1e-10)
    np.testing.assert_array_equal(oracle.argmax_rows(x), exp["argmax"])
    # fp32 restatement of node.py:400-404 agrees with the closed form far inside the parity tolerance
    np.testing.assert_allclose(oracle.local_compute_logprobs_f32(x, t, T), exp["lp"], atol=2e-5)
    np.testing.assert_allclose(cport.local_compute_logprobs_c(x, t, T), exp["lp"], atol=5e-5)


def test_golden_lmhead():
    h, w, t, T = G["f0_h"], G["f0_w"], G["f0_t"], float(G["f0_T"])
    st = oracle.lmhead_stats(h, w, t, T, row_chunk=7)
    np.testing.assert_allclose(st["lp"], G["f0_lp"], atol=1e-12)
    np.testing.assert_allclose(st["lse"], G["f0_lse"], atol=1e-12)
    np.testing.assert_allclose(st["entropy"], G["f0_ent"], atol=1e-12)
    np.testing.assert_array_equal(st["argmax"], G["f0_argmax"])
    assert (st["top1"] >= st["top2"]).all()


# ---- closed forms -----------------------------------------------------------------------------
def test_all_equal_row_is_minus_log_v():
    x = np.full((2, V_QWEN3), -7.5, dtype=np.float32)
    np.testing.assert_allclose(oracle.logprob_rows(x, [0, V_QWEN3 - 1], 0.6), -math.log(V_QWEN3), atol=1e-12)
    assert abs(-math.log(V_QWEN3) - (-11.9312147)) < 1e-6      # ln 128 + ln 1187
    np.testing.assert_allclose(oracle.entropy_rows(x, 0.6), math.log(V_QWEN3), atol=1e-10)


@pytest.mark.parametrize("c,T", [(15.0, 1.0), (15.0, 0.7), (3.0, 2.0)])
def test_single_spike_closed_form(c, T):
    V = V_QWEN3
    x = np.zeros((1, V), dtype=np.float32)
    x[0, 4242] = c
    want_spike = -math.log1p((V - 1) * math.exp(-c / T))
    np.testing.assert_allclose(oracle.logprob_rows(x, [4242], T), want_spike, atol=1e-12)
    np.testing.assert_allclose(oracle.logprob_rows(x, [0], T), want_spike - c / T, atol=1e-12)


def test_shift_invariance_and_temperature_identity():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 1000)) * 4
    t = rng.integers(0, 1000, size=5)
    base = oracle.logprob_rows(x, t, 0.7)
    np.testing.assert_allclose(oracle.logprob_rows(x + 123.0, t, 0.7), base, atol=1e-10)
    np.testing.assert_allclose(oracle.logprob_rows(x / 0.7, t, 1.0), base, atol=1e-10)
    # a large offset must not overflow (the max shift is there)
    assert np.isfinite(oracle.lse_rows(x + 5000.0)).all()


def test_bruteforce_tiny_rows():
    rng = np.random.default_rng(1)
    for V in (1, 2, 3, 16):
        x = rng.standard_normal((4, V)) * 3
        for r in range(4):
            for t in range(V):
                for T in (1.0, 0.5):
                    assert abs(oracle.logprob_rows(x[r:r + 1], [t], T)[0] - _brute_logprob(x[r], t, T)) < 1e-12
    # probabilities of a row sum to one
    lp_all = oracle.full_log_softmax64(x, 0.8)
    np.testing.assert_allclose(np.exp(lp_all).sum(-1), 1.0, atol=1e-12)


def test_against_scipy_and_torch_routines():
    import torch
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((6, 5000)) * 3).astype(np.float32)
    t = rng.integers(0, 5000, size=6)
    T = 1.7
    z = x.astype(np.float64) / T
    np.testing.assert_allclose(oracle.lse_rows(x, T), scipy.special.logsumexp(z, axis=-1), atol=1e-12)
    ls = scipy.special.log_softmax(z, axis=-1)
    np.testing.assert_allclose(oracle.full_log_softmax64(x, T), ls, atol=1e-12)
    np.testing.assert_allclose(oracle.logprob_rows(x, t, T), ls[np.arange(6), t], atol=1e-12)
    np.testing.assert_allclose(oracle.entropy_rows(x, T), scipy.stats.entropy(np.exp(ls), axis=-1), atol=1e-10)
    tl = torch.log_softmax(torch.from_numpy(z), -1).numpy()
    np.testing.assert_allclose(oracle.full_log_softmax64(x, T), tl, atol=1e-12)


def test_entropy_bounds_and_limits():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((8, 777)) * 5
    h = oracle.entropy_rows(x, 1.0)
    assert (h >= 0).all() and (h <= math.log(777) + 1e-12).all()
    onehot = np.zeros((1, 50)); onehot[0, 7] = 80.0
    assert oracle.entropy_rows(onehot)[0] < 1e-20 + 1e-9
    # higher temperature flattens the distribution
    assert (oracle.entropy_rows(x, 2.0) > h).all()


def test_k3_properties():
    rng = np.random.default_rng(4)
    lp = -rng.random(100) * 5
    ref = lp + rng.standard_normal(100) * 0.3
    k = oracle.k3(lp, ref)
    assert (k >= 0).all()
    assert (oracle.k3(lp, lp) == 0).all()
    d = 1e-3
    assert abs(oracle.k3(np.array([-1.0]), np.array([-1.0 + d]))[0] - (d * d / 2 + d ** 3 / 6)) < 1e-12
    np.testing.assert_allclose(k, np.exp(ref - lp) - (ref - lp) - 1, atol=1e-12)
    # sign convention: d = ref_lp - lp (k3 estimates KL(pi || pi_ref) at a sample from pi)
    assert abs(oracle.k3(np.array([0.0]), np.array([-1.0]))[0] - (math.exp(-1) + 1 - 1)) < 1e-12


def test_argmax_first_max_wins():
    x = np.zeros((3, 100), dtype=np.float32)
    x[0, [5, 50]] = 2.0
    x[1, [99, 0]] = 1.0
    x[2, 60] = 3.0
    assert oracle.argmax_rows(x).tolist() == [5, 0, 60]
    assert oracle.argmax_rows(oracle.bf16_round(x)).tolist() == [5, 0, 60]


def test_bf16_conversions():
    import torch
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(10000).astype(np.float32) * 100,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.4e38, 1e-40], dtype=np.float32)])
    bits = oracle.bf16_round(x)
    want = torch.from_numpy(x).to(torch.bfloat16)
    np.testing.assert_array_equal(bits, want.view(torch.int16).numpy().view(np.uint16))   # round-to-nearest-even
    np.testing.assert_array_equal(oracle.bf16_to_f32(bits), want.float().numpy())


def test_lmhead_orientation_and_bruteforce():
    """logits = hidden @ W.T with W [V, H] (model.py:538); a transposed operand fails this."""
    rng = np.random.default_rng(6)
    n, H, V = 3, 5, 7
    h = oracle.bf16_round(rng.standard_normal((n, H)).astype(np.float32))
    w = oracle.bf16_round(rng.standard_normal((V, H)).astype(np.float32))
    hf, wf = oracle.bf16_to_f32(h).astype(np.float64), oracle.bf16_to_f32(w).astype(np.float64)
    logits = oracle.lmhead_logits64(h, w)
    assert logits.shape == (n, V)
    for r in range(n):
        for v in range(V):
            assert abs(logits[r, v] - math.fsum(hf[r, k] * wf[v, k] for k in range(H))) < 1e-12
    t = np.array([0, 6, 3])
    st = oracle.lmhead_stats(h, w, t, 0.5, row_chunk=2)
    np.testing.assert_allclose(st["lp"], oracle.logprob_rows(logits, t, 0.5), atol=1e-12)
    np.testing.assert_array_equal(st["argmax"], oracle.argmax_rows(logits))


# ---- restatements of the reference's own arithmetic ------------------------------------------------
def test_reference_kernel_check_restated():
    """tests/test_logprob_comparison.py:84-102: bf16 [1, 151936] ~ N(0, 1), T = 1, kernel vs
    `logits - logsumexp(logits)` in bf16, max abs diff < 5e-3."""
    rng = np.random.default_rng(7)
    bits = oracle.bf16_round(rng.standard_normal((1, V_QWEN3)).astype(np.float32))
    lse_b = oracle.bf16_to_f32(oracle.bf16_round(oracle.lse_rows(bits).astype(np.float32)))
    expected = oracle.bf16_to_f32(oracle.bf16_round(oracle.bf16_to_f32(bits) - lse_b[:, None]))
    for impl in (oracle.fused_log_softmax_f32, cport.metal_log_softmax):
        actual = oracle.bf16_to_f32(impl(bits, 1.0))
        assert np.abs(actual - expected).max() < 5e-3


@pytest.mark.parametrize("V", [4096, 4097, 8192 + 384, V_QWEN3, 166144, 5])
def test_metal_restatement_tails(V):
    """Tail handling of model.py:17-20,34-36: V % 4096 in {0, 1, 384}, V < one block."""
    rng = np.random.default_rng(V)
    x = (rng.standard_normal((2, V)) * 2).astype(np.float32)
    for T in (1.0, 0.7):
        want = oracle.full_log_softmax64(x, T)
        np.testing.assert_allclose(cport.metal_log_softmax(x, T), want, atol=2e-5)
        np.testing.assert_allclose(oracle.fused_log_softmax_f32(x, T), want, atol=2e-5)


def test_local_compute_logprobs_restatement_divides_by_temp():
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((4, 3000)) * 3).astype(np.float32)
    t = rng.integers(0, 3000, size=4)
    for T in (1.0, 0.7, 1.9):
        np.testing.assert_allclose(oracle.local_compute_logprobs_f32(x, t, T), oracle.logprob_rows(x, t, T), atol=1e-5)
    # bf16 input is upcast exactly first (node.py:401)
    b = oracle.bf16_round(x)
    np.testing.assert_allclose(oracle.local_compute_logprobs_f32(b, t, 0.7), oracle.logprob_rows(b, t, 0.7), atol=1e-5)


# ---- final RMSNorm (model.py:336-343, :536) -------------------------------------------------------
def test_rms_norm_closed_forms_and_library():
    import torch
    rng = np.random.default_rng(11)
    x = rng.standard_normal((5, 96)) * 3.0
    w = rng.standard_normal(96)
    y = oracle.rms_norm64(x, w, 1e-6)
    # independent library routine, float64
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x), (96,), torch.from_numpy(w), 1e-6).numpy()
    np.testing.assert_allclose(y, ref, rtol=1e-12, atol=1e-12)
    # brute force with exact summation: a dropped eps, a sum instead of a mean or sqrt instead of rsqrt fails
    for r in range(5):
        ms = math.fsum(v * v for v in x[r]) / 96
        want = [x[r, j] / math.sqrt(ms + 1e-6) * w[j] for j in range(96)]
        np.testing.assert_allclose(y[r], want, rtol=1e-12)
    # closed forms: unit RMS with w = 1; scale invariance as eps -> 0; constant row -> sign(x) * w
    y1 = oracle.rms_norm64(x, np.ones(96), 0.0)
    np.testing.assert_allclose(np.sqrt((y1 * y1).mean(-1)), 1.0, rtol=1e-12)
    np.testing.assert_allclose(oracle.rms_norm64(7.5 * x, w, 0.0), oracle.rms_norm64(x, w, 0.0), rtol=1e-12)
    np.testing.assert_allclose(oracle.rms_norm64(np.full((1, 8), -2.0), np.arange(8.0), 0.0), -np.arange(8.0)[None], rtol=1e-12)
    # eps matters for a tiny row: y = x / sqrt(x^2 + eps)
    np.testing.assert_allclose(oracle.rms_norm64(np.full((1, 4), 1e-3), np.ones(4), 1e-6), 1e-3 / math.sqrt(2e-6), rtol=1e-12)


def test_rms_norm_bf16_is_the_closed_form_within_two_roundings():
    import torch
    rng = np.random.default_rng(12)
    xb = oracle.bf16_round((rng.standard_normal((64, 256)) * 2.0).astype(np.float32))
    wb = oracle.bf16_round((1.0 + 0.1 * rng.standard_normal(256)).astype(np.float32))
    yb = oracle.rms_norm_bf16(xb, wb, 1e-6)
    assert yb.dtype == np.uint16 and yb.shape == xb.shape
    y64 = oracle.rms_norm64(xb, wb, 1e-6)
    got = oracle.to_f64(yb)
    # two bf16 roundings of 2^-8 relative each (+ tiny slack)
    assert np.all(np.abs(got - y64) <= 2.0 ** -7 * np.abs(y64) * 1.01 + 1e-30)
    assert np.mean(np.abs(got - y64) / np.abs(y64)) < 2.0 ** -9      # and unbiased on average
    # torch's bf16 rms_norm rounds once at the end; it must agree to the same bound
    tx = torch.from_numpy(oracle.bf16_to_f32(xb)).to(torch.bfloat16)
    tw = torch.from_numpy(oracle.bf16_to_f32(wb)).to(torch.bfloat16)
    ty = torch.nn.functional.rms_norm(tx, (256,), tw, 1e-6).float().numpy().astype(np.float64)
    assert np.all(np.abs(got - ty) <= 3 * 2.0 ** -8 * np.abs(y64) * 1.01 + 1e-30)


# ---- sampler (_sample_token, node.py:894-907) -------------------------------------------------------
def test_top_k_rows_against_argpartition_and_bruteforce():
    rng = np.random.default_rng(21)
    x = rng.standard_normal((6, 500))
    idx, val = oracle.top_k_rows(x, 20)
    for r in range(6):
        part = np.argpartition(x[r], x.shape[1] - 20)[-20:]          # the reference's expression, node.py:902
        assert set(part.tolist()) == set(idx[r].tolist())
        assert np.all(np.diff(val[r]) <= 0) and np.array_equal(val[r], x[r, idx[r]])
    # planted ties: equal values enter by ascending index, and the cut through a tie keeps the lowest ids
    t = np.zeros((1, 12)); t[0, [7, 2, 9]] = 5.0; t[0, [4, 1, 11, 6]] = 3.0
    idx, _ = oracle.top_k_rows(t, 5)
    assert idx[0].tolist() == [2, 7, 9, 1, 4]
    # NaN and -inf are never candidates (a -inf logit has probability zero in the draw of node.py:906, so the
    # law of the draw is the same with or without it); short rows are padded with -1
    s = np.array([[np.nan, 1.0, -np.inf, 2.0], [-np.inf] * 4])
    idx, val = oracle.top_k_rows(s, 4)
    assert idx[0].tolist() == [3, 1, -1, -1] and val[0, 0] == 2.0 and idx[1].tolist() == [-1] * 4
    # fewer finite logits than top_k: the draw is over the finite ones with their softmax masses (e^2 : e^1)
    short = np.full((1, 50), -np.inf); short[0, [5, 9]] = [1.0, 2.0]
    p9 = math.exp(2.0) / (math.exp(2.0) + math.exp(1.0))
    assert [int(oracle.sample_top_k(short, [u], 1.0, 20)[0][0]) for u in (0.0, p9 - 1e-9, p9 + 1e-9, 0.999)] == [9, 9, 5, 5]
    # no candidate at all: token -1, lp NaN
    tok, lp = oracle.sample_top_k(s[1:], [0.5], 1.0, 4)
    assert tok[0] == -1 and np.isnan(lp[0])


def test_sample_top_k_law_and_limits():
    rng = np.random.default_rng(22)
    x = rng.standard_normal((1, 300)) * 2.0
    T, k = 0.7, 8
    idx, val = oracle.top_k_rows(x, k)
    p = scipy.special.softmax(val[0] / T)                              # what a categorical over top_logits samples
    n = 20000
    us = (np.arange(n) + 0.5) / n
    toks = np.array([oracle.sample_top_k(x, [u], T, k)[0][0] for u in us[::20]])   # coarse grid: 1000 draws
    freq = np.array([(toks == i).mean() for i in idx[0]])
    np.testing.assert_allclose(freq, p, atol=2e-3)
    assert set(toks.tolist()) <= set(idx[0].tolist())                  # never outside the top k
    # limits: u -> 0 is the largest logit, u -> 1 the k-th; temperature 0 is argmax with lp at T = 1
    assert oracle.sample_top_k(x, [0.0], T, k)[0][0] == idx[0, 0] == np.argmax(x[0])
    assert oracle.sample_top_k(x, [1.0 - 1e-12], T, k)[0][0] == idx[0, k - 1]
    tok0, lp0 = oracle.sample_top_k(x, None, 0, k)
    assert tok0[0] == np.argmax(x[0])
    np.testing.assert_allclose(lp0, oracle.logprob_rows(x, tok0, 1.0))
    # the log-prob is over the WHOLE vocabulary at the sampling temperature, not renormalised over the top k
    tok, lp = oracle.sample_top_k(x, [0.3], T, k)
    np.testing.assert_allclose(lp[0], scipy.special.log_softmax(x[0] / T)[tok[0]], atol=1e-12)
    # brute force on a tiny row: k = 3 of 4 values, hand-computed CDF
    y = np.array([[0.0, math.log(2.0), math.log(4.0), -50.0]])
    got = [oracle.sample_top_k(y, [u], 1.0, 3)[0][0] for u in (0.0, 0.56, 0.58, 0.85, 0.86, 0.99)]
    assert got == [2, 2, 1, 1, 0, 0]                                   # masses 4/7, 2/7, 1/7


# ---- decode loops (node.py:556-612 Rollout, node.py:325-374 Judge) ----------------------------------
def _table_model(table):
    """Greedy transition table: logits[b] peak at table[token]."""
    V = len(table)
    def step(tokens):
        out = np.full((len(tokens), V), -5.0)
        out[np.arange(len(tokens)), [table[int(t)] for t in tokens]] = 5.0
        return out
    return step


def test_decode_loops_known_answers_at_temperature_zero():
    EOS = 0
    table = [0, 2, 3, 0, 5, 6, 7, 1, 8]                 # 1 -> 2 -> 3 -> 0 (EOS);  4 -> 5 -> 6 -> 7 -> 1 -> ...
    model = _table_model(table)
    first = np.full((2, 9), -5.0); first[0, 1] = 5.0; first[1, 4] = 5.0          # prompt 0 starts at 1, prompt 1 at 4
    lp_peak = 5.0 - np.log(np.exp(5.0) + 8 * np.exp(-5.0))
    # Rollout, G = 2, max_tokens = 5: EOS is kept with its log-prob; the other chain is cut at 5 tokens
    seq = oracle.rollout_decode(model, first, 2, 0.0, 5, EOS, None)
    assert [s["tokens"] for s in seq] == [[1, 2, 3, 0], [1, 2, 3, 0], [4, 5, 6, 7, 1], [4, 5, 6, 7, 1]]
    for s in seq:
        assert len(s["log_probs"]) == len(s["tokens"])                            # tests/test_grpo.py:78-80
        np.testing.assert_allclose(s["log_probs"], lp_peak, atol=1e-12)
    # Judge, same model: EOS ends the item and is NOT recorded
    res = oracle.judge_decode(model, first, 0.0, 5, EOS, None)
    assert [r["tokens"] for r in res] == [[1, 2, 3], [4, 5, 6, 7, 1]]
    # a first token equal to EOS: Rollout does not check it and goes on feeding it; Judge keeps it too (node.py:334-342)
    first_eos = np.full((1, 9), -5.0); first_eos[0, EOS] = 5.0
    assert oracle.rollout_decode(model, first_eos, 1, 0.0, 3, EOS, None)[0]["tokens"] == [0, 0]      # table[0] = 0 = EOS -> finished
    assert oracle.judge_decode(model, first_eos, 0.0, 3, EOS, None)[0]["tokens"] == [0]
    # finished rows are fed eos (Rollout) / 0 (Judge): record the inputs the model sees
    seen = []
    def spy(tokens):
        seen.append([int(t) for t in tokens]); return model(tokens)
    oracle.rollout_decode(spy, first, 1, 0.0, 6, 7, None)                          # EOS id 7 here
    assert seen[3] == [0, 7] and seen[4] == [0, 7]                                 # chain 1 drew 7 at step 3 and is fed 7 afterwards
    seen.clear()
    oracle.judge_decode(spy, first, 0.0, 6, 3, None)                               # EOS id 3: item 0 stops after [1, 2]
    assert seen[2][0] == 0                                                         # inactive item is fed 0 (node.py:350)


def test_decode_loops_use_the_sampler_with_temperature():
    rng = np.random.default_rng(31)
    V = 40
    W = rng.standard_normal((V, V)) * 2.0
    model = lambda tokens: W[np.asarray(tokens)]
    first = rng.standard_normal((2, V)) * 2.0
    us = rng.random((6, 4))
    seq = oracle.rollout_decode(model, first, 2, 0.8, 6, -1, us, top_k=5)
    assert all(len(s["tokens"]) == 6 for s in seq)
    # every token is one of the 5 best of its row, and its log-prob is the full-vocabulary one at T = 0.8
    for b, s in enumerate(seq):
        rows = [first[b // 2]] + [W[t] for t in s["tokens"][:-1]]
        for row, tok, lp in zip(rows, s["tokens"], s["log_probs"]):
            assert tok in np.argsort(-row)[:5]
            np.testing.assert_allclose(lp, scipy.special.log_softmax(row / 0.8)[tok], atol=1e-12)


def test_masked_vocabulary_rows_against_scipy_and_torch():
    """Rows with -inf entries (a masked vocabulary): the closed forms reduce to those of the kept entries, checked
    against scipy / torch.float64 on the same rows and against the oracle on the row with the masked entries removed."""
    import torch
    rng = np.random.default_rng(41)
    V, T = 3000, 0.8
    x = (rng.standard_normal((5, V)) * 3).astype(np.float32)
    keep = rng.random((5, V)) > 0.4
    keep[:, 7] = True
    xm = np.where(keep, x, -np.inf).astype(np.float32)
    t = np.array([7, 7, 7, 7, int(np.flatnonzero(~keep[4])[0])])        # the last target is a masked id
    z = xm.astype(np.float64) / T
    np.testing.assert_allclose(oracle.lse_rows(xm, T), scipy.special.logsumexp(z, axis=-1), atol=1e-12)
    tl = torch.log_softmax(torch.from_numpy(z), dim=-1).numpy()
    got = oracle.logprob_rows(xm, t, T)
    np.testing.assert_allclose(got[:4], tl[np.arange(4), t[:4]], atol=1e-12)
    assert got[4] == -np.inf
    for r in range(5):
        dense = x[r][keep[r]][None, :]
        np.testing.assert_allclose(oracle.lse_rows(xm[r:r + 1], T), oracle.lse_rows(dense, T), atol=1e-12)
        np.testing.assert_allclose(oracle.entropy_rows(xm[r:r + 1], T), oracle.entropy_rows(dense, T), atol=1e-12)
        assert oracle.argmax_rows(xm[r:r + 1])[0] == np.flatnonzero(keep[r])[np.argmax(x[r][keep[r]])]
    np.testing.assert_allclose(oracle.entropy_rows(xm, T), scipy.stats.entropy(np.exp(tl), axis=-1), atol=1e-10)
