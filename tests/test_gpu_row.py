"""GPU parity of the row kernel (tome_row_logprob through the Python mirror) against the fp64 oracle.

Tolerances are the ones stated for this path: 1e-4 abs for fp32 logits, 2e-3 abs for bf16 inputs (the bf16 -> fp32
upcast is exact, so the bf16 cases are also held to 1e-4); target ids and argmax bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import V_QWEN3, bf16_bits_of

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4
TOL_BF16 = 2e-3


def _check(logits_t, targets, T, **kw):
    r = tome_amd.token_logprobs(logits_t, torch.from_numpy(targets).to(logits_t.device), T,
                                want_lse=True, want_entropy=True, want_argmax=True, **kw)
    torch.cuda.synchronize()
    x = bf16_bits_of(logits_t) if logits_t.dtype == torch.bfloat16 else logits_t.cpu().numpy()
    return r, x


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,V,T", [
    (1, 16, 1.0), (3, 4096, 1.0), (5, 4097, 0.7), (7, 8191, 1.3), (64, V_QWEN3, 1.0),
    (2, 166144, 0.5), (300, 1000, 2.0), (2500, 4104, 1.0), (1, V_QWEN3, 0.7), (17, 37, 1.0),
])
def test_row_matches_oracle(dev, dtype, rows, V, T):
    rng = np.random.default_rng(rows * 1000003 + V)
    x32 = (rng.standard_normal((rows, V)) * 2.0).astype(np.float32)
    t = rng.integers(0, V, size=rows).astype(np.int32)
    xt = torch.from_numpy(x32).to(dev).to(dtype)
    r, x = _check(xt, t, T)
    tol = TOL_F32
    np.testing.assert_allclose(r.lp.cpu().numpy(), oracle.logprob_rows(x, t, T), atol=tol, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), oracle.lse_rows(x, T), atol=tol, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), oracle.entropy_rows(x, T), atol=tol, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy(), oracle.argmax_rows(x))
    assert (r.lp.cpu().numpy() <= 1e-6).all()


def test_row_strided_and_misaligned_views(dev):
    """Row slices of a [B, L, V] tensor (node.py:449) and views that break 16-byte alignment."""
    rng = np.random.default_rng(5)
    big = torch.from_numpy(rng.standard_normal((4, 9, 1031)).astype(np.float32)).to(dev)
    t = rng.integers(0, 1031, size=5).astype(np.int32)
    sl = big[2, 3:8]                       # strided rows, contiguous V
    r, x = _check(sl, t, 0.9)
    np.testing.assert_allclose(r.lp.cpu().numpy(), oracle.logprob_rows(x, t, 0.9), atol=TOL_F32, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy(), oracle.argmax_rows(x))
    odd = big[1, :5, 1:1030]               # base pointer off by one element, V = 1029
    t2 = rng.integers(0, 1029, size=5).astype(np.int32)
    r, _ = _check(odd, t2, 1.0)
    x = odd.cpu().numpy()
    np.testing.assert_allclose(r.lp.cpu().numpy(), oracle.logprob_rows(x, t2, 1.0), atol=TOL_F32, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy(), oracle.argmax_rows(x))
    b16 = big.to(torch.bfloat16)[0, :, 3:1027]   # bf16, base off by 6 bytes
    t3 = rng.integers(0, 1024, size=9).astype(np.int32)
    r, x = _check(b16, t3, 1.0)
    np.testing.assert_allclose(r.lp.cpu().numpy(), oracle.logprob_rows(x, t3, 1.0), atol=TOL_F32, rtol=0)
    np.testing.assert_array_equal(r.argmax.cpu().numpy(), oracle.argmax_rows(x))


def test_closed_forms(dev):
    V = V_QWEN3
    flat = torch.zeros((2, V), device=dev, dtype=torch.float32) + 3.25
    r = tome_amd.token_logprobs(flat, torch.tensor([0, V - 1], device=dev), 1.0, want_entropy=True, want_argmax=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), -np.log(V), atol=TOL_F32)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), np.log(V), atol=TOL_F32)
    assert r.argmax.cpu().tolist() == [0, 0]          # all tied: lowest index
    spike = torch.zeros((1, V), device=dev, dtype=torch.bfloat16)
    spike[0, 777] = 15.0
    r = tome_amd.token_logprobs(spike, torch.tensor([777], device=dev), 1.0, want_argmax=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), -np.log1p((V - 1) * np.exp(-15.0)), atol=TOL_F32)
    assert r.argmax.item() == 777


def test_argmax_ties_lowest_index(dev):
    rng = np.random.default_rng(11)
    V = 40000
    x = rng.standard_normal((6, V)).astype(np.float32)
    spots = [(0, [5, 39999]), (1, [12345, 12346]), (2, [39999, 7]), (3, [8, 9, 10]), (4, [2047, 2048]), (5, [39992, 39993])]
    for r_, idx in spots:
        x[r_, idx] = 9.5
    for dtype in (torch.float32, torch.bfloat16):
        xt = torch.from_numpy(x).to(dev).to(dtype)
        r = tome_amd.token_logprobs(xt, torch.zeros(6, dtype=torch.int32, device=dev), 1.0, want_argmax=True)
        assert r.argmax.cpu().tolist() == [min(i) for _, i in spots]


def test_masked_rows_and_lengths(dev):
    rng = np.random.default_rng(3)
    G, L, V = 4, 33, 5000
    x = torch.from_numpy(rng.standard_normal((G, L, V)).astype(np.float32)).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=(G, L)).astype(np.int32)
    lengths = np.array([33, 1, 0, 17])
    r = tome_amd.token_logprobs(x, torch.from_numpy(t).to(dev), 1.0, lengths=torch.from_numpy(lengths),
                                want_lse=True, want_argmax=True)
    want = oracle.logprob_rows(bf16_bits_of(x), t, 1.0)
    mask = np.arange(L)[None, :] < lengths[:, None]
    got = r.lp.cpu().numpy()
    assert got.shape == (G, L)
    np.testing.assert_allclose(got[mask], want[mask], atol=TOL_F32, rtol=0)
    assert (got[~mask] == 0).all() and (r.lse.cpu().numpy()[~mask] == 0).all()
    assert (r.argmax.cpu().numpy()[~mask] == -1).all()


def test_shift_and_temperature_identities(dev):
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((16, 30000)) * 3).astype(np.float32)
    t = rng.integers(0, 30000, size=16).astype(np.int32)
    tt = torch.from_numpy(t).to(dev)
    a = tome_amd.token_logprobs(torch.from_numpy(x).to(dev), tt, 0.7).lp
    b = tome_amd.token_logprobs(torch.from_numpy(x + 100.0).to(dev), tt, 0.7).lp
    c = tome_amd.token_logprobs(torch.from_numpy((x / np.float32(0.7)).astype(np.float32)).to(dev), tt, 1.0).lp
    np.testing.assert_allclose(a.cpu().numpy(), b.cpu().numpy(), atol=1e-4)
    np.testing.assert_allclose(a.cpu().numpy(), c.cpu().numpy(), atol=1e-4)


def test_out_of_range_target_is_nan(dev):
    x = torch.zeros((3, 64), device=dev)
    r = tome_amd.token_logprobs(x, torch.tensor([-1, 64, 5], device=dev), 1.0)
    got = r.lp.cpu().numpy()
    assert np.isnan(got[0]) and np.isnan(got[1]) and np.isfinite(got[2])


def test_local_compute_logprobs_dropin(dev):
    """Same call shape as node.py:451: [Lc, V] bf16 slice, uint-like ids, temp."""
    rng = np.random.default_rng(21)
    logits = torch.from_numpy((rng.standard_normal((2, 40, V_QWEN3)) * 3).astype(np.float32)).to(dev).to(torch.bfloat16)
    c_toks = rng.integers(0, V_QWEN3, size=12)
    c_logits = logits[1, 6:18]
    lps = tome_amd.local_compute_logprobs(c_logits, torch.tensor(c_toks, device=dev), 0.8)
    assert lps.dtype == torch.float32 and lps.shape == (12,)
    want = oracle.logprob_rows(bf16_bits_of(c_logits), c_toks, 0.8)
    np.testing.assert_allclose(lps.cpu().numpy(), want, atol=TOL_BF16, rtol=0)
    np.testing.assert_allclose(lps.cpu().numpy(), want, atol=TOL_F32, rtol=0)
    ref32 = oracle.local_compute_logprobs_f32(bf16_bits_of(c_logits), c_toks, 0.8)
    np.testing.assert_allclose(lps.cpu().numpy(), ref32, atol=TOL_F32, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,V,T", [(1, V_QWEN3, 1.0), (3, 4096 * 2 + 1, 0.7), (64, 4096, 1.0), (5, 8192 + 384, 2.0),
                                      (1400, 4100, 1.0), (1301, 1030, 0.7), (40, 2051, 1.3)])
def test_fused_log_softmax_full_matrix(dev, dtype, rows, V, T):
    """model.py:77-89 drop-in, incl. the kernel's tail cases (V % 4096 in {0, 1, 384}) and batches of more rows than
    workgroups fit the chip at once, with rows that end in a partial workgroup and in single elements."""
    rng = np.random.default_rng(V + rows)
    x = torch.from_numpy(rng.standard_normal((rows, V)).astype(np.float32)).to(dev).to(dtype)
    out = tome_amd.fused_log_softmax(x, T)
    assert out.shape == x.shape and out.dtype == x.dtype
    if dtype == torch.float32:
        want = oracle.full_log_softmax64(x.cpu().numpy(), T)
        np.testing.assert_allclose(out.cpu().numpy(), want, atol=TOL_F32, rtol=0)
        # probabilities sum to one
        np.testing.assert_allclose(np.exp(out.cpu().numpy().astype(np.float64)).sum(-1), 1.0, atol=1e-4)
    else:
        bits = bf16_bits_of(x)
        want = oracle.fused_log_softmax_f32(bits, T)           # bf16 arithmetic of model.py:57-60
        got = bf16_bits_of(out)
        diff = np.abs(oracle.bf16_to_f32(got) - oracle.bf16_to_f32(want))
        # identical except where the fp32 lse sits within rounding of a bf16 tie
        assert (diff <= 0.0625 + 1e-6).all() and (diff == 0).mean() > 0.99
        # the reference's own check (tests/test_logprob_comparison.py:84-102): against
        # `logits - mx.logsumexp(logits)` evaluated in bf16, max abs diff < 5e-3
        if T == 1.0:
            lse_b = oracle.bf16_to_f32(oracle.bf16_round(oracle.lse_rows(bits, 1.0).astype(np.float32)))
            expected = oracle.bf16_to_f32(oracle.bf16_round(oracle.bf16_to_f32(bits) - lse_b[:, None]))
            assert np.abs(oracle.bf16_to_f32(got) - expected).max() < 5e-3


def test_entry_points_replay_correctly_from_a_hip_graph(dev):
    """Callers that capture their step as a HIP graph: the row kernel (with its split + combine launches) and
    the fused path (compaction, main and combine kernels, device-side schedule) record no memsets and keep
    no state, so replays on changing inputs must equal eager calls on the same inputs."""
    rng = np.random.default_rng(77)
    rows, V, n, H, Vf = 24, 20011, 600, 128, 3001
    x = torch.zeros((rows, V), dtype=torch.float32, device=dev)
    t = torch.zeros(rows, dtype=torch.int32, device=dev)
    h = torch.zeros((n, H), dtype=torch.bfloat16, device=dev)
    w = torch.from_numpy((rng.standard_normal((Vf, H)) * 0.2).astype(np.float32)).to(dev).to(torch.bfloat16)
    tf = torch.zeros(n, dtype=torch.int32, device=dev)
    valid = torch.ones(n, dtype=torch.int32, device=dev)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):                                   # warm-up outside the capture
        tome_amd.token_logprobs(x, t, 0.9, want_argmax=True)
        tome_amd.fused_lmhead_logprobs(h, w, tf, 1.1, row_valid=valid, want_entropy=True)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        r_row = tome_amd.token_logprobs(x, t, 0.9, want_argmax=True)
        r_fused = tome_amd.fused_lmhead_logprobs(h, w, tf, 1.1, row_valid=valid, want_entropy=True)
    for it in range(3):
        x.copy_(torch.from_numpy((rng.standard_normal((rows, V)) * 2).astype(np.float32)))
        t.copy_(torch.from_numpy(rng.integers(0, V, rows).astype(np.int32)))
        h.copy_(torch.from_numpy(rng.standard_normal((n, H)).astype(np.float32)).to(torch.bfloat16))
        tf.copy_(torch.from_numpy(rng.integers(0, Vf, n).astype(np.int32)))
        valid.copy_(torch.from_numpy((rng.random(n) < 0.3 + 0.3 * it).astype(np.int32)))   # the valid count changes per replay
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [r_row.lp.clone(), r_row.argmax.clone(), r_fused.lp.clone(), r_fused.entropy.clone()]
        e_row = tome_amd.token_logprobs(x, t, 0.9, want_argmax=True)
        e_fused = tome_amd.fused_lmhead_logprobs(h, w, tf, 1.1, row_valid=valid, want_entropy=True)
        torch.cuda.synchronize()
        for a, b in zip(got, [e_row.lp, e_row.argmax, e_fused.lp, e_fused.entropy]):
            assert torch.equal(a, b)
        (h.float() @ w.float().T).sum().item()                       # unrelated eager work between replays


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,V,n_index", [(64, 151936, 37), (700, 4097, 700), (4096, 8192, 1500), (9, 50, 30)])
def test_row_list_matches_full_call_and_oracle(dev, dtype, rows, V, n_index):
    """tome_row_logprob_rows (the completion rows of mlx-impl/node.py:449 as a packed list) against the oracle and
    against the plain call on the gathered rows; order, repeats and out-of-range entries of the list are honoured."""
    rng = np.random.default_rng(rows + V + n_index)
    x = torch.from_numpy((rng.standard_normal((rows, V)) * 2.5).astype(np.float32)).to(dev).to(dtype)
    idx = rng.integers(0, rows, size=n_index).astype(np.int32)       # unsorted, with repeats
    idx[: min(rows, n_index)] = rng.permutation(rows)[: min(rows, n_index)]
    t = rng.integers(0, V, size=n_index).astype(np.int32)
    bad = [1, n_index - 1]
    idx_bad = idx.copy()
    idx_bad[bad[0]], idx_bad[bad[1]] = rows, -1                       # not rows of the matrix
    got = tome_amd.token_logprobs_rows(x, torch.from_numpy(idx_bad).to(dev), torch.from_numpy(t).to(dev), 0.9,
                                       want_lse=True, want_entropy=True, want_argmax=True)
    ok = np.ones(n_index, bool)
    ok[bad] = False
    src = x.float().cpu().numpy() if dtype == torch.float32 else bf16_bits_of(x)
    lp, lse, ent, am = (v.cpu().numpy() for v in got)
    assert lp.shape == (n_index,)
    np.testing.assert_allclose(lp[ok], oracle.logprob_rows(src[idx[ok]], t[ok], 0.9), atol=1e-4, rtol=0)
    np.testing.assert_allclose(lse[ok], oracle.lse_rows(src[idx[ok]], 0.9), atol=1e-4, rtol=0)
    np.testing.assert_allclose(ent[ok], oracle.entropy_rows(src[idx[ok]], 0.9), atol=1e-4, rtol=0)
    np.testing.assert_array_equal(am[ok], oracle.argmax_rows(src[idx[ok]]))
    assert np.isnan(lp[bad]).all() and np.isnan(lse[bad]).all() and (am[bad] == -1).all()
    # against the plain entry point on the gathered rows (same number of problems -> same split of a row)
    dense = tome_amd.token_logprobs(x[torch.from_numpy(idx[ok]).to(dev).long()], torch.from_numpy(t[ok]).to(dev), 0.9,
                                    want_lse=True, want_argmax=True)
    np.testing.assert_allclose(lp[ok], dense.lp.cpu().numpy(), atol=2e-6, rtol=0)
    np.testing.assert_array_equal(am[ok], dense.argmax.cpu().numpy())



@pytest.mark.parametrize("rows,V,T", [(300, 20000, 1.0), (7, 151941, 0.7), (100, 155648, 1.0), (2, 155656, 1.3), (100, 16384, 2.0),
                                      (5, 16376, 1.0), (51, 151936, 1.0), (50, 151936, 0.9), (3, 20000, 0.9), (21, 65536, 1.0), (22, 65536, 1.1)])
def test_full_log_softmax_bf16_one_pass_and_its_limits(dev, rows, V, T):
    """bf16 rows of 16384 .. 155648 elements take the one-pass kernel (the row stays in a workgroup's registers) - at any
    batch size up to 40960 elements, from V / 3000 rows on above; smaller batches of long rows, shorter and longer rows,
    and rows that are not 16-byte aligned, take the two passes.  Same bar for all: the bf16 arithmetic of
    mlx-impl/model.py:57-60 as the oracle restates it, identical except where the fp32 lse sits within rounding of a bf16
    tie; ragged V (V % 8 != 0), rows with -inf entries and a NaN row included."""
    rng = np.random.default_rng(rows * 7 + V)
    x32 = (rng.standard_normal((rows, V)) * 2).astype(np.float32)
    x32[0, rng.random(V) < 0.2] = -np.inf                      # a masked vocabulary
    if rows > 2:
        x32[2, V // 3] = np.nan                                # NaN makes the whole row NaN
    x = torch.from_numpy(x32).to(dev).to(torch.bfloat16)
    out = tome_amd.fused_log_softmax(x, T)
    assert out.shape == x.shape and out.dtype == torch.bfloat16
    bits = bf16_bits_of(x)
    ok = np.array([r for r in range(rows) if not (rows > 2 and r == 2)])
    want = oracle.fused_log_softmax_f32(bits[ok], T)
    got = bf16_bits_of(out)
    a, b = oracle.bf16_to_f32(got[ok]), oracle.bf16_to_f32(want)
    fin = np.isfinite(b)
    np.testing.assert_array_equal(np.isneginf(a), np.isneginf(b))    # masked entries stay -inf
    diff = np.abs(a[fin] - b[fin])
    assert (diff <= 0.125 + 1e-6).all() and (diff == 0).mean() > 0.99
    if rows > 2:
        assert np.isnan(oracle.bf16_to_f32(got[2])).all()
    # a strided input and output view give the same bits as the contiguous call
    wide_in = torch.zeros((rows, V + 24), dtype=torch.bfloat16, device=dev)
    wide_in[:, 8:V + 8] = x
    out2 = tome_amd.fused_log_softmax(wide_in[:, 8:V + 8], T)
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16))


@pytest.mark.parametrize("rows,V,pad,T", [(50, 20003, 5, 1.0), (64, 151941, 3, 0.7), (45, 16391, 9, 1.3)])
def test_full_log_softmax_one_pass_with_single_trailing_elements(dev, rows, V, pad, T):
    """Through the C ABI with padded row strides (a multiple of 8 elements, which the tensor wrapper's contiguous output
    never has when V is not): the one-pass kernel then also takes rows whose last V % 8 elements are single elements.
    Same bar as the other bf16 cases; the padding of the output rows stays untouched."""
    from tome_amd import _lib
    lib = tome_amd.load_library()
    rng = np.random.default_rng(rows + V)
    stride = V + pad
    assert stride % 8 == 0
    x32 = (rng.standard_normal((rows, V)) * 2).astype(np.float32)
    x32[1, rng.random(V) < 0.3] = -np.inf
    xin = torch.zeros((rows, stride), dtype=torch.bfloat16, device=dev)
    xin[:, :V] = torch.from_numpy(x32).to(dev).to(torch.bfloat16)
    out = torch.full((rows, stride), 7.0, dtype=torch.bfloat16, device=dev)
    lse = torch.empty(rows, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_row_logprob_workspace(rows, V)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _lib.check(lib.tome_full_log_softmax(xin.data_ptr(), out.data_ptr(), 1, rows, V, stride, stride, T, lse.data_ptr(),
                                         ws.data_ptr(), ws_bytes, torch.cuda.current_stream(dev).cuda_stream))
    torch.cuda.synchronize()
    bits = bf16_bits_of(xin[:, :V].contiguous())
    want = oracle.fused_log_softmax_f32(bits, T)
    got = bf16_bits_of(out[:, :V].contiguous())
    a, b = oracle.bf16_to_f32(got), oracle.bf16_to_f32(want)
    fin = np.isfinite(b)
    np.testing.assert_array_equal(np.isneginf(a), np.isneginf(b))
    diff = np.abs(a[fin] - b[fin])
    assert (diff <= 0.125 + 1e-6).all() and (diff == 0).mean() > 0.99
    assert (diff[-1000:] == 0).mean() > 0.98                                   # the trailing elements among them
    np.testing.assert_allclose(lse.cpu().numpy(), oracle.lse_rows(bits, T), atol=2e-5 * max(1.0, 1.0 / T), rtol=1e-6)
    assert (out[:, V:] == 7.0).all()


def test_full_log_softmax_fp32_above_three_quarters_of_a_gigabyte(dev):
    """fp32 matrices above 3/4 GB: the first pass streams the rows past the caches and the second pass runs workgroups of one
    load per lane.  Too large for the fp64 oracle as a whole: 24 rows spread over the matrix against it at 1e-4, every row's
    probabilities summing to one, and the last elements of the last row (a ragged V) in place."""
    rows, V, T = 1400, V_QWEN3 + 3, 0.9
    g = torch.Generator(device=dev).manual_seed(9)
    x = torch.empty((rows, V), dtype=torch.float32, device=dev)
    for i in range(0, rows, 200):
        x[i:i + 200] = torch.randn((min(200, rows - i), V), device=dev, generator=g) * 2
    out = tome_amd.fused_log_softmax(x, T)
    pick = np.linspace(0, rows - 1, 24).astype(np.int64)
    want = oracle.full_log_softmax64(x[torch.from_numpy(pick).to(dev)].cpu().numpy(), T)
    np.testing.assert_allclose(out[torch.from_numpy(pick).to(dev)].cpu().numpy(), want, atol=TOL_F32, rtol=0)
    total = torch.exp(out.double()).sum(-1)
    assert (total - 1.0).abs().max().item() < 1e-4
    del out, x
    torch.cuda.empty_cache()


def test_full_log_softmax_fp32_split_rows_merge_inside_the_second_pass(dev):
    """fp32 batches of fewer than 512 rows are split over several workgroups in the first pass; the second pass merges
    the partials itself.  Against the fp64 oracle at 1e-4, and the lse it leaves must equal token_logprobs' lse."""
    rng = np.random.default_rng(123)
    for rows, V in ((64, V_QWEN3), (9, 50001), (511, 6000)):
        x = torch.from_numpy((rng.standard_normal((rows, V)) * 2).astype(np.float32)).to(dev)
        out = tome_amd.fused_log_softmax(x, 0.8)
        want = oracle.full_log_softmax64(x.cpu().numpy(), 0.8)
        np.testing.assert_allclose(out.cpu().numpy(), want, atol=TOL_F32, rtol=0)
        lse = tome_amd.token_logprobs(x, torch.zeros(rows, dtype=torch.int32, device=dev), 0.8, want_lse=True).lse
        np.testing.assert_allclose((x[:, 0] / 0.8 - out[:, 0]).cpu().numpy(), lse.cpu().numpy(), atol=2e-5, rtol=0)
