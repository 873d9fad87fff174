"""GPU parity of the fused lm_head + log-softmax kernels against the fp64 oracle.

Oracle = exact (fp64) product of the bf16 inputs followed by the closed-form row statistics;
tolerance 2e-3 abs (bf16 inputs, fp32 accumulation), the bar stated for this path.
"""
import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import V_QWEN3, bf16_bits_of, check_argmax

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.fixture
def force_kernel():
    """tome_select_fused_kernel for one test: 'generic' / 'dma' force that sweep kernel, 'dma_whole_tiles' the LDS-DMA
    kernel with vocab ranges cut at whole 256-row tiles (no short last tile); reset afterwards."""
    lib = tome_amd.load_library()
    yield lambda kind: lib.tome_select_fused_kernel({"generic": 0, "dma": 1, "dma_whole_tiles": 3, "dma_two_w_buffers": 4,
                                                     "dma_three_w_buffers": 5}[kind])
    lib.tome_select_fused_kernel(-1)


def _inputs(dev, n, H, V, seed, h_scale=1.0, w_scale=0.02):
    rng = np.random.default_rng(seed)
    h = torch.from_numpy((rng.standard_normal((n, H)) * h_scale).astype(np.float32)).to(dev).to(torch.bfloat16)
    w = torch.from_numpy((rng.standard_normal((V, H)) * w_scale).astype(np.float32)).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    return h, w, t


@pytest.mark.parametrize("n,H,V,T,w_scale", [
    (1, 8, 16, 1.0, 1.0), (37, 64, 300, 1.0, 0.5), (130, 72, 1000, 0.7, 0.3), (128, 1024, 2048 + 17, 1.0, 0.05),
    (300, 256, 5000, 1.3, 0.1), (5, 200, 256, 1.0, 0.2), (129, 128, 257, 1.0, 0.2), (64, 2560, 4096, 0.7, 0.02),
])
def test_fused_matches_oracle_small(dev, n, H, V, T, w_scale):
    h, w, t = _inputs(dev, n, H, V, seed=n * 7 + V, w_scale=w_scale)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), T, want_lse=True, want_entropy=True)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, T)
    np.testing.assert_allclose(r.lp.cpu().numpy(), want["lp"], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), want["lse"], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), want["entropy"], atol=TOL, rtol=0)
    assert (r.lp.cpu().numpy() <= 1e-5).all()


def test_fused_targets_on_tile_edges(dev):
    """Target ids at the first/last row of vocab tiles, 32-row blocks and the partial last tile."""
    V, H = 256 * 3 + 40, 128
    ids = [0, 1, 3, 4, 7, 8, 31, 32, 127, 128, 255, 256, 257, 511, 512, 767, 768, 769, 800, V - 1]
    n = len(ids)
    h, w, _ = _inputs(dev, n, H, V, seed=99, w_scale=0.3)
    t = np.array(ids, dtype=np.int32)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 1.0)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 1.0)
    np.testing.assert_allclose(r.lp.cpu().numpy(), want["lp"], atol=TOL, rtol=0)


def test_fused_qwen3_06b_shape_sampled_rows(dev):
    """Config 3 shape (H=1024, V=151936): 192 tokens against the oracle."""
    n, H, V = 192, 1024, V_QWEN3
    h, w, t = _inputs(dev, n, H, V, seed=2024)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 1.0, want_lse=True, want_entropy=True)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 1.0)
    np.testing.assert_allclose(r.lp.cpu().numpy(), want["lp"], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), want["lse"], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy(), want["entropy"], atol=TOL, rtol=0)


def test_fused_full_config3_against_row_kernel(dev):
    """All 4096 x 151936 of config 3: fused path vs the row kernel on fp32 logits from a library GEMM.

    Size-independent cross-check (the two paths share no code besides the reduction algebra); the
    oracle pins a sample of the same rows.
    """
    n, H, V = 4096, 1024, V_QWEN3
    g = torch.Generator(device=dev).manual_seed(7)
    h = torch.randn((n, H), device=dev, generator=g).to(torch.bfloat16)
    w = (torch.randn((V, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (n,), device=dev, generator=g, dtype=torch.int64)
    r = tome_amd.fused_lmhead_logprobs(h, w, t, 1.0, want_lse=True)
    logits = h.float() @ w.float().t()
    ref = tome_amd.token_logprobs(logits, t, 1.0, want_lse=True)
    np.testing.assert_allclose(r.lp.cpu().numpy(), ref.lp.cpu().numpy(), atol=TOL, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), ref.lse.cpu().numpy(), atol=TOL, rtol=0)
    rows = np.arange(0, n, 64)
    want = oracle.lmhead_stats(bf16_bits_of(h[rows]), bf16_bits_of(w), t.cpu().numpy()[rows], 1.0)
    np.testing.assert_allclose(r.lp.cpu().numpy()[rows], want["lp"], atol=TOL, rtol=0)


def test_fused_varlen_mask_temperature(dev):
    """Config 4 flavour: [B, L, H] hidden, lengths mask, T = 0.7."""
    B, L, H, V = 5, 70, 320, 3000
    rng = np.random.default_rng(17)
    h = torch.from_numpy(rng.standard_normal((B, L, H)).astype(np.float32)).to(dev).to(torch.bfloat16)
    w = torch.from_numpy((rng.standard_normal((V, H)) * 0.1).astype(np.float32)).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=(B, L)).astype(np.int32)
    lengths = np.array([70, 0, 13, 64, 1])
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.7, lengths=torch.from_numpy(lengths),
                                       want_entropy=True)
    want = oracle.lmhead_stats(bf16_bits_of(h).reshape(B * L, H), bf16_bits_of(w), t.reshape(-1), 0.7)
    mask = (np.arange(L)[None, :] < lengths[:, None])
    got = r.lp.cpu().numpy()
    assert got.shape == (B, L)
    np.testing.assert_allclose(got[mask], want["lp"].reshape(B, L)[mask], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[mask], want["entropy"].reshape(B, L)[mask], atol=TOL, rtol=0)
    assert (got[~mask] == 0).all() and (r.entropy.cpu().numpy()[~mask] == 0).all()
    none = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.7, lengths=torch.zeros(B, dtype=torch.int64))
    assert (none.lp.cpu().numpy() == 0).all()


def test_grpo_dual_matches_oracle(dev):
    """Config 5 flavour: ref = policy + small perturbation; lp, ref_lp, k3, entropy."""
    n, H, V = 200, 512, 6000
    rng = np.random.default_rng(5)
    h = torch.from_numpy(rng.standard_normal((n, H)).astype(np.float32)).to(dev).to(torch.bfloat16)
    wp32 = (rng.standard_normal((V, H)) * 0.05).astype(np.float32)
    wp = torch.from_numpy(wp32).to(dev).to(torch.bfloat16)
    wr = torch.from_numpy(wp32 + (rng.standard_normal((V, H)) * 0.005).astype(np.float32)).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    valid = (rng.random(n) < 0.8).astype(np.int32)
    r = tome_amd.grpo_dual_logprobs(h, wp, wr, torch.from_numpy(t).to(dev), 0.9, row_valid=torch.from_numpy(valid).to(dev))
    pol = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(wp), t, 0.9)
    ref = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(wr), t, 0.9)
    m = valid.astype(bool)
    np.testing.assert_allclose(r.lp.cpu().numpy()[m], pol["lp"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.ref_lp.cpu().numpy()[m], ref["lp"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[m], pol["entropy"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.k3.cpu().numpy()[m], oracle.k3(pol["lp"], ref["lp"])[m], atol=2 * TOL, rtol=0)
    assert (r.k3.cpu().numpy() >= -1e-6).all()
    for o in r:
        assert (o.cpu().numpy()[~m] == 0).all()
    same = tome_amd.grpo_dual_logprobs(h, wp, wp, torch.from_numpy(t).to(dev), 0.9)
    assert np.abs(same.k3.cpu().numpy()).max() == 0.0
    np.testing.assert_array_equal(same.lp.cpu().numpy(), same.ref_lp.cpu().numpy())


def test_fused_rejects_bad_inputs(dev):
    h = torch.zeros((4, 64), device=dev, dtype=torch.bfloat16)
    w = torch.zeros((100, 64), device=dev, dtype=torch.bfloat16)
    t = torch.zeros(4, dtype=torch.int32, device=dev)
    with pytest.raises(TypeError):
        tome_amd.fused_lmhead_logprobs(h.float(), w, t)
    with pytest.raises(ValueError):
        tome_amd.fused_lmhead_logprobs(h, w[:, :32], t)
    with pytest.raises(ValueError):
        tome_amd.fused_lmhead_logprobs(h, w, t, 0.0)
    with pytest.raises(ValueError):
        tome_amd.fused_lmhead_logprobs(h[:, :60], w[:, :60].contiguous(), t)   # H % 8 != 0


@pytest.mark.parametrize("n,H,V", [(200, 256, 5000), (70, 72, 1000), (300, 1024, 20000)])
def test_fused_argmax(dev, n, H, V):
    """Greedy id on every row: the first maximum of the fp32 logits the sweep computed (check_argmax)."""
    h, w, t = _inputs(dev, n, H, V, seed=V + n, w_scale=0.1)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 1.0, want_argmax=True)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 1.0)
    check_argmax(h, w, r.argmax.cpu().numpy(), want)


def test_fused_argmax_spike_and_ties(dev):
    n, H, V = 160, 128, 3000
    rng = np.random.default_rng(12)
    h = torch.from_numpy(rng.standard_normal((n, H)).astype(np.float32)).to(dev).to(torch.bfloat16)
    w32 = (rng.standard_normal((V, H)) * 0.05).astype(np.float32)
    # rows 100, 1500 and 2999 are identical and aligned with every token: a three-way exact tie at the top
    w32[[100, 1500, 2999]] = 0.0
    wt = torch.from_numpy(w32).to(dev).to(torch.bfloat16)
    hb = h.float()
    big = (hb / hb.norm(dim=-1, keepdim=True)).mean(0)
    wt[[100, 1500, 2999]] = (big * 50).to(torch.bfloat16)
    t = torch.zeros(n, dtype=torch.int32, device=dev)
    r = tome_amd.fused_lmhead_logprobs(h, wt, t, 1.0, want_argmax=True)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(wt), np.zeros(n, np.int32), 1.0)
    tied = want["argmax"] == 100
    assert tied.sum() > 0
    got = r.argmax.cpu().numpy()
    assert (got[tied] == 100).all()                  # first of the tied rows, in different vocab tiles
    check_argmax(h, wt, got, want, min_clear=0.0)     # the planted rows are large: few gaps exceed the bound
    masked = tome_amd.fused_lmhead_logprobs(h, wt, t, 1.0, want_argmax=True, row_valid=torch.zeros(n, dtype=torch.int32, device=dev))
    assert (masked.argmax.cpu().numpy() == -1).all()


@pytest.mark.parametrize("kind", ["generic", "dma", "dma_whole_tiles"])
def test_fused_every_kernel_path(dev, kind, force_kernel):
    """The two GEMM kernels behind tome_fused_lmhead_logprob (generic / LDS-DMA) are picked
    by shape; tome_select_fused_kernel forces each of them onto the same problem."""
    force_kernel(kind)
    n, H, V = 700, 256, 9000          # 3 token tiles of 256 (one ragged), partial last vocab tile, H % 128 == 0
    h, w, t = _inputs(dev, n, H, V, seed=31, w_scale=0.1)
    valid = (np.random.default_rng(1).random(n) < 0.7).astype(np.int32)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.8, want_lse=True, want_entropy=True,
                                       want_argmax=True, row_valid=torch.from_numpy(valid).to(dev))
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 0.8)
    m = valid.astype(bool)
    np.testing.assert_allclose(r.lp.cpu().numpy()[m], want["lp"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy()[m], want["lse"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[m], want["entropy"][m], atol=TOL, rtol=0)
    check_argmax(h, w, r.argmax.cpu().numpy(), want, 0.8, rows=np.flatnonzero(m))
    assert (r.lp.cpu().numpy()[~m] == 0).all() and (r.argmax.cpu().numpy()[~m] == -1).all()


def _dma_tail_heights(n, V):
    """The short-tile heights (16-row blocks per wave, 0 = none) the LDS-DMA kernel meets on this shape: a host-side
    restatement of how it deals the vocab axis - 32-row units, `splits` contiguous ranges, whole 256-row tiles first.
    Valid where all workgroups run in one round (token tiles * 8 <= 256), which is every shape this is used on."""
    bt = 256 if n > 128 else (128 if n > 64 else 64)
    tt = -(-n // bt)
    assert tt * 8 <= 256
    units, tiles = -(-V // 32), -(-V // 256)
    splits = max(1, min(256 // tt, tiles))
    return {((s + 1) * units // splits - s * units // splits) % 8 for s in range(splits)}


# vocabulary sizes whose ranges end in short tiles of every height, for 256-, 128- and 64-token tiles (n > 128, > 64, <= 64):
# with fewer splits than tiles a range is (units / splits) 32-row units long, i.e. a tail of that modulo 8
TAIL_SHAPES = [(1000, 64, 18432), (1000, 128, 21504), (600, 64, 33920), (1000, 64, 28992), (100, 64, 77824), (100, 128, 93312),
               (50, 64, 108096), (50, 192, 32 * (256 * 9 + 10) + 5), (256, 1024, 20000), (200, 64, 223), (1000, 256, 4481)]


def test_tail_shapes_cover_every_short_tile_height():
    seen = {256: set(), 128: set(), 64: set()}
    for n, _, V in TAIL_SHAPES:
        seen[256 if n > 128 else (128 if n > 64 else 64)] |= _dma_tail_heights(n, V)
    assert seen[256] >= set(range(8)) and seen[128] >= {1, 2, 3, 4} and seen[64] >= {1, 2, 5, 6}


@pytest.mark.parametrize("n,H,V", TAIL_SHAPES)
def test_fused_tile_heights_agree(dev, n, H, V, force_kernel):
    """The LDS-DMA kernel deals the vocab axis in 32-row units: a workgroup's range is whole 256-row tiles plus at most
    one short tile of 1 .. 7 sixteen-row blocks per wave.  Every height (the shapes above cover 0 .. 7 on 64-, 128- and
    256-token tiles) against the oracle, targets on the first and last rows of tiles, units and blocks; and the same
    problem with ranges of whole tiles only must name the same argmax."""
    h, w, t = _inputs(dev, n, H, V, seed=n + V, w_scale=0.1)
    edges = [v for v in (0, 15, 16, 31, 32, 111, 112, 127, 128, 223, 224, 255, 256, 447, 448, V - 33, V - 32, V - 1) if 0 <= v < V]
    t[: len(edges)] = edges[: n]
    valid = np.ones(n, dtype=np.int32)
    valid[n // 3] = 0
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 0.9)
    got = {}
    for kind in ("dma", "dma_whole_tiles"):
        force_kernel(kind)
        r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.9, want_lse=True, want_entropy=True,
                                           want_argmax=True, row_valid=torch.from_numpy(valid).to(dev))
        m = valid.astype(bool)
        np.testing.assert_allclose(r.lp.cpu().numpy()[m], want["lp"][m], atol=TOL, rtol=0)
        np.testing.assert_allclose(r.lse.cpu().numpy()[m], want["lse"][m], atol=TOL, rtol=0)
        np.testing.assert_allclose(r.entropy.cpu().numpy()[m], want["entropy"][m], atol=TOL, rtol=0)
        check_argmax(h, w, r.argmax.cpu().numpy(), want, 0.9, rows=np.flatnonzero(m), min_clear=0.0)
        assert r.lp.cpu().numpy()[n // 3] == 0 and r.argmax.cpu().numpy()[n // 3] == -1
        got[kind] = r.argmax.cpu().numpy()
    np.testing.assert_array_equal(got["dma"], got["dma_whole_tiles"])


@pytest.mark.parametrize("n,H,V,outputs", [
    (200, 256, 30000, "all"),       # one token tile, 224-row tiles
    (200, 64, 3000, "plain"),       # a single K slab per vocab tile: the ring wraps at every tile
    (700, 192, 12000, "all"),       # three token tiles, several vocab tiles per workgroup
    (700, 192, 12000, "plain"),
    (256, 1024, 20000, "entropy"),
    (1500, 128, 256 * 9 + 77, "argmax"),
])
def test_fused_w_ring_depths_agree(dev, n, H, V, outputs, force_kernel):
    """The 256-token tile of the LDS-DMA kernel exists with two and with three W buffers (the shape picks one): the
    request schedule differs, the arithmetic does not, so both must match the oracle and each other bit for bit."""
    h, w, t = _inputs(dev, n, H, V, seed=n + H, w_scale=0.1)
    t[:4] = [0, V - 1, V // 2, 255]
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 1.1)
    ent, am = outputs in ("all", "entropy"), outputs in ("all", "argmax")
    got = {}
    for kind in ("dma_two_w_buffers", "dma_three_w_buffers"):
        force_kernel(kind)
        r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 1.1, want_lse=True, want_entropy=ent, want_argmax=am)
        np.testing.assert_allclose(r.lp.cpu().numpy(), want["lp"], atol=TOL, rtol=0)
        np.testing.assert_allclose(r.lse.cpu().numpy(), want["lse"], atol=TOL, rtol=0)
        if ent:
            np.testing.assert_allclose(r.entropy.cpu().numpy(), want["entropy"], atol=TOL, rtol=0)
        if am:
            check_argmax(h, w, r.argmax.cpu().numpy(), want, 1.1, min_clear=0.0)
        got[kind] = r
    a, b = got["dma_two_w_buffers"], got["dma_three_w_buffers"]
    assert torch.equal(a.lp, b.lp) and torch.equal(a.lse, b.lse)
    if ent:
        assert torch.equal(a.entropy, b.entropy)
    if am:
        assert torch.equal(a.argmax, b.argmax)


@pytest.mark.parametrize("kind", ["generic", "dma", "dma_whole_tiles"])
@pytest.mark.parametrize("n,frac_valid", [(300, 1.0), (2304, 1.0), (9000, 1.0), (9000, 0.45), (20000, 0.8)])
def test_fused_every_partial_is_written(dev, kind, n, frac_valid, force_kernel):
    """The work decomposition (token tiles x vocab splits, one or several rounds of workgroups, chosen on
    the device when a mask is given) must cover every (token, split) exactly: the workspace is poisoned
    with NaN bit patterns before the call, so a partial that no workgroup wrote shows up in the output."""
    force_kernel(kind)
    H, V = 64, 256 * 40 + 3
    lib = tome_amd.load_library()
    h, w, t = _inputs(dev, n, H, V, seed=n, w_scale=0.2)
    rng = np.random.default_rng(n + 1)
    valid = (rng.random(n) < frac_valid).astype(np.int32)
    tt = torch.from_numpy(t).to(dev)
    vv = torch.from_numpy(valid).to(dev) if frac_valid < 1.0 else None
    lp = torch.empty(n, dtype=torch.float32, device=dev)
    lse = torch.empty(n, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_fused_lmhead_logprob_workspace(n, H, V)
    ws = torch.full((ws_bytes,), 0xFF, dtype=torch.uint8, device=dev)
    rc = lib.tome_fused_lmhead_logprob(h.data_ptr(), w.data_ptr(), n, H, V, H, H, tt.data_ptr(),
                                       vv.data_ptr() if vv is not None else None, 1.0, lp.data_ptr(), lse.data_ptr(),
                                       None, None, ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    m = valid.astype(bool)
    got_lp, got_lse = lp.cpu().numpy(), lse.cpu().numpy()
    assert np.isfinite(got_lp).all() and np.isfinite(got_lse[m]).all()
    idx = np.flatnonzero(m)[:: max(1, int(m.sum()) // 64)]            # a sample of rows against the oracle
    want = oracle.lmhead_stats(bf16_bits_of(h)[idx], bf16_bits_of(w), t[idx], 1.0)
    np.testing.assert_allclose(got_lp[idx], want["lp"], atol=TOL, rtol=0)
    np.testing.assert_allclose(got_lse[idx], want["lse"], atol=TOL, rtol=0)
    # the exact row sums agree with a plain fp32 matmul everywhere (every token tile and split took part)
    ref = torch.logsumexp(h.float() @ w.float().T, dim=-1).cpu().numpy()
    np.testing.assert_allclose(got_lse[m], ref[m], atol=TOL, rtol=0)
    assert (got_lp[~m] == 0).all()


@pytest.mark.parametrize("n,H,V,masked", [(40, 64, 700, False), (300, 256, 3000, True), (1500, 1024, 5000, True)])
def test_norm_lmhead_matches_oracle(dev, n, H, V, masked):
    """Final RMSNorm folded in front of the lm_head (mlx-impl/model.py:536-538): rows are normalised as the
    oracle's bf16 restatement does, then scored; masked rows are neither normalised nor multiplied."""
    rng = np.random.default_rng(n + H)
    h, w, t = _inputs(dev, n, H, V, seed=n + 1, h_scale=4.0, w_scale=0.2)
    h = (h.float() * torch.linspace(0.2, 3.0, n, device=dev)[:, None]).to(torch.bfloat16)   # rows of very different norms
    gamma = torch.from_numpy((1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32)).to(dev).to(torch.bfloat16)
    valid = (rng.random(n) < 0.6).astype(np.int32) if masked else np.ones(n, np.int32)
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.9, want_lse=True, want_entropy=True, want_argmax=True,
                                       row_valid=torch.from_numpy(valid).to(dev) if masked else None,
                                       norm_weight=gamma, norm_eps=1e-6)
    normed = oracle.rms_norm_bf16(bf16_bits_of(h), bf16_bits_of(gamma), 1e-6)
    want = oracle.lmhead_stats(normed, bf16_bits_of(w), t, 0.9)
    m = valid.astype(bool)
    # 2e-3 of the fused path + rare one-ulp flips of a normalised value (fp32 statistics summed in another order)
    np.testing.assert_allclose(r.lp.cpu().numpy()[m], want["lp"][m], atol=4e-3, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy()[m], want["lse"][m], atol=4e-3, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[m], want["entropy"][m], atol=4e-3, rtol=0)
    clear = m & ((want["top1"] - want["top2"]) > 1e-2)
    np.testing.assert_array_equal(r.argmax.cpu().numpy()[clear], want["argmax"][clear])
    assert (r.lp.cpu().numpy()[~m] == 0).all()
    # the norm must really have been applied: without it the answer is far away
    raw = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.9).lp.cpu().numpy()
    assert np.abs(raw[m] - want["lp"][m]).max() > 0.1


@pytest.mark.parametrize("n,H,V,masked", [
    (1, 1024, 151936, False), (16, 1024, 40000, True), (17, 1024, 8191, False), (64, 1024, 151936, True),
    (33, 2048, 30001, False), (64, 2048, 12345, True), (9, 4096, 20000, False), (32, 4096, 33000, True),
    (20, 2560, 9000, False), (5, 512, 7000, False), (64, 1536, 5000, False), (48, 1024, 70, False),
    (65, 1024, 5001, False), (100, 1024, 30000, True), (128, 1024, 151936, False), (128, 1024, 200, True)])
def test_fused_small_batch_kernel(dev, n, H, V, masked):
    """Decode-sized batches (<= 64 tokens; <= 16 at H = 1024) take the streaming kernel with K split across waves
    (where the shape rules allow it; the other shapes here go to the tiled kernel's 64- and 128-token tiles, which
    request W non-temporally) - same bar either way."""
    rng = np.random.default_rng(n * 31 + H + V)
    h, w, t = _inputs(dev, n, H, V, n * 31 + H + V, w_scale=0.05)
    valid = (rng.random(n) < 0.7).astype(np.int32) if masked else np.ones(n, dtype=np.int32)
    if masked:
        valid[rng.integers(0, n)] = 1
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.8, want_lse=True, want_entropy=True,
                                       want_argmax=True, row_valid=torch.from_numpy(valid).to(dev) if masked else None)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 0.8)
    m = valid.astype(bool)
    np.testing.assert_allclose(r.lp.cpu().numpy()[m], want["lp"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy()[m], want["lse"][m], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[m], want["entropy"][m], atol=TOL, rtol=0)
    check_argmax(h, w, r.argmax.cpu().numpy(), want, 0.8, rows=np.flatnonzero(m))
    assert (r.lp.cpu().numpy()[~m] == 0).all() and (r.argmax.cpu().numpy()[~m] == -1).all()
    plain = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 0.8)     # the variant without extras
    np.testing.assert_allclose(plain.lp.cpu().numpy(), want["lp"], atol=TOL, rtol=0)


@pytest.mark.parametrize("n,H", [(10, 1024), (100, 1024), (50, 4096), (100, 2560), (300, 1024), (40, 72)])
def test_fused_all_masked_and_single_valid_row(dev, n, H):
    """Every sweep kernel (streaming with 1 / 2 token blocks, DMA with 64- / 128- / 256-token tiles, generic) with
    no valid row at all - nothing may be read, every output is the masked value - and with exactly one."""
    V = 5000
    h, w, t = _inputs(dev, n, H, V, n + H, w_scale=0.05)
    tt = torch.from_numpy(t).to(dev)
    none = torch.zeros(n, dtype=torch.int32, device=dev)
    r = tome_amd.fused_lmhead_logprobs(h, w, tt, 1.0, row_valid=none, want_entropy=True, want_argmax=True, want_lse=True)
    assert (r.lp == 0).all() and (r.lse == 0).all() and (r.entropy == 0).all() and (r.argmax == -1).all()
    one = none.clone()
    one[n // 2] = 1
    r = tome_amd.fused_lmhead_logprobs(h, w, tt, 1.0, row_valid=one)
    want = oracle.lmhead_stats(bf16_bits_of(h[n // 2:n // 2 + 1]), bf16_bits_of(w), t[n // 2:n // 2 + 1], 1.0)
    assert abs(r.lp[n // 2].item() - want["lp"][0]) < TOL and (r.lp[one == 0] == 0).all()
    d = tome_amd.grpo_dual_logprobs(h, w, w, tt, 1.0, row_valid=one)
    assert d.k3[n // 2].item() == 0.0 and (d.k3[one == 0] == 0).all()


@pytest.mark.parametrize("which,kind,n", [("weight", "dma", 200), ("weight", "dma", 100), ("weight", "small", 32),
                                          ("hidden", "dma", 300)])
def test_fused_matrices_of_4_gib_and_more(dev, which, kind, n):
    """The LDS-DMA and streaming kernels address both matrices with 64-bit offsets, so a weight (or hidden-state)
    matrix whose extent V * weight_stride * 2 (n * hidden_stride * 2) reaches 2^32 bytes is accepted; only the
    generic kernel refuses it.  A padded row stride makes the extent 4.3 GB while 512 columns are used.  Targets
    and a planted maximum sit in the LAST rows, which lie beyond the 4 GiB mark."""
    H, V = 512, 40000
    lib = tome_amd.load_library()
    rng = np.random.default_rng(n)
    stride = 53760 if which == "weight" else 512                      # 40000 * 53760 * 2 = 4.30e9 >= 2^32
    hstride = 512 if which == "weight" else 7158336                   # 300 * 7158336 * 2 = 4.29e9 >= 2^32
    assert (V * stride * 2 >= 1 << 32) != (n * hstride * 2 >= 1 << 32)
    w_store = torch.empty((V, stride), dtype=torch.bfloat16, device=dev)
    w = w_store[:, :H]
    w.copy_(torch.from_numpy((rng.standard_normal((V, H)) * 0.05).astype(np.float32)).to(dev))
    h_store = torch.empty((n, hstride), dtype=torch.bfloat16, device=dev)
    h = h_store[:, :H]
    h.copy_(torch.from_numpy(rng.standard_normal((n, H)).astype(np.float32)).to(dev))
    t = rng.integers(V - 300, V, size=n).astype(np.int32)            # rows past the 4 GiB mark of the weight matrix
    w[V - 3] = 0.5 * torch.sign(h[n - 1].float()).to(torch.bfloat16)  # token n-1 (past the mark of the hidden matrix): row V-3 wins
    lib.tome_select_fused_kernel({"dma": 1, "small": -1}[kind])
    try:
        r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 1.0, want_lse=True, want_argmax=True)
        torch.cuda.synchronize()
        lib.tome_select_fused_kernel(0)                              # the generic kernel keeps refusing the shape
        with pytest.raises(ValueError):
            tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), 1.0)
    finally:
        lib.tome_select_fused_kernel(-1)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 1.0)
    np.testing.assert_allclose(r.lp.cpu().numpy(), want["lp"], atol=TOL, rtol=0)
    np.testing.assert_allclose(r.lse.cpu().numpy(), want["lse"], atol=TOL, rtol=0)
    assert r.argmax.cpu().numpy()[n - 1] == V - 3 == want["argmax"][n - 1]
    check_argmax(h, w, r.argmax.cpu().numpy(), want)
