"""GPU parity at the edges of the reference's domain, row and fused kernels against the fp64 oracle.

Cases: rows with -inf entries (a masked vocabulary) including a -inf target, rows of -inf only, rows whose
finite entries all sit below the -1e30 floor that the reference's kernel shares (mlx-impl/model.py:28), NaN
entries (NaN propagates, as through mx.logsumexp at mlx-impl/node.py:402), extreme temperatures on logits of
magnitude 30, hidden rows of zeros and a dominant weight row for the fused kernels.  Every case runs as a split
launch (few rows) and as an unsplit one (>= 512 rows) of the row kernel, and on all three fused sweep kernels.

Where a result is fixed by the contract rather than by the mathematics (rows below the floor, all -inf rows,
argmax with NaN present) the test states the contract of include/tome_logprob.h and checks exactly that.
"""
import numpy as np
import pytest
import torch

import oracle
import tome_amd
from conftest import V_QWEN3, bf16_bits_of

pytestmark = pytest.mark.gpu

# (rows, V): fewer than 512 rows are split over several workgroups with a combine launch; 520 are not.
ROW_SHAPES = [(5, 40000), (3, V_QWEN3), (520, 4104)]
DTYPES = [torch.float32, torch.bfloat16]


def _run(x, t, T=1.0):
    r = tome_amd.token_logprobs(x, torch.from_numpy(t).to(x.device), T, want_lse=True, want_entropy=True, want_argmax=True)
    torch.cuda.synchronize()
    src = bf16_bits_of(x) if x.dtype == torch.bfloat16 else x.cpu().numpy()
    return (v.cpu().numpy() for v in r), src


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,V", ROW_SHAPES)
def test_row_masked_vocabulary(dev, dtype, rows, V):
    """-inf entries: they carry no probability; a -inf target scores -inf; argmax is the first maximum of the rest."""
    rng = np.random.default_rng(rows + V)
    x = (rng.standard_normal((rows, V)) * 3).astype(np.float32)
    x[rng.random((rows, V)) < 0.3] = -np.inf
    t = rng.integers(0, V, size=rows).astype(np.int32)
    x[0, t[0]] = -np.inf                                    # a masked target
    x[1, t[1]] = 4.0                                        # a kept one
    x[2, : V - 3] = -np.inf                                 # nearly everything masked
    x[2, V - 3:] = [0.5, 2.0, 1.0]
    xt = torch.from_numpy(x).to(dev).to(dtype)
    (lp, lse, ent, am), src = _run(xt, t, 0.9)
    want_lp = oracle.logprob_rows(src, t, 0.9)
    assert lp[0] == -np.inf and want_lp[0] == -np.inf
    fin = np.isfinite(want_lp)
    np.testing.assert_array_equal(np.isneginf(lp), np.isneginf(want_lp))
    np.testing.assert_allclose(lp[fin], want_lp[fin], atol=1e-4, rtol=0)
    np.testing.assert_allclose(lse, oracle.lse_rows(src, 0.9), atol=1e-4, rtol=0)
    np.testing.assert_allclose(ent, oracle.entropy_rows(src, 0.9), atol=1e-4, rtol=0)
    np.testing.assert_array_equal(am, oracle.argmax_rows(src))
    assert am[2] == V - 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,V", ROW_SHAPES)
def test_row_outside_the_floor(dev, dtype, rows, V):
    """Rows of -inf only, and rows whose entries all lie below -1e30.  The running maximum starts at -1e30, as in
    the reference's kernel (mlx-impl/model.py:28), so such rows are outside the domain; the contract is:
    lse = -inf, argmax 0, and lp = NaN when the target logit is -inf, +inf when it is finite (below the floor)."""
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((rows, V)) * 2).astype(np.float32)
    x[0, :] = -np.inf
    x[1, :] = -2e30
    x[1, 5] = -1.5e30
    x[2, :] = -3e30                                         # mixed: one entry above the floor makes the row ordinary
    x[2, 11] = -7.0
    t = rng.integers(0, V, size=rows).astype(np.int32)
    t[2] = 11
    xt = torch.from_numpy(x).to(dev).to(dtype)
    (lp, lse, ent, am), src = _run(xt, t)
    assert lse[0] == -np.inf and np.isnan(lp[0]) and am[0] == 0
    assert lse[1] == -np.inf and lp[1] == np.inf and am[1] == 0
    np.testing.assert_allclose(lp[2], 0.0, atol=1e-6)       # the one ordinary entry holds all the mass
    np.testing.assert_allclose(lse[2], -7.0, atol=1e-5)
    np.testing.assert_allclose(ent[2], 0.0, atol=1e-5)
    assert am[2] == 11
    rest = np.arange(3, rows)
    np.testing.assert_allclose(lp[rest], oracle.logprob_rows(src[rest], t[rest], 1.0), atol=1e-4, rtol=0)
    np.testing.assert_array_equal(am[rest], oracle.argmax_rows(src[rest]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,V", ROW_SHAPES)
def test_row_nan_propagates(dev, dtype, rows, V):
    """A NaN logit makes the row's lse, lp and entropy NaN (mx.logsumexp does the same); the other rows are
    untouched.  Contract for the argmax: NaN is never the maximum (MLX's own rule is not pinned)."""
    rng = np.random.default_rng(3 * rows + V)
    x = (rng.standard_normal((rows, V)) * 2).astype(np.float32)
    t = rng.integers(0, V, size=rows).astype(np.int32)
    x[0, V // 2] = np.nan
    x[1, 0] = np.nan
    x[1, V - 1] = np.nan
    x[2, t[2]] = np.nan                                     # the target itself
    xt = torch.from_numpy(x).to(dev).to(dtype)
    (lp, lse, ent, am), src = _run(xt, t)
    assert np.isnan(lp[:3]).all() and np.isnan(lse[:3]).all() and np.isnan(ent[:3]).all()
    x64 = oracle.to_f64(src)
    np.testing.assert_array_equal(am[:3], np.nanargmax(x64[:3], axis=-1))
    with np.errstate(invalid="ignore"):
        assert np.isnan(oracle.lse_rows(src[:3])).all()      # the oracle agrees that these rows are NaN
    rest = np.arange(3, rows)
    np.testing.assert_allclose(lp[rest], oracle.logprob_rows(src[rest], t[rest], 1.0), atol=1e-4, rtol=0)
    np.testing.assert_allclose(lse[rest], oracle.lse_rows(src[rest], 1.0), atol=1e-4, rtol=0)
    np.testing.assert_array_equal(am[rest], oracle.argmax_rows(src[rest]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [0.01, 0.05, 50.0])
@pytest.mark.parametrize("rows,V", ROW_SHAPES)
def test_row_extreme_temperature(dev, dtype, T, rows, V):
    """Logits of magnitude 30 at T = 0.01 .. 50: |x| / T reaches 3000.  The shift by the row maximum cancels in
    lse and lp; what is left is fp32 rounding at the magnitude of the result, which the reference's fp32 path
    (mlx-impl/node.py:401-404) carries too: |lp| reaches 60 / T = 6000, where one fp32 ulp is 4.9e-4.
    Tolerance: 1e-4 + 2 ulp_f32(60 / T)."""
    rng = np.random.default_rng(int(T * 100) + rows)
    x = (rng.uniform(-30, 30, size=(rows, V))).astype(np.float32)
    t = rng.integers(0, V, size=rows).astype(np.int32)
    xt = torch.from_numpy(x).to(dev).to(dtype)
    (lp, lse, ent, am), src = _run(xt, t, T)
    tol = 1e-4 + 2 * float(np.spacing(np.float32(60.0 / T)))
    np.testing.assert_allclose(lp, oracle.logprob_rows(src, t, T), atol=tol, rtol=0)
    np.testing.assert_allclose(lse, oracle.lse_rows(src, T), atol=tol, rtol=0)
    np.testing.assert_allclose(ent, oracle.entropy_rows(src, T), atol=tol, rtol=0)
    np.testing.assert_array_equal(am, oracle.argmax_rows(src))
    assert np.isfinite(lp).all() and (lp <= tol).all()


# ---- fused kernels ------------------------------------------------------------------------------------
# (kernel, n, H, V): the streaming kernel takes <= 64 tokens with H % 256 == 0, the LDS-DMA kernel H % 64 == 0
# (forced for the batch sizes used here as well: 100 and 300 tokens run its 128-token tile, 200 tokens one 256-token tile on
# three W buffers, 1100 tokens five 256-token tiles on two - with the entropy asked for), the generic kernel everything else.
FUSED = [("small", 48, 1024, 3000), ("dma", 300, 256, 3000), ("dma", 100, 256, 3000), ("dma", 200, 256, 3000),
         ("dma", 1100, 128, 3000), ("generic", 150, 72, 3000)]


@pytest.fixture
def select_kernel():
    lib = tome_amd.load_library()
    yield lambda kind: lib.tome_select_fused_kernel({"small": -1, "generic": 0, "dma": 1}[kind])
    lib.tome_select_fused_kernel(-1)


def _fused(dev, h, w, t, T=1.0):
    r = tome_amd.fused_lmhead_logprobs(h, w, torch.from_numpy(t).to(dev), T, want_lse=True, want_entropy=True, want_argmax=True)
    torch.cuda.synchronize()
    return tuple(v.cpu().numpy() for v in r)


@pytest.mark.parametrize("kind,n,H,V", FUSED)
def test_fused_zero_rows_and_dominant_weight_row(dev, select_kernel, kind, n, H, V):
    """Hidden rows of zeros make all logits equal: lp = -ln V, entropy ln V, argmax 0 (first of the tied maxima).
    One weight row of +8 makes that id's logit 8 * sum(h), far above or below the rest."""
    select_kernel(kind)
    rng = np.random.default_rng(n + H)
    h32 = rng.standard_normal((n, H)).astype(np.float32)
    h32[0] = 0.0
    h32[n - 1] = 0.0
    w32 = (rng.standard_normal((V, H)) * 0.05).astype(np.float32)
    big = V - 7
    w32[big] = 8.0
    h = torch.from_numpy(h32).to(dev).to(torch.bfloat16)
    w = torch.from_numpy(w32).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    t[1] = big
    lp, lse, ent, am = _fused(dev, h, w, t)
    for r in (0, n - 1):
        np.testing.assert_allclose(lp[r], -np.log(V), atol=1e-5)
        np.testing.assert_allclose(ent[r], np.log(V), atol=1e-5)
        assert am[r] == 0
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, 1.0)
    # fp32 accumulation of a logit of magnitude 8 * |sum h|: H * 2^-24 * max|h| * max|w| on top of the path's 2e-3
    tol = 2e-3 + H * 2.0 ** -24 * float(np.abs(h32).max()) * 8.0
    np.testing.assert_allclose(lp, want["lp"], atol=tol, rtol=0)
    np.testing.assert_allclose(lse, want["lse"], atol=tol, rtol=0)
    np.testing.assert_allclose(ent, want["entropy"], atol=tol, rtol=0)
    s = oracle.to_f64(bf16_bits_of(h)).sum(axis=1)
    up = np.flatnonzero(s > 1.0)                            # 8 * sum(h) > 8 dominates the N(0, 0.05^2 H) rest
    assert len(up) > n // 8
    np.testing.assert_array_equal(am[up], big)
    np.testing.assert_array_equal(am[up], want["argmax"][up])


@pytest.mark.parametrize("kind,n,H,V", FUSED)
def test_fused_nan_stays_in_its_row(dev, select_kernel, kind, n, H, V):
    """A NaN in one token's hidden state makes that token's outputs NaN and leaves every other token alone."""
    select_kernel(kind)
    rng = np.random.default_rng(n * 3 + H)
    h32 = rng.standard_normal((n, H)).astype(np.float32)
    w32 = (rng.standard_normal((V, H)) * 0.1).astype(np.float32)
    bad = [2, n // 2]
    h32[bad[0], 5] = np.nan
    h32[bad[1], H - 1] = np.nan
    h = torch.from_numpy(h32).to(dev).to(torch.bfloat16)
    w = torch.from_numpy(w32).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    lp, lse, ent, am = _fused(dev, h, w, t)
    assert np.isnan(lp[bad]).all() and np.isnan(lse[bad]).all() and np.isnan(ent[bad]).all()
    ok = np.setdiff1d(np.arange(n), bad)
    want = oracle.lmhead_stats(bf16_bits_of(h[torch.from_numpy(ok).to(dev)]), bf16_bits_of(w), t[ok], 1.0)
    np.testing.assert_allclose(lp[ok], want["lp"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(lse[ok], want["lse"], atol=2e-3, rtol=0)
    np.testing.assert_allclose(ent[ok], want["entropy"], atol=2e-3, rtol=0)


@pytest.mark.parametrize("T", [0.05, 50.0])
@pytest.mark.parametrize("kind,n,H,V", FUSED)
def test_fused_extreme_temperature(dev, select_kernel, kind, n, H, V, T):
    """Logits of magnitude up to ~30 (|h| ~ 1, |w| ~ 8 / sqrt(H)) at T = 0.05 and 50.  Tolerance: the path's 2e-3,
    plus the fp32 accumulation bound of a logit (H * 2^-24 * max|h| * max|w|) divided by T with the logit, plus
    the fp32 rounding of z = x / T at its largest magnitude."""
    select_kernel(kind)
    rng = np.random.default_rng(int(T * 10) + n)
    h32 = rng.standard_normal((n, H)).astype(np.float32)
    w32 = (rng.standard_normal((V, H)) * (8.0 / np.sqrt(H))).astype(np.float32)
    h = torch.from_numpy(h32).to(dev).to(torch.bfloat16)
    w = torch.from_numpy(w32).to(dev).to(torch.bfloat16)
    t = rng.integers(0, V, size=n).astype(np.int32)
    lp, lse, ent, am = _fused(dev, h, w, t, T)
    want = oracle.lmhead_stats(bf16_bits_of(h), bf16_bits_of(w), t, T)
    zmax = 2 * float(np.abs(want["top1"]).max())            # |lp| reaches about twice the largest |z|
    acc = H * 2.0 ** -24 * float(np.abs(h32).max()) * float(np.abs(w32).max())
    tol = 2e-3 + acc / T + 2 * float(np.spacing(np.float32(max(zmax, 1.0))))
    np.testing.assert_allclose(lp, want["lp"], atol=tol, rtol=0)
    np.testing.assert_allclose(lse, want["lse"], atol=tol, rtol=0)
    np.testing.assert_allclose(ent, want["entropy"], atol=tol, rtol=0)
    assert np.isfinite(lp).all()
