import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

V_QWEN3 = 151936


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def bf16_bits_of(t):
    """torch bf16 tensor (any device) -> numpy uint16 bit patterns, as the oracle reads them."""
    import torch
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def torch_bf16_from_f32(a, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(device).to(torch.bfloat16)


def check_argmax(h, w, got, want, temperature=1.0, rows=None, min_clear=0.9):
    """The fused kernels return the first maximum of the fp32 logits they accumulate (the rule stated in
    include/tome_logprob.h).  Against the exact (fp64) logits of the same bf16 inputs that means, on EVERY
    row: the logit of the id returned is within the fp32 summation bound of the maximum, and the id IS the exact
    argmax whenever the top two logits differ by more than that bound.
    Bound per row: H * 2^-24 * max|h_row| * max|w| (the header's figure), doubled because two computed logits
    are compared."""
    import oracle
    hb, wb = bf16_bits_of(h), bf16_bits_of(w)
    h64, w64 = oracle.to_f64(hb), oracle.to_f64(wb)
    rows = np.arange(h64.shape[0]) if rows is None else np.asarray(rows)
    H = h64.shape[1]
    bound = 2 * H * 2.0 ** -24 * np.abs(h64[rows]).max(axis=1) * np.abs(w64).max() / temperature
    assert ((got[rows] >= 0) & (got[rows] < w64.shape[0])).all()
    logit_got = np.einsum("rk,rk->r", h64[rows], w64[got[rows]]) / temperature
    assert (want["top1"][rows] - logit_got <= bound).all()
    clear = (want["top1"][rows] - want["top2"][rows]) > bound
    assert clear.mean() >= min_clear
    np.testing.assert_array_equal(got[rows][clear], want["argmax"][rows][clear])


@pytest.fixture(scope="session")
def dev():
    import torch
    return torch.device("cuda:0")
