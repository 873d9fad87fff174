"""tome_row_logprob_noalloc (partials in the library's own scratch array) against tome_row_logprob
(partials in a caller workspace): same kernels, so every output must be bit-identical.  Called through
the C ABI directly, twice in a row, the second call on a smaller input that reuses the same scratch."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run_both(lib, check, torch, dev, rows, V, dtype, seed, mask=False, temperature=1.0):
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn((rows, V), device=dev, generator=g) * 2.0
    if dtype == 1:
        x = x.to(torch.bfloat16)
    t = torch.randint(0, V, (rows,), device=dev, generator=g).to(torch.int32)
    valid = None
    if mask:
        valid = (torch.rand(rows, device=dev, generator=g) < 0.6).to(torch.int32)
        valid[0] = 1
    stream = torch.cuda.current_stream(dev).cuda_stream
    outs = []
    for which in ("workspace", "noalloc"):
        lp = torch.full((rows,), 7.0, dtype=torch.float32, device=dev)
        lse = torch.full((rows,), 7.0, dtype=torch.float32, device=dev)
        ent = torch.full((rows,), 7.0, dtype=torch.float32, device=dev)
        am = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        vp = valid.data_ptr() if valid is not None else None
        if which == "workspace":
            need = lib.tome_row_logprob_workspace(rows, V)
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
            check(lib.tome_row_logprob(x.data_ptr(), dtype, rows, V, V, t.data_ptr(), vp, temperature, lp.data_ptr(),
                                       lse.data_ptr(), ent.data_ptr(), am.data_ptr(), ws.data_ptr(), need, stream))
        else:
            check(lib.tome_row_logprob_noalloc(x.data_ptr(), dtype, rows, V, V, t.data_ptr(), vp, temperature,
                                               lp.data_ptr(), lse.data_ptr(), ent.data_ptr(), am.data_ptr(), stream))
        torch.cuda.synchronize()
        outs.append([o.cpu().numpy() for o in (lp, lse, ent, am)])
    for a, b in zip(*outs):
        assert np.array_equal(a.view(np.int32), b.view(np.int32))
    return outs[1]


def test_noalloc_matches_workspace_entry_on_two_calls_in_a_row(dev):
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    V = 151936
    # first call: 64 rows of fp32 logits, 8 workgroups per row; second: a smaller batch and vocabulary
    lp, lse, ent, am = _run_both(lib, _lib.check, torch, dev, 64, V, 0, seed=1)
    assert np.isfinite(lp).all() and (lp <= 1e-5).all() and (am >= 0).all() and (ent > 0).all()
    lp2, _, _, am2 = _run_both(lib, _lib.check, torch, dev, 5, 50000, 1, seed=2, mask=True, temperature=0.7)
    assert np.isfinite(lp2).all() and (am2 >= -1).all()
    # and a batch large enough that no row is split (the scratch is not touched at all)
    _run_both(lib, _lib.check, torch, dev, 600, 8192, 1, seed=3, mask=True)


def test_noalloc_checked_against_the_oracle(dev):
    import torch
    import oracle
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    rows, V = 16, 151936
    g = torch.Generator(device=dev).manual_seed(11)
    x = (torch.randn((rows, V), device=dev, generator=g) * 2.0).contiguous()
    t = torch.randint(0, V, (rows,), device=dev, generator=g).to(torch.int32)
    lp = torch.empty(rows, dtype=torch.float32, device=dev)
    am = torch.empty(rows, dtype=torch.int32, device=dev)
    _lib.check(lib.tome_row_logprob_noalloc(x.data_ptr(), 0, rows, V, V, t.data_ptr(), None, 1.0, lp.data_ptr(), None,
                                            None, am.data_ptr(), torch.cuda.current_stream(dev).cuda_stream))
    torch.cuda.synchronize()
    want = oracle.logprob_rows(x.cpu().numpy(), t.cpu().numpy(), 1.0)
    assert np.abs(lp.cpu().numpy() - want).max() < 1e-4     # fp32 logits: 1e-4 abs
    assert (am.cpu().numpy() == oracle.argmax_rows(x.cpu().numpy())).all()


def test_noalloc_replays_from_a_hip_graph(dev):
    """The callers this entry point is for include code under HIP graph capture: after one eager call (which looks
    the scratch address up, outside any capture) the call is captured and replayed on changing inputs; every replay
    must equal the eager call on the same inputs bit for bit, with unrelated eager work between the replays."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    rows, V = 48, 60000
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.zeros((rows, V), dtype=torch.float32, device=dev)
    t = torch.zeros(rows, dtype=torch.int32, device=dev)
    outs = {k: (torch.empty(rows, dtype=torch.float32, device=dev), torch.empty(rows, dtype=torch.int32, device=dev))
            for k in ("graph", "eager")}

    def call(which, stream):
        lp, am = outs[which]
        _lib.check(lib.tome_row_logprob_noalloc(x.data_ptr(), 0, rows, V, V, t.data_ptr(), None, 0.8, lp.data_ptr(), None,
                                                None, am.data_ptr(), stream))
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        call("graph", side.cuda_stream)                                   # warm-up: resolves the scratch address
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call("graph", torch.cuda.current_stream(dev).cuda_stream)
    for it in range(3):
        x.copy_(torch.randn((rows, V), device=dev, generator=g) * (1.0 + it))
        t.copy_(torch.randint(0, V, (rows,), device=dev, generator=g).to(torch.int32))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        call("eager", torch.cuda.current_stream(dev).cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(outs["graph"][0], outs["eager"][0]) and torch.equal(outs["graph"][1], outs["eager"][1])
        assert torch.isfinite(outs["graph"][0]).all()
        (x[:8] @ x[:8].T).sum().item()                                    # unrelated eager work between replays
