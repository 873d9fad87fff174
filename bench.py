#!/usr/bin/env python3
"""Benchmark of the token-log-prob path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already resident in
HBM.  The headline workload is benchmark configuration 2 (the Qwen3-0.6B GRPO ref-logprob shape:
bf16 logits [8 x 512, 151936] with a padding mask).  The same JSON line carries one object per
further workload: configuration 2 without its mask, configuration 1 (64 x 151936 fp32, the
CPU-comparison shape), the whole `process_ref_logprobs_batched` call on configuration 2's batch
(`ref_entry`, logits and hidden-state mode: wall time per call, the kernels' share of it, host time per
chunk), the full-matrix log-softmax drop-in, the fused lm_head + log-softmax kernel at configurations
3, 4 and 5, the same entry behind the final RMSNorm and as the policy + reference pair over a shared
lm_head, at decode-step and small-batch sizes, one decode step's sampler, and the LoRA merge of one
UpdateWeights request.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only LEG[,LEG...]]

Every leg does W untimed warm-up steps, then an untimed settle phase (launches until the GPU has been
busy for SETTLE_MS, so that clocks have left their idle state; the count is reported as
`settle_launches`), then times EXACTLY K back-to-back steps between two HIP events on the launch
stream (`ms_per_step`, the mean), and finally repeats K steps with an event between launches for the
median of the per-launch times (`median_ms`, `min_ms`; this second pass does not feed `ms_per_step`).
The matrix-core legs add a clock pass: the same step is queued for CLOCK_MS of GPU time (untimed) and the
host meanwhile reads the engine clock the driver reports (`pp_dpm_sclk` of the device in sysfs, a
smoothed value) every few milliseconds; the median of the samples from the second half of that pass
is `sclk_mhz` (with the socket power and its cap from the same device's hwmon files as `power_w`, `power_cap_w`), and these legs price themselves against the published peak scaled to that clock as well
(`roofline.peak_at_sclk`, `roofline.frac_at_sclk`): the published 2.5 PFLOP/s is 256 CUs x 4096 FLOP per clock at the 2.4 GHz peak engine clock, which the part does not
hold under a matrix-core load on random operands.  The `ceiling` leg times the fused kernel's LDS -> MFMA loop
alone on random operands (`sustained_peak` in the later matrix-core legs), with the kernel's fill requests
(`sustained_peak_with_fill`) and with requests, softmax fold and step barrier together (`design_ceiling`
of the `fused_lmhead` leg: the kernel at config 3 on a memory system that always answers from cache).

Prints ONE JSON line on stdout.  Everything else goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

V = 151936
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
PEAK_ENGINE_CLOCK_MHZ = 2400.0  # the clock the published matrix-core figures are quoted at
SETTLE_MS = 60.0                # untimed GPU-busy time in front of every timed region (default of --settle-ms)
SETTLE = {"ms": SETTLE_MS}
CLOCK = {"ms": 400.0}           # GPU-busy time of the clock pass of the matrix-core legs (--clock-ms; 0 = none)
SETTLE_MAX_LAUNCHES = 2000
LEGS = ["row", "entry", "config1", "fullmatrix", "ceiling", "fused", "norm", "gemm", "config4", "config5", "pair", "small", "midsize",
        "decode", "lora"]
SUSTAINED = {"tflops": None, "with_fill": None, "with_fill_and_fold": None}   # bf16 MFMA rate of the probe loop on random operands, bare and with the
                                                  # fused kernel's fill requests, measured by the `ceiling` leg


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def load_counters():
    """HBM-side traffic per launch and the sustained MFMA rate, as measured with rocprofv3 and recorded
    beside the summaries they come from (profiles/counters.json).  Missing entries read as None."""
    try:
        with open(os.path.join(ROOT, "profiles", "counters.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


COUNTERS = load_counters()


def traffic_of(key):
    e = COUNTERS.get("traffic", {}).get(key)
    return None if e is None else float(e["fetch_bytes"]) + float(e["write_bytes"])


def make_config2(dev, seed=1234):
    """bf16 logits [8, 512, V] ~ N(0, 3^2) + one +15 spike per row; targets 50% spike / 50% uniform;
    lengths uniform in [64, 512]."""
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    G, L = 8, 512
    logits = torch.empty((G, L, V), device=dev, dtype=torch.bfloat16)
    for i in range(G):   # generate per group to bound the fp32 temporary
        logits[i] = (torch.randn((L, V), device=dev, generator=g) * 3.0).to(torch.bfloat16)
    spike = torch.randint(0, V, (G, L), device=dev, generator=g)
    flat = logits.view(G * L, V)
    rows = torch.arange(G * L, device=dev)
    flat[rows, spike.view(-1)] = (flat[rows, spike.view(-1)].float() + 15.0).to(torch.bfloat16)
    uniform = torch.randint(0, V, (G, L), device=dev, generator=g)
    pick = torch.rand((G, L), device=dev, generator=g) < 0.5
    targets = torch.where(pick, spike, uniform).to(torch.int32)
    lengths = torch.randint(64, 513, (G,), device=dev, generator=g)
    return logits, targets, lengths, spike


_SCLK = {"path": False}


def sclk_path():
    """sysfs file with the engine clock levels of the GPU that torch calls device 0, or None."""
    if _SCLK["path"] is False:
        import glob
        import torch
        found = None
        try:
            pr = torch.cuda.get_device_properties(0)
            want = "%04x:%02x:%02x." % (pr.pci_domain_id, pr.pci_bus_id, pr.pci_device_id)
            paths = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
            hits = [q for q in paths if want in os.path.realpath(os.path.dirname(q))]
            found = hits[0] if hits else (paths[0] if len(paths) == 1 else None)
        except Exception:  # noqa: BLE001 - the clock is an optional extra
            found = None
        _SCLK["path"] = found
    return _SCLK["path"]


def read_sclk_mhz():
    """The level the driver marks as current ('1: 1836Mhz *'), in MHz, or None."""
    path = sclk_path()
    if not path:
        return None
    try:
        with open(path) as f:
            for line in f:
                if line.rstrip().endswith("*"):
                    return float(line.split(":")[1].strip().split("Mhz")[0])
    except (OSError, ValueError, IndexError):
        return None
    return None


def power_paths():
    """(sysfs file with the socket power in microwatts, file with its cap) of the same GPU, or (None, None)."""
    if "power" not in _SCLK:
        import glob
        avg = cap = None
        if sclk_path():
            dev = os.path.dirname(sclk_path())
            for name in ("power1_average", "power1_input"):
                hits = sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*", name)))
                if hits:
                    avg = hits[0]
                    break
            hits = sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*", "power1_cap")))
            cap = hits[0] if hits else None
        _SCLK["power"] = (avg, cap)
    return _SCLK["power"]


def read_watts(path):
    if not path:
        return None
    try:
        with open(path) as f:
            return float(f.read().strip()) / 1e6
    except (OSError, ValueError):
        return None


def time_steps(fn, steps, warmup, clock=False):
    """Warm-up, settle, timed region, per-launch pass (see the module docstring).  Times in milliseconds by
    HIP events recorded on the stream the kernels run on (torch's current stream, which the library
    launches into)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    # settle: untimed launches until the GPU has been busy for SETTLE_MS
    settle, busy, batch = 0, 0.0, 1
    while busy < SETTLE["ms"] and settle < SETTLE_MAX_LAUNCHES:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if settle:   # size the next batch from the time per launch seen so far
            batch = int(min(max(1.0, (SETTLE["ms"] - busy) / (busy / settle)) + 1, 200, SETTLE_MAX_LAUNCHES - settle))
        a.record()
        for _ in range(batch):
            fn()
        b.record()
        torch.cuda.synchronize()
        busy += a.elapsed_time(b)
        settle += batch
    # the timed region: exactly `steps` launches between two events
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    mean_ms = start.elapsed_time(stop) / steps
    # per-launch times: a second pass with an event between launches
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    per = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    clocks, watts = [], []   # clock pass: the engine clock (and the socket power) while the same step keeps the GPU busy for CLOCK["ms"]
    if clock and CLOCK["ms"] > 0 and sclk_path():
        n = max(steps, int(CLOCK["ms"] / mean_ms) + 1)
        done = torch.cuda.Event()
        t1 = time.perf_counter()
        for _ in range(n):
            fn()
        done.record()
        while not done.query():
            c = read_sclk_mhz()
            w = read_watts(power_paths()[0])
            if c and not done.query():
                clocks.append((time.perf_counter() - t1, c))
                if w:
                    watts.append((time.perf_counter() - t1, w))
            time.sleep(0.003)
        torch.cuda.synchronize()
        half = (time.perf_counter() - t1) / 2
        clocks = sorted(c for (at, c) in clocks if at >= half)
        watts = sorted(w for (at, w) in watts if at >= half)
    return {"ms": mean_ms, "wall_ms": wall_ms, "median_ms": per[len(per) // 2], "min_ms": per[0],
            "settle_launches": settle, "sclk_mhz": clocks[len(clocks) // 2] if clocks else None,
            "power_w": watts[len(watts) // 2] if watts else None,
            "power_cap_w": read_watts(power_paths()[1]) if watts else None}


def timing_fields(t):
    d = {"ms_per_step": t["ms"], "median_ms": t["median_ms"], "min_ms": t["min_ms"],
         "settle_launches": t["settle_launches"]}
    if t.get("sclk_mhz"):
        d["sclk_mhz"] = t["sclk_mhz"]
    if t.get("power_w"):   # socket power the driver reports during the clock pass, and the cap it regulates to
        d["power_w"] = t["power_w"]
        d["power_cap_w"] = t.get("power_cap_w")
    return d


def hbm_roofline(nbytes, ms, traffic, kernel):
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
            "traffic": traffic, "kernel": kernel, "bytes_per_launch": nbytes}


def mfma_roofline(flop, ms, traffic, kernel, sclk_mhz=None):
    tf = flop / (ms * 1e-3) / 1e12
    r = {"bound": "mfma", "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
         "frac": tf / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic, "kernel": kernel, "flop_per_launch": flop}
    if sclk_mhz:   # the published peak at the engine clock the part held during this leg
        r["peak_at_sclk"] = MFMA_BF16_PEAK_TFLOPS * sclk_mhz / PEAK_ENGINE_CLOCK_MHZ
        r["frac_at_sclk"] = tf / r["peak_at_sclk"]
    if SUSTAINED["tflops"]:   # what the bare LDS -> MFMA loop reaches on random bf16 operands, same run (`ceiling` leg)
        r["sustained_peak"] = SUSTAINED["tflops"]
        r["frac_of_sustained"] = tf / SUSTAINED["tflops"]
    if SUSTAINED["with_fill"]:   # the same loop issuing the fused kernel's eight global -> LDS requests per wave and slab
        r["sustained_peak_with_fill"] = SUSTAINED["with_fill"]
        r["frac_of_sustained_with_fill"] = tf / SUSTAINED["with_fill"]
    return r


# ---- row kernel: configuration 2 (headline) and configuration 1 -----------------------------------------
def bench_row(dev, steps, warmup, variant="both"):
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    logits, targets, lengths, spike = make_config2(dev)
    G, L, _ = logits.shape
    rows = G * L
    valid = (torch.arange(L, device=dev)[None, :] < lengths[:, None]).to(torch.int32).reshape(-1).contiguous()
    n_valid = int(valid.sum().item())
    flat = logits.view(rows, V)
    tg = targets.reshape(-1).contiguous()
    lp = torch.empty(rows, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_row_logprob_workspace(rows, V)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step(mask):
        _lib.check(lib.tome_row_logprob(flat.data_ptr(), 1, rows, V, V, tg.data_ptr(),
                                        valid.data_ptr() if mask else None, 1.0, lp.data_ptr(), None, None, None,
                                        ws.data_ptr(), ws_bytes, stream))

    # correctness gate on what is being timed: log-probs are finite and <= 0, masked rows are zero
    step(True)
    torch.cuda.synchronize()
    got = lp.clone()
    assert torch.isfinite(got).all() and (got <= 1e-5).all()
    assert (got[valid == 0] == 0).all()

    # the same rows as a packed row list (tome_row_logprob_rows): only the valid rows are launched
    idx = torch.nonzero(valid).view(-1).to(torch.int32).contiguous()
    tg_packed = tg[idx.long()].contiguous()
    lp_packed = torch.empty(n_valid, dtype=torch.float32, device=dev)
    ws2_bytes = lib.tome_row_logprob_workspace(n_valid, V)
    ws2 = torch.empty(max(ws2_bytes, 1), dtype=torch.uint8, device=dev)

    def step_list():
        _lib.check(lib.tome_row_logprob_rows(flat.data_ptr(), 1, rows, V, V, idx.data_ptr(), n_valid, tg_packed.data_ptr(), 1.0,
                                             lp_packed.data_ptr(), None, None, None, ws2.data_ptr(), ws2_bytes, stream))
    step_list()
    torch.cuda.synchronize()
    assert torch.equal(lp_packed, got[idx.long()])       # the row list scores exactly what the mask scores

    out = {"n_valid": n_valid, "rows": rows, "bytes_mask": n_valid * V * 2, "bytes_all": rows * V * 2}
    if variant in ("both", "mask"):
        out["mask"] = time_steps(lambda: step(True), steps, warmup)
    if variant in ("both", "list"):
        out["list"] = time_steps(step_list, steps, warmup)
    if variant in ("both", "all"):
        out["all"] = time_steps(lambda: step(False), steps, warmup)
    del logits, flat
    torch.cuda.empty_cache()
    return out


def bench_config1(dev, steps, warmup):
    """Configuration 1: 64 rows x 151936 fp32 logits ~ N(0, 2^2), uniform targets - the shape of the reference's
    CPU path (mlx-impl/node.py:400-404).  38.9 MB per launch would sit in the 256 MB last-level cache, so the
    launches rotate through 16 buffers (622 MB) and every row comes from HBM."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    rows, nbuf = 64, 16
    g = torch.Generator(device=dev).manual_seed(11)
    xs = [torch.randn((rows, V), device=dev, generator=g) * 2.0 for _ in range(nbuf)]
    t = torch.randint(0, V, (rows,), device=dev, generator=g).to(torch.int32)
    lp = torch.empty(rows, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_row_logprob_workspace(rows, V)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    i = [0]

    def step():
        x = xs[i[0] % nbuf]
        i[0] += 1
        _lib.check(lib.tome_row_logprob(x.data_ptr(), 0, rows, V, V, t.data_ptr(), None, 1.0, lp.data_ptr(), None, None,
                                        None, ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    want = torch.log_softmax(xs[0].double(), dim=-1)[torch.arange(rows, device=dev), t.long()]
    assert (lp.double() - want).abs().max().item() < 1e-4        # gate on what is timed (fp32 logits: 1e-4 abs)
    tm = time_steps(step, steps, warmup)
    tm.update({"rows": rows, "bytes": rows * V * 4})
    return tm


# ---- fused lm_head + log-softmax ---------------------------------------------------------------------
def bench_fused(dev, steps, warmup, n=4096, H=1024, temperature=1.0, lengths=None, seed=4321):
    """Fused lm_head + log-softmax on [n, H] x [V, H]: config 3 by default.  `lengths` = (sequences, L, lo, hi)
    gives the padding mask of config 4 (per-sequence valid prefixes, lengths uniform in [lo, hi])."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    g = torch.Generator(device=dev).manual_seed(seed)
    hidden = torch.randn((n, H), device=dev, generator=g).to(torch.bfloat16)
    weight = (torch.randn((V, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    targets = torch.randint(0, V, (n,), device=dev, generator=g).to(torch.int32)
    valid, n_valid = None, n
    if lengths is not None:
        S, L, lo, hi = lengths
        assert S * L == n
        lens = torch.randint(lo, hi + 1, (S,), device=dev, generator=g)
        valid = (torch.arange(L, device=dev)[None, :] < lens[:, None]).to(torch.int32).reshape(-1).contiguous()
        n_valid = int(valid.sum().item())
    lp = torch.empty(n, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_fused_lmhead_logprob_workspace(n, H, V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_fused_lmhead_logprob(hidden.data_ptr(), weight.data_ptr(), n, H, V, H, H,
                                                 targets.data_ptr(), valid.data_ptr() if valid is not None else None,
                                                 temperature, lp.data_ptr(), None, None, None,
                                                 ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    assert torch.isfinite(lp).all() and (lp <= 1e-5).all()
    # gate on what is timed: 64 valid rows against a plain fp32 matmul + log_softmax
    idx = (torch.arange(n, device=dev) if valid is None else torch.nonzero(valid).view(-1))[:: max(1, n_valid // 64)][:64]
    ref = torch.log_softmax((hidden[idx].float() @ weight.float().T) / temperature, dim=-1)
    ref = ref[torch.arange(idx.numel(), device=dev), targets[idx].long()]
    assert (lp[idx] - ref).abs().max().item() < 2e-3
    del ref
    tm = time_steps(step, steps, warmup, clock=True)
    tm.update({"tokens": n, "valid": n_valid, "H": H, "flop": 2.0 * n_valid * H * V,
               "bytes": V * H * 2 + n_valid * H * 2})
    return tm


def bench_library_gemm(dev, steps, warmup, n=4096, H=1024, vocab=V):
    """The vendor library's bf16 GEMM alone, for scale: logits = hidden @ W^T written as bf16 [n, vocab] (what
    mlx-impl/model.py:538 materialises), no softmax - on config 3's shape, and on a square 8192^3 product (the shape
    such libraries are tuned for: what this part sustains on random operands).  torch.mm dispatches to hipBLASLt / rocBLAS."""
    import torch
    g = torch.Generator(device=dev).manual_seed(4321)
    hidden = torch.randn((n, H), device=dev, generator=g).to(torch.bfloat16)
    weight = (torch.randn((vocab, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    out = torch.empty((n, vocab), device=dev, dtype=torch.bfloat16)
    wt = weight.t()

    def step():
        torch.mm(hidden, wt, out=out)
    step()
    torch.cuda.synchronize()
    tm = time_steps(step, steps, warmup, clock=True)
    tm.update({"tokens": n, "H": H, "flop": 2.0 * n * H * vocab})
    return tm


def bench_dual(dev, steps, warmup, n=32 * 2048, H=4096):
    """Configuration 5: GRPO policy + reference dual pass, two weight sets [V, 4096] (ref = policy + N(0, 0.002^2)),
    hidden [32 x 2048, 4096]; outputs lp, ref_lp, k3 and entropy per token."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    g = torch.Generator(device=dev).manual_seed(555)
    hidden = torch.empty((n, H), device=dev, dtype=torch.bfloat16)
    for i in range(0, n, 8192):
        hidden[i:i + 8192] = torch.randn((min(8192, n - i), H), device=dev, generator=g).to(torch.bfloat16)
    w_pol = torch.empty((V, H), device=dev, dtype=torch.bfloat16)
    w_ref = torch.empty((V, H), device=dev, dtype=torch.bfloat16)
    for i in range(0, V, 16384):
        m = min(16384, V - i)
        wp = (torch.randn((m, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
        w_pol[i:i + m] = wp
        w_ref[i:i + m] = (wp.float() + torch.randn((m, H), device=dev, generator=g) * 0.002).to(torch.bfloat16)
    targets = torch.randint(0, V, (n,), device=dev, generator=g).to(torch.int32)
    outs = [torch.empty(n, dtype=torch.float32, device=dev) for _ in range(4)]
    ws_bytes = lib.tome_grpo_dual_workspace(n, H, V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_grpo_dual(hidden.data_ptr(), w_pol.data_ptr(), w_ref.data_ptr(), n, H, V, H, H,
                                      targets.data_ptr(), None, 1.0, outs[0].data_ptr(), outs[1].data_ptr(),
                                      outs[2].data_ptr(), outs[3].data_ptr(), ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    lp, ref_lp, k3, ent = outs
    assert torch.isfinite(lp).all() and (lp <= 1e-5).all() and (k3 >= 0).all() and (ent > 0).all()
    idx = torch.arange(0, n, n // 32, device=dev)[:32]
    for w, got in ((w_pol, lp), (w_ref, ref_lp)):       # gate: 32 rows of each weight set against fp32 torch
        ref = torch.log_softmax(hidden[idx].float() @ w.float().T, dim=-1)[torch.arange(32, device=dev), targets[idx].long()]
        assert (got[idx] - ref).abs().max().item() < 2e-3
    tm = time_steps(step, steps, warmup, clock=True)
    tm.update({"tokens": n, "H": H, "flop": 2.0 * 2.0 * n * H * V, "bytes": 2 * V * H * 2 + n * H * 2})
    return tm


def bench_ceiling(dev, steps, warmup, operands="random", with_requests=False, with_fold=False, with_barrier=False):
    """The fused kernel's LDS -> MFMA inner loop alone (tome_probe_mfma_ceiling): one workgroup per CU, operands
    copied into LDS once, no global loads, barriers or epilogue in the loop.  `random`: W rows ~N(0, 0.02^2) and
    token rows ~N(0, 1) as in config 3; `constant`: every operand 1.0."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    g = torch.Generator(device=dev).manual_seed(31)
    if operands == "random":
        ops = torch.cat([torch.randn(256 * 64, device=dev, generator=g) * 0.02, torch.randn(256 * 64, device=dev, generator=g)])
    else:
        ops = torch.ones(512 * 64, device=dev)
    ops = ops.to(torch.bfloat16).contiguous()
    n_wg = torch.cuda.get_device_properties(dev).multi_processor_count
    k_steps = 1024                                      # 64-wide K slabs per launch: about 1 ms
    sink = torch.empty(n_wg * 512, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_probe_mfma_ceiling(ops.data_ptr(), ops.numel() * 2, n_wg, k_steps,
                                                (1 if with_requests else 0) | (2 if with_fold else 0) | (4 if with_barrier else 0),
                                                sink.data_ptr(), sink.numel() * 4, stream))
    step()
    torch.cuda.synchronize()
    assert torch.isfinite(sink).all()
    tm = time_steps(step, steps, warmup, clock=True)
    tm.update({"flop": float(n_wg) * k_steps * 2 * 256 * 256 * 64, "workgroups": n_wg, "k_steps": k_steps})
    return tm


def bench_decode(dev, steps, warmup):
    """One decode step's sampler + log-prob (mlx-impl/node.py:590-605) on config 1's shape: 64 rows of fp32
    logits, top-k 20.  The buffers rotate so that the rows come from HBM, not from a warm cache."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    rows, k, nbuf = 64, 20, 16
    g = torch.Generator(device=dev).manual_seed(77)
    xs = [torch.randn((rows, V), device=dev, generator=g) * 2.0 for _ in range(nbuf)]
    u = torch.rand(rows, device=dev, generator=g)
    tok = torch.empty(rows, dtype=torch.int32, device=dev)
    lp = torch.empty(rows, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_row_sample_workspace(0, rows, V, k)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    i = [0]

    def step():
        x = xs[i[0] % nbuf]
        i[0] += 1
        _lib.check(lib.tome_row_sample(x.data_ptr(), 0, rows, V, V, u.data_ptr(), None, 1.0, k, tok.data_ptr(),
                                       lp.data_ptr(), None, None, None, None, ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    assert (tok >= 0).all() and (tok < V).all() and torch.isfinite(lp).all()
    tm = time_steps(step, steps, warmup)
    tm.update({"rows": rows, "top_k": k, "bytes": rows * V * 4})
    return tm


def bench_lora(dev, steps, warmup):
    """One UpdateWeights (mlx-impl/node.py:102-164) at Qwen3-0.6B's shape: 28 layers x (qkv_proj [4096, 1024],
    gate_up_proj [6144, 1024], down_proj [1024, 3072]), rank 8, scale 2.5 - 84 merges, one C-ABI call.
    Algorithmic bytes: every base weight read once and every policy weight written once."""
    import ctypes
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    layers, rank = 28, 8
    shapes = [(4096, 1024), (6144, 1024), (1024, 3072)]
    g = torch.Generator(device=dev).manual_seed(99)
    keep, n_bytes = [], 0
    jobs = (_lib.TomeLoraJob * (layers * len(shapes)))()
    for i in range(layers * len(shapes)):
        rows, cols = shapes[i % len(shapes)]
        base = (torch.randn((rows, cols), device=dev, generator=g) * 0.02).to(torch.bfloat16)
        out = torch.empty_like(base)
        a = (torch.randn((rank, cols), device=dev, generator=g) * 0.05).to(torch.bfloat16)
        b = (torch.randn((rows, rank), device=dev, generator=g) * 0.05).to(torch.bfloat16)
        keep += [base, out, a, b]
        j = jobs[i]
        j.base, j.out, j.lora_a, j.lora_b = base.data_ptr(), out.data_ptr(), a.data_ptr(), b.data_ptr()
        j.rows, j.cols, j.rank, j.base_stride, j.out_stride, j.scale = rows, cols, rank, cols, cols, 2.5
        n_bytes += rows * cols * 4
    jp = ctypes.cast(jobs, ctypes.c_void_p)
    ws_bytes = lib.tome_lora_merge_workspace(jp, len(jobs))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_lora_merge(jp, len(jobs), ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    base, out, a, b = keep[:4]                      # gate on what is timed: the first merge against fp32 torch
    want = base.float() + 2.5 * (b.float() @ a.float())
    assert (out.float() - want).abs().max().item() <= 2.0 ** -8 * want.abs().max().item() + 1e-3
    tm = time_steps(step, steps, warmup)
    tm.update({"bytes": n_bytes, "jobs": len(jobs), "rank": rank})
    return tm


def bench_full_matrix(dev, steps, warmup, rows, dtype_name):
    """tome_full_log_softmax, the drop-in of fused_log_softmax (mlx-impl/model.py:77-89): the whole [rows, V] matrix
    of log-probs in the input dtype.  Algorithmic bytes: 3 * V * sizeof(T) per row with two passes (one read for the row's
    lse, one read and one write of the matrix), 2 * V * sizeof(T) where the one-pass kernel applies.  The small shape
    rotates through 16 input / output pairs so that rows come from HBM, not from the last-level cache."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    dt = torch.bfloat16 if dtype_name == "bf16" else torch.float32
    code, esize = (1, 2) if dtype_name == "bf16" else (0, 4)
    nbuf = 1 if rows * V * esize > (1 << 30) else 16
    g = torch.Generator(device=dev).manual_seed(21)
    xs = []
    for _ in range(nbuf):
        x = torch.empty((rows, V), device=dev, dtype=dt)
        for i in range(0, rows, 512):
            x[i:i + 512] = (torch.randn((min(512, rows - i), V), device=dev, generator=g) * 2.0).to(dt)
        xs.append(x)
    outs = [torch.empty_like(xs[0]) for _ in range(nbuf)]
    row_lse = torch.empty(rows, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_row_logprob_workspace(rows, V)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    i = [0]

    def step():
        k = i[0] % nbuf
        i[0] += 1
        _lib.check(lib.tome_full_log_softmax(xs[k].data_ptr(), outs[k].data_ptr(), code, rows, V, V, V, 1.0,
                                             row_lse.data_ptr(), ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    sample = torch.arange(0, rows, max(1, rows // 16), device=dev)[:16]     # gate: 16 rows against torch in fp64
    want = torch.log_softmax(xs[0][sample].double(), dim=-1)
    tol = 1e-4 if dtype_name == "f32" else 0.25                              # bf16 output and subtraction: two ulps at |x| in [16, 32)
    assert (outs[0][sample].double() - want).abs().max().item() <= tol
    tm = time_steps(step, steps, warmup)
    # bf16 rows of up to 155648 elements take the one-pass kernel (the row stays in a workgroup's registers): read once,
    # written once.  Everything else is two passes: read for the row's lse, read again and written.
    passes = 2 if (dtype_name == "bf16" and V >= 16384 and V // 8 <= 19 * 1024) else 3
    tm.update({"rows": rows, "bytes": passes * rows * V * esize, "passes_over_the_matrix": passes,
               "bytes_if_three_passes": 3 * rows * V * esize})
    if nbuf == 1:
        # For scale: the same read + write volume through torch's elementwise kernel (tiny workgroups: the grain at which
        # reads and writes mix best on this part), and torch's own log_softmax on the same matrix.
        tm["torch_mul_same_bytes_ms"] = time_steps(lambda: torch.mul(xs[0], 2.0, out=outs[0]), steps, warmup)["ms"]
        tm["torch_log_softmax_ms"] = time_steps(lambda: torch.log_softmax(xs[0], dim=-1), max(2, steps // 4), 1)["ms"]
    return tm


def bench_norm_lmhead(dev, steps, warmup, n=4096, H=1024):
    """tome_norm_lmhead_logprob (mlx-impl/model.py:536-538 + node.py:400-404) at config 3's shape with config 2's
    padding mask (8 sequences x 512 positions, lengths uniform in [64, 512]): the final RMSNorm is applied to the
    valid rows only, which are then multiplied.  FLOP counted on valid tokens."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    g = torch.Generator(device=dev).manual_seed(808)
    hidden = (torch.randn((n, H), device=dev, generator=g) * 3.0).to(torch.bfloat16)       # pre-norm states
    norm_w = (1.0 + 0.1 * torch.randn((H,), device=dev, generator=g)).to(torch.bfloat16)
    weight = (torch.randn((V, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    targets = torch.randint(0, V, (n,), device=dev, generator=g).to(torch.int32)
    lens = torch.randint(64, 513, (8,), device=dev, generator=g)
    valid = (torch.arange(512, device=dev)[None, :] < lens[:, None]).to(torch.int32).reshape(-1).contiguous()
    n_valid = int(valid.sum().item())
    lp = torch.empty(n, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_norm_lmhead_logprob_workspace(n, H, V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_norm_lmhead_logprob(hidden.data_ptr(), norm_w.data_ptr(), 1e-6, weight.data_ptr(), n, H, V, H, H,
                                                targets.data_ptr(), valid.data_ptr(), 1.0, lp.data_ptr(), None, None, None,
                                                ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    idx = torch.nonzero(valid).view(-1)[:: max(1, n_valid // 64)][:64]      # gate: 64 valid rows against torch
    x = hidden[idx].float()
    y = (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16).float() * norm_w.float()
    ref = torch.log_softmax(y.to(torch.bfloat16).float() @ weight.float().T, dim=-1)
    ref = ref[torch.arange(idx.numel(), device=dev), targets[idx].long()]
    assert (lp[idx] - ref).abs().max().item() < 4e-3 and (lp[valid == 0] == 0).all()
    tm = time_steps(step, steps, warmup, clock=True)
    tm.update({"tokens": n, "valid": n_valid, "H": H, "flop": 2.0 * n_valid * H * V})
    return tm


def bench_pair(dev, steps, warmup, n=8192, H=4096):
    """tome_grpo_pair: the policy + reference pass in the reference's own layout (mlx-impl/node.py:65-66, 443): one
    hidden-state matrix per model, one shared lm_head.  Outputs lp, ref_lp, k3, entropy."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    g = torch.Generator(device=dev).manual_seed(909)
    h_pol = torch.randn((n, H), device=dev, generator=g).to(torch.bfloat16)
    h_ref = (h_pol.float() + 0.05 * torch.randn((n, H), device=dev, generator=g)).to(torch.bfloat16)
    weight = torch.empty((V, H), device=dev, dtype=torch.bfloat16)
    for i in range(0, V, 16384):
        m = min(16384, V - i)
        weight[i:i + m] = (torch.randn((m, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    targets = torch.randint(0, V, (n,), device=dev, generator=g).to(torch.int32)
    outs = [torch.empty(n, dtype=torch.float32, device=dev) for _ in range(4)]
    ws_bytes = lib.tome_grpo_pair_workspace(n, H, V, 0)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_grpo_pair(h_pol.data_ptr(), h_ref.data_ptr(), None, 0.0, weight.data_ptr(), weight.data_ptr(),
                                      n, H, V, H, H, targets.data_ptr(), None, 1.0, outs[0].data_ptr(), outs[1].data_ptr(),
                                      outs[2].data_ptr(), outs[3].data_ptr(), ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    lp, ref_lp, k3, ent = outs
    assert torch.isfinite(lp).all() and (lp <= 1e-5).all() and (k3 >= 0).all() and (ent > 0).all()
    idx = torch.arange(0, n, n // 32, device=dev)[:32]
    for h, got in ((h_pol, lp), (h_ref, ref_lp)):       # gate: 32 rows of each model against fp32 torch
        ref = torch.log_softmax(h[idx].float() @ weight.float().T, dim=-1)[torch.arange(32, device=dev), targets[idx].long()]
        assert (got[idx] - ref).abs().max().item() < 2e-3
    tm = time_steps(step, steps, warmup, clock=True)
    tm.update({"tokens": n, "H": H, "flop": 2.0 * 2.0 * n * H * V})
    return tm


def bench_ref_entry(dev, steps, warmup, mode):
    """The entry itself, RefLogprobServicer.process_ref_logprobs_batched (mlx-impl/node.py:391-461), end to end on the
    host clock: config 2's batch - 256-token prompts, G = 8 completions of U[64, 512] tokens each - over 32 prompts,
    i.e. 8 chunks of max_ref_batch_size = 32 sequences per call.  The model is a stub whose output is already
    resident in HBM (the model's forward is not part of this path): `logits` mode returns bf16 logits
    [32, max_len, V]; `hidden` mode returns final hidden states [32, max_len, 1024] for the fused lm_head kernel.
    A step is one call of the entry; it ends with the last chunk's log-probs appended to the Python lists."""
    import numpy as np
    import torch
    import tome_amd
    from tome_amd.node import Completion, Prompt, PromptRollout
    from tome_amd.wire import iter_ref_work, scatter_ref_logprobs
    n_prompts, G, p_len, batch, H = 32, 8, 256, 32, 1024
    rng = np.random.default_rng(2024)
    prompts = [Prompt(f"p{i}", rng.integers(0, V, size=p_len).tolist()) for i in range(n_prompts)]
    comp = [[rng.integers(0, V, size=int(rng.integers(64, 513))).tolist() for _ in range(G)] for _ in range(n_prompts)]

    def fresh_results():
        return [PromptRollout(f"p{i}", [Completion(tokens=c) for c in comp[i]]) for i in range(n_prompts)]
    max_len = p_len + 511
    g = torch.Generator(device=dev).manual_seed(3)
    if mode == "logits":
        store = torch.empty(batch * max_len * V, device=dev, dtype=torch.bfloat16)
        for i in range(0, store.numel(), 1 << 28):
            store[i:i + (1 << 28)] = (torch.randn((min(1 << 28, store.numel() - i),), device=dev, generator=g) * 3.0).to(torch.bfloat16)
        width, weight = V, None
    else:
        store = torch.randn((batch * max_len * H,), device=dev, generator=g).to(torch.bfloat16)
        weight = (torch.randn((V, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
        width = H

    def model(full_ids, cache=None):                   # output already in HBM: a contiguous [B, L, width] view
        b, length = full_ids.shape
        return store[: b * length * width].view(b, length, width), None
    svc = tome_amd.RefLogprobServicer(model, device=dev, max_ref_batch_size=batch, lm_head_weight=weight)

    # gate on what is timed: the entry's lists against direct kernel calls on the same chunks
    results = fresh_results()
    svc.process_ref_logprobs_batched(prompts, results, G, 1.0)
    chunks = list(iter_ref_work(prompts, fresh_results(), G, batch))
    n_tokens = sum(c.n_scored for c in chunks)
    assert svc.last_ref_tokens == n_tokens and all(len(c.ref_log_probs) == len(c.tokens) for r in results for c in r.completions)
    ch = chunks[1]
    out, _ = model(torch.from_numpy(ch.ids).to(dev))
    rows_d, tg_d = torch.from_numpy(ch.scored_rows).to(dev), torch.from_numpy(ch.scored_targets).to(dev)
    if mode == "logits":
        direct = tome_amd.token_logprobs_rows(out, rows_d, tg_d, 1.0).lp
    else:
        direct = tome_amd.fused_lmhead_logprobs(out.reshape(-1, H).index_select(0, rows_d.long()), weight, tg_d, 1.0).lp
    p_idx, gi = ch.owners[0]
    assert np.allclose(results[p_idx].completions[gi].ref_log_probs, direct[: int(ch.cu_lens[1])].cpu().numpy(), atol=0, rtol=0)

    def kernel_pass():                                 # the GPU work of one call, without the entry around it
        for c, (r, t) in zip(chunks, dev_lists):
            o, _ = model(torch.empty((c.ids.shape[0], c.ids.shape[1]), dtype=torch.int64, device="meta"))
            if mode == "logits":
                tome_amd.token_logprobs_rows(o, r, t, 1.0)
            else:
                tome_amd.fused_lmhead_logprobs(o.reshape(-1, H).index_select(0, r.long()), weight, t, 1.0)
    dev_lists = [(torch.from_numpy(c.scored_rows).to(dev), torch.from_numpy(c.scored_targets).to(dev)) for c in chunks]
    kt = time_steps(kernel_pass, steps, warmup)

    def host_pass():                                   # the host bookkeeping of one call, without the GPU
        res = fresh_results()
        t0 = time.perf_counter()
        for c in iter_ref_work(prompts, res, G, batch):
            scatter_ref_logprobs(c, np.zeros(c.n_scored, dtype=np.float32), res)
        return time.perf_counter() - t0
    host_s = sorted(host_pass() for _ in range(max(5, steps)))

    for _ in range(warmup):
        svc.process_ref_logprobs_batched(prompts, fresh_results(), G, 1.0)
    walls = []
    for _ in range(steps):
        res = fresh_results()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        svc.process_ref_logprobs_batched(prompts, res, G, 1.0)
        walls.append((time.perf_counter() - t0) * 1e3)
    mean_ms = sum(walls) / len(walls)
    walls.sort()
    return {"ms": mean_ms, "median_ms": walls[len(walls) // 2], "min_ms": walls[0], "settle_launches": 0,
            "tokens": n_tokens, "chunks": len(chunks), "sequences": n_prompts * G,
            "kernel_ms": kt["ms"], "host_us_per_chunk": host_s[len(host_s) // 2] * 1e6 / len(chunks),
            "bytes": n_tokens * V * 2 if mode == "logits" else None,
            "flop": 2.0 * n_tokens * H * V if mode == "hidden" else None}


# ---- CPU baseline -------------------------------------------------------------------------------------
def cpu_baseline(budget_s=10.0):
    """The reference's CPU path, local_compute_logprobs (mlx-impl/node.py:400-404), on configuration 1 (64 rows x
    151936 fp32 logits ~ N(0, 2^2), uniform targets): the oracle's NumPy fp32 restatement (one core), the same
    arithmetic with torch's CPU operators (its thread count stated) and in scalar C with OpenMP over rows."""
    import numpy as np
    import oracle
    rows = 64
    rng = np.random.default_rng(99)
    x = (rng.standard_normal((rows, V)) * 2.0).astype(np.float32)
    t = rng.integers(0, V, size=rows).astype(np.int32)

    def median_time(fn, budget, cap=5000):
        fn()
        times = []
        t_end = time.perf_counter() + budget
        while time.perf_counter() < t_end and len(times) < cap:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2], len(times)

    med, n = median_time(lambda: oracle.local_compute_logprobs_f32(x, t, 1.0), budget_s)
    out = {"value": rows / med, "unit": "token-logprobs/s", "cores": 1, "kind": "port",
           "sample": f"config 1: {rows} rows x {V} fp32 logits, NumPy fp32 restatement of node.py:400-404 "
                     f"(oracle.local_compute_logprobs_f32), median of {n} passes"}
    try:   # the same expression on torch's CPU operators: the multi-threaded library figure
        import torch
        xt, tt = torch.from_numpy(x), torch.from_numpy(t.astype(np.int64))

        def torch_pass():
            z = xt / 1.0
            return torch.take_along_dim(z, tt[:, None], dim=-1)[:, 0] - torch.logsumexp(z, dim=-1)
        med_t, n_t = median_time(torch_pass, budget_s / 2)
        out["torch_cpu"] = {"value": rows / med_t, "cores": torch.get_num_threads(), "kind": "port",
                            "sample": f"same rows, torch CPU operators (x / T, logsumexp, take_along_dim), "
                                      f"torch.get_num_threads() = {torch.get_num_threads()}, median of {n_t} passes"}
    except Exception as e:
        log("cpu torch baseline skipped:", e)
    try:   # scalar C with OpenMP over rows
        from oracle import cport
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        med_c, n_c = median_time(lambda: cport.local_compute_logprobs_c(x, t, 1.0), budget_s / 4)
        out["multicore"] = {"value": rows / med_c, "cores": threads, "kind": "port",
                            "sample": f"same rows, scalar C + OpenMP restatement (oracle/metal_logsoftmax.c), median of {n_c} passes"}
    except Exception as e:  # the C port is optional for the baseline
        log("cpu multicore baseline skipped:", e)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed GPU-busy time in front of every timed region (counter runs pass 0)")
    ap.add_argument("--clock-ms", type=float, default=CLOCK["ms"],
                    help="GPU-busy time of the clock pass after each matrix-core leg (0 = none; profiling runs pass 0)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default=None, help="comma-separated subset of: " + ", ".join(LEGS))
    ap.add_argument("--row-variant", choices=["both", "mask", "list", "all"], default="both",
                    help="time config 2 with its padding mask, with the valid rows as a packed list, without the mask, "
                         "or all three (profiling runs pick one)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, so a counter run can scale FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this path is measured on ONE GPU (rows are independent; more GPUs would each run "
            "this same kernel on their own share of the tokens). --gpus must be 1.")
        sys.exit(2)
    only = LEGS if args.only is None else [s for s in args.only.split(",") if s]
    for s in only:
        if s not in LEGS:
            log(f"bench.py: unknown leg {s!r}; choose from {LEGS}")
            sys.exit(2)

    import torch
    import tome_amd
    tome_amd.load_library()          # fail loudly if the HIP library was not built
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    log("device:", torch.cuda.get_device_name(dev))

    if args.calibrate_copy:   # known traffic: 2^30 bytes read + 2^30 bytes written per copy
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    K, W = args.steps, args.warmup
    SETTLE["ms"] = args.settle_ms
    CLOCK["ms"] = args.clock_ms
    legs = {}   # name -> JSON object; the first one present also becomes the top-level line

    def done(name):
        log(f"{name}: {legs[name]['ms_per_step'] * 1e3:.1f} us/step (median {legs[name]['median_ms'] * 1e3:.1f}), "
            f"roofline {legs[name]['roofline']['frac']:.3f}")
        torch.cuda.empty_cache()

    if "row" in only:
        row = bench_row(dev, K, W, args.row_variant)
        if "mask" in row:
            t = row["mask"]
            legs["headline"] = {
                "value": row["n_valid"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t),
                "dtype": "f32", "input_dtype": "bf16",
                "config": {"workload": "config 2: row log-softmax + target gather, bf16 logits [8x512, 151936], "
                                       "padding mask lengths~U[64,512], fp32 out",
                           "rows": row["rows"], "valid_rows": row["n_valid"], "vocab": V, "temperature": 1.0},
                "roofline": hbm_roofline(row["bytes_mask"], t["ms"], traffic_of("row_logprob_config2_masked"),
                                         "row_logprob_kernel<bf16>")}
            done("headline")
        if "list" in row:
            t = row["list"]
            legs["row_list"] = {
                "value": row["n_valid"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t),
                "dtype": "f32", "input_dtype": "bf16",
                "config": {"workload": "config 2 with the valid rows given as a packed row list instead of a mask "
                                       "(tome_row_logprob_rows): bf16 logits [8x512, 151936], lengths~U[64,512], packed fp32 out",
                           "rows": row["rows"], "valid_rows": row["n_valid"], "vocab": V, "temperature": 1.0},
                "roofline": hbm_roofline(row["bytes_mask"], t["ms"], traffic_of("row_logprob_config2_masked"),
                                         "row_logprob_kernel<bf16>")}
            done("row_list")
        if "all" in row:
            t = row["all"]
            legs["all_rows"] = {
                "value": row["rows"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t),
                "dtype": "f32", "input_dtype": "bf16",
                "config": {"workload": "config 2 without the padding mask: all 4096 rows of bf16 logits [4096, 151936] read",
                           "rows": row["rows"], "vocab": V, "temperature": 1.0},
                "roofline": hbm_roofline(row["bytes_all"], t["ms"], traffic_of("row_logprob_config2_all_rows"),
                                         "row_logprob_kernel<bf16>")}
            done("all_rows")
    if "entry" in only:
        for mode in ("logits", "hidden"):
            t = bench_ref_entry(dev, K, W, mode)
            name = "ref_entry" if mode == "logits" else "ref_entry_hidden_mode"
            what = ("the stub model's bf16 logits [32, max_len, 151936] are resident in HBM; tome_row_logprob_rows scores the completion rows"
                    if mode == "logits" else
                    "the stub model returns final hidden states [32, max_len, 1024]; the completion rows go through the fused lm_head kernel")
            roof = (hbm_roofline(t["bytes"], t["kernel_ms"], None, "row_logprob_kernel<bf16> over the scored rows, 8 launches") if mode == "logits"
                    else mfma_roofline(t["flop"], t["kernel_ms"], None, "fused_lmhead_dma_kernel, 8 launches"))
            roof["note"] = "priced on kernel_ms (the same launches without the entry around them), not on ms_per_step"
            legs[name] = {
                "value": t["tokens"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s at the entry (host clock, lists filled)",
                **timing_fields(t), "dtype": "f32", "input_dtype": "bf16",
                "config": {"workload": "RefLogprobServicer.process_ref_logprobs_batched (node.py:391-461) on config 2's batch: 32 prompts of 256 "
                                       "tokens x G=8 completions of U[64,512] tokens, max_ref_batch_size 32 (8 chunks per call); " + what,
                           "sequences": t["sequences"], "chunks": t["chunks"], "scored_tokens": t["tokens"], "vocab": V},
                "kernel_ms": t["kernel_ms"], "kernel_share_of_wall": t["kernel_ms"] / t["ms"],
                "host_us_per_chunk": t["host_us_per_chunk"], "wall_us_per_chunk": t["ms"] * 1e3 / t["chunks"],
                "roofline": roof}
            log(f"{name}: {t['ms']:.2f} ms per call ({t['chunks']} chunks, {t['tokens']} tokens), kernels {t['kernel_ms']:.2f} ms "
                f"= {t['kernel_ms'] / t['ms']:.2f} of the wall time, host {t['host_us_per_chunk']:.0f} us per chunk")
            torch.cuda.empty_cache()
    if "config1" in only:
        t = bench_config1(dev, K, W)
        legs["config1_row"] = {
            "value": t["rows"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t), "dtype": "f32",
            "config": {"workload": "config 1: row log-softmax + target gather, fp32 logits [64, 151936] ~N(0,2^2), "
                                   "uniform targets; 16 rotating input buffers (rows come from HBM)",
                       "rows": t["rows"], "vocab": V, "temperature": 1.0},
            "roofline": hbm_roofline(t["bytes"], t["ms"], traffic_of("row_logprob_config1"),
                                     "row_logprob_kernel<f32> (8 workgroups per row) + row_combine_kernel")}
        done("config1_row")
    if "fullmatrix" in only:
        shapes = {}
        for rows, dn in ((4096, "bf16"), (64, "f32")):
            t = bench_full_matrix(dev, K, W, rows, dn)
            shapes[f"{rows}x{V}_{dn}"] = {**timing_fields(t), "passes_over_the_matrix": t["passes_over_the_matrix"],
                                          **{k: t[k] for k in ("torch_mul_same_bytes_ms", "torch_log_softmax_ms") if k in t},
                                          "gbs_if_priced_on_three_passes": t["bytes_if_three_passes"] / (t["ms"] * 1e-3) / 1e9,
                                          "roofline": hbm_roofline(
                t["bytes"], t["ms"], traffic_of(f"full_log_softmax_{rows}rows_{dn}"),
                "full_log_softmax_onepass_kernel" if t["passes_over_the_matrix"] == 2 else
                "row_logprob_kernel (lse partials) + full_log_softmax_kernel")}
            log(f"full matrix {rows} x {V} {dn}: {t['ms'] * 1e3:.1f} us, {shapes[f'{rows}x{V}_{dn}']['roofline']['frac']:.3f} of HBM peak")
            torch.cuda.empty_cache()
        big = shapes[f"4096x{V}_bf16"]
        legs["full_log_softmax"] = {
            "value": 4096 * V / (big["ms_per_step"] * 1e-3), "unit": "log-probs written/s (4096 x 151936 bf16)",
            **{k: big[k] for k in ("ms_per_step", "median_ms", "min_ms", "settle_launches")}, "dtype": "f32", "input_dtype": "bf16",
            "config": {"workload": "tome_full_log_softmax, the drop-in of fused_log_softmax (model.py:77-89): the whole log-prob matrix in the "
                                   "input dtype; [4096, 151936] bf16 (one pass: the row stays in a workgroup's registers, 2 V sizeof(T) bytes per row) "
                                   "and [64, 151936] fp32 (the callers' dtype; two passes, 3 V sizeof(T) bytes per row; 16 rotating buffers)",
                       "shapes": shapes},
            "roofline": big["roofline"]}
        done("full_log_softmax")
    if "ceiling" in only:
        t = bench_ceiling(dev, K, W, "random")
        c = bench_ceiling(dev, K, W, "constant")
        q = bench_ceiling(dev, K, W, "random", with_requests=True)
        SUSTAINED["tflops"] = t["flop"] / (t["ms"] * 1e-3) / 1e12
        f = bench_ceiling(dev, K, W, "random", with_requests=True, with_fold=True, with_barrier=True)
        SUSTAINED["with_fill"] = q["flop"] / (q["ms"] * 1e-3) / 1e12
        SUSTAINED["with_fill_and_fold"] = f["flop"] / (f["ms"] * 1e-3) / 1e12
        legs["mfma_ceiling"] = {
            "value": SUSTAINED["tflops"], "unit": "TFLOP/s", **timing_fields(t), "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "bare LDS -> MFMA loop of the fused kernel (256x256 workgroup tile, v_mfma_f32_16x16x32_bf16, "
                                   "one workgroup per CU, operands resident in LDS): random operands as in config 3",
                       "workgroups": t["workgroups"], "k_slabs_per_launch": t["k_steps"],
                       "constant_operands_tflops": c["flop"] / (c["ms"] * 1e-3) / 1e12,
                       "constant_operands_sclk_mhz": c.get("sclk_mhz"),
                       "random_operands_with_fill_requests_tflops": q["flop"] / (q["ms"] * 1e-3) / 1e12,
                       "random_operands_with_fill_requests_sclk_mhz": q.get("sclk_mhz"),
                       "random_operands_with_fill_requests_softmax_fold_every_16_slabs_and_step_barrier_tflops": SUSTAINED["with_fill_and_fold"],
                       "random_operands_with_fill_requests_softmax_fold_every_16_slabs_and_step_barrier_sclk_mhz": f.get("sclk_mhz")},
            "roofline": mfma_roofline(t["flop"], t["ms"], None, "mfma_ceiling_kernel", t.get("sclk_mhz"))}
        legs["mfma_ceiling"]["roofline"].pop("sustained_peak", None)
        legs["mfma_ceiling"]["roofline"].pop("frac_of_sustained", None)
        legs["mfma_ceiling"]["roofline"].pop("sustained_peak_with_fill", None)
        legs["mfma_ceiling"]["roofline"].pop("frac_of_sustained_with_fill", None)
        done("mfma_ceiling")
    if "fused" in only:
        t = bench_fused(dev, K, W)
        legs["fused_lmhead"] = {
            "value": t["tokens"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t),
            "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "config 3: fused lm_head + log-softmax, hidden [4096,1024] x W [151936,1024] bf16",
                       "tokens": t["tokens"], "hidden": t["H"], "vocab": V, "temperature": 1.0},
            "roofline": mfma_roofline(t["flop"], t["ms"], traffic_of("fused_lmhead_config3"), "fused_lmhead_dma_kernel", t.get("sclk_mhz"))}
        if SUSTAINED["with_fill_and_fold"]:   # the probe with fill requests, a softmax fold per 16 slabs and the step barrier:
            r = legs["fused_lmhead"]["roofline"]   # this design at K = 1024 on a memory system that always answers from cache
            r["design_ceiling"] = SUSTAINED["with_fill_and_fold"]
            r["frac_of_design_ceiling"] = r["achieved"] / r["design_ceiling"]
        done("fused_lmhead")
    if "norm" in only:
        t = bench_norm_lmhead(dev, K, W)
        legs["norm_lmhead"] = {
            "value": t["valid"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t), "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "tome_norm_lmhead_logprob (model.py:536-538): final RMSNorm + lm_head + log-softmax, pre-norm hidden "
                                   "[8x512, 1024] x W [151936, 1024] bf16 with config 2's padding mask (lengths~U[64,512]); FLOP on valid tokens",
                       "tokens": t["tokens"], "valid_tokens": t["valid"], "hidden": t["H"], "vocab": V},
            "roofline": mfma_roofline(t["flop"], t["ms"], traffic_of("norm_lmhead_config3_masked"),
                                      "compact_rows + rmsnorm_rows + fused_lmhead_dma_kernel + combine", t.get("sclk_mhz"))}
        done("norm_lmhead")
    if "gemm" in only:
        t = bench_library_gemm(dev, K, W)
        legs["library_gemm_config3"] = {
            "value": t["flop"] / (t["ms"] * 1e-3) / 1e12, "unit": "TFLOP/s", **timing_fields(t), "dtype": "bf16 x bf16 -> bf16",
            "config": {"workload": "for scale, not part of the path: torch.mm (vendor GEMM library) on config 3's shape, bf16 logits "
                                   "[4096, 151936] written, no softmax", "tokens": t["tokens"], "hidden": t["H"], "vocab": V},
            "roofline": mfma_roofline(t["flop"], t["ms"], None, "vendor library GEMM (hipBLASLt / rocBLAS via torch.mm)", t.get("sclk_mhz"))}
        done("library_gemm_config3")
        t = bench_library_gemm(dev, K, W, n=8192, H=8192, vocab=8192)
        legs["library_gemm_square_8192"] = {
            "value": t["flop"] / (t["ms"] * 1e-3) / 1e12, "unit": "TFLOP/s", **timing_fields(t), "dtype": "bf16 x bf16 -> bf16",
            "config": {"workload": "for scale, not part of the path: torch.mm (vendor GEMM library) on 8192 x 8192 x 8192, random "
                                   "operands", "m": 8192, "n": 8192, "k": 8192},
            "roofline": mfma_roofline(t["flop"], t["ms"], None, "vendor library GEMM (hipBLASLt / rocBLAS via torch.mm)", t.get("sclk_mhz"))}
        done("library_gemm_square_8192")
    if "config4" in only:
        t = bench_fused(dev, K, W, n=16 * 1024, H=2560, temperature=0.7, lengths=(16, 1024, 128, 1024), seed=444)
        legs["config4_fused_varlen"] = {
            "value": t["valid"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t),
            "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "config 4: fused lm_head + log-softmax, hidden [16x1024, 2560] x W [151936, 2560] bf16, "
                                   "temperature 0.7, sequence lengths~U[128,1024] as a padding mask (FLOP counted on valid tokens)",
                       "tokens": t["tokens"], "valid_tokens": t["valid"], "hidden": t["H"], "vocab": V, "temperature": 0.7},
            "roofline": mfma_roofline(t["flop"], t["ms"], traffic_of("fused_lmhead_config4"), "fused_lmhead_dma_kernel", t.get("sclk_mhz"))}
        done("config4_fused_varlen")
    if "config5" in only:
        t = bench_dual(dev, max(3, K // 4), max(1, W // 4))     # 0.1 s per step: a quarter of the steps
        legs["config5_grpo_dual"] = {
            "value": t["tokens"] / (t["ms"] * 1e-3), "unit": "tokens/s (lp, ref_lp, k3, entropy each)", **timing_fields(t),
            "steps": max(3, K // 4), "warmup": max(1, W // 4), "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "config 5: GRPO policy + reference dual pass, hidden [32x2048, 4096] x two W [151936, 4096] bf16 "
                                   "(ref = policy + N(0, 0.002^2)); outputs lp, ref_lp, k3, entropy",
                       "tokens": t["tokens"], "hidden": t["H"], "vocab": V, "temperature": 1.0},
            "roofline": mfma_roofline(t["flop"], t["ms"], traffic_of("grpo_dual_config5"),
                                      "fused_lmhead_dma_kernel (two sweeps) + fused_combine_kernel", t.get("sclk_mhz"))}
        done("config5_grpo_dual")
    if "pair" in only:
        t = bench_pair(dev, K, W)
        legs["grpo_pair"] = {
            "value": t["tokens"] / (t["ms"] * 1e-3), "unit": "tokens/s (lp, ref_lp, k3, entropy each)", **timing_fields(t),
            "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "tome_grpo_pair (node.py:65-66, 443): policy and reference hidden states [8192, 4096] each, one shared "
                                   "W [151936, 4096] bf16; outputs lp, ref_lp, k3, entropy",
                       "tokens": t["tokens"], "hidden": t["H"], "vocab": V, "temperature": 1.0},
            "roofline": mfma_roofline(t["flop"], t["ms"], traffic_of("grpo_pair_8192x4096"),
                                      "fused_lmhead_dma_kernel (two sweeps) + fused_combine_kernel", t.get("sclk_mhz"))}
        done("grpo_pair")
    if "small" in only:
        t = bench_fused(dev, K, W, n=64)
        # the streaming kernel's own shapes: up to 16 tokens at H = 1024, up to 64 at larger hidden sizes
        stream = {}
        for n, H in ((16, 1024), (64, 2048)):
            u = bench_fused(dev, K, W, n=n, H=H, seed=2000 + n + H)
            stream[f"{n}x{H}"] = {**timing_fields(u),
                                  "roofline": hbm_roofline(u["bytes"], u["ms"], None, "fused_lmhead_small_kernel + fused_combine_kernel")}
            log(f"streaming kernel {n}x{H}: {u['ms'] * 1e3:.1f} us, {stream[f'{n}x{H}']['roofline']['frac']:.3f} of HBM peak")
            torch.cuda.empty_cache()
        legs["fused_lmhead_decode_batch"] = {
            "value": t["tokens"] / (t["ms"] * 1e-3), "unit": "token-logprobs/s", **timing_fields(t),
            "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "fused lm_head + log-softmax at a decode-step batch: hidden [64,1024] x W [151936,1024] bf16 "
                                   "(the tiled kernel's 64-token tile, W requested non-temporally); `streaming_kernel_shapes`: the "
                                   "kernel that splits K over the waves, on shapes it serves",
                       "tokens": t["tokens"], "hidden": t["H"], "vocab": V, "streaming_kernel_shapes": stream},
            "roofline": hbm_roofline(t["bytes"], t["ms"], traffic_of("fused_lmhead_decode_64tokens"),
                                     "fused_lmhead_dma_kernel<64-token tile> + fused_combine_kernel")}
        done("fused_lmhead_decode_batch")
    if "midsize" in only:   # batches of up to one token tile: W streams once, HBM-bound
        mid = {}
        for n, H in ((160, 1024), (256, 1024), (64, 4096), (128, 4096)):
            t = bench_fused(dev, K, W, n=n, H=H, seed=1000 + n + H)
            mid[f"{n}x{H}"] = {**timing_fields(t),
                               "roofline": hbm_roofline(t["bytes"], t["ms"], None, "fused lm_head sweep + combine")}
            log(f"midsize {n}x{H}: {t['ms'] * 1e3:.1f} us, {mid[f'{n}x{H}']['roofline']['frac']:.3f} of HBM peak")
            torch.cuda.empty_cache()
        worst = min(mid.values(), key=lambda d: d["roofline"]["frac"])
        legs["fused_lmhead_small_batches"] = {
            "value": worst["roofline"]["achieved"], "unit": "GB/s (lowest of the shapes)",
            **{k: worst[k] for k in ("ms_per_step", "median_ms", "min_ms", "settle_launches")},
            "dtype": "bf16 x bf16 -> f32",
            "config": {"workload": "fused lm_head + log-softmax where W streams once: tokens x hidden in {160x1024, 256x1024, "
                                   "64x4096, 128x4096}, V = 151936", "shapes": mid},
            "roofline": worst["roofline"]}
    if "decode" in only:
        t = bench_decode(dev, K, W)
        legs["decode_sampler"] = {
            "value": t["rows"] / (t["ms"] * 1e-3), "unit": "sampled tokens/s", **timing_fields(t), "dtype": "f32",
            "config": {"workload": "one decode step: top-k sampling + log-prob + argmax, "
                                   "fp32 logits [64, 151936] (config 1's shape), top_k 20",
                       "rows": t["rows"], "top_k": t["top_k"], "vocab": V},
            "roofline": hbm_roofline(t["bytes"], t["ms"], traffic_of("row_sample_decode_64rows"),
                                     "row_sample_kernel<f32> + row_sample_combine_kernel")}
        done("decode_sampler")
    if "lora" in only:
        t = bench_lora(dev, K, W)
        legs["lora_merge"] = {
            "value": t["jobs"] / (t["ms"] * 1e-3), "unit": "weight matrices merged/s", **timing_fields(t), "dtype": "bf16",
            "config": {"workload": "UpdateWeights at Qwen3-0.6B's shape: 28 layers x (qkv, gate_up, down), LoRA rank 8",
                       "matrices": t["jobs"], "rank": t["rank"]},
            "roofline": hbm_roofline(t["bytes"], t["ms"], traffic_of("lora_merge_qwen3_0.6b"), "lora_merge_kernel<1>")}
        done("lora_merge")
    cpu = None if args.no_cpu else cpu_baseline()

    line = {
        "metric": "token-logprobs/sec + % HBM/MFMA peak at V=151936, Qwen3-0.6B shape",
        "n_gpus": 1, "steps": K, "warmup": W,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic",
    }
    first = next(iter(legs))
    line.update(legs[first])                 # headline = config 2 with its mask, unless --only left it out
    line["unit"] = legs[first]["unit"]
    for name, obj in legs.items():
        if name != first:
            line[name] = obj
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
