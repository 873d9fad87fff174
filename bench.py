#!/usr/bin/env python3
"""Benchmark of the token-log-prob path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM.  The headline workload is benchmark configuration 2 (the Qwen3-0.6B GRPO
ref-logprob shape: bf16 logits [8 x 512, 151936] with a padding mask); the same JSON line
also carries the unmasked variant, the fused lm_head + log-softmax kernel at configuration 3
(4096 tokens) and at a decode-step batch (64 tokens), one decode step's sampler, and the LoRA
merge of one UpdateWeights request.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only row|fused|small|decode|lora]

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
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
# HBM-side bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE counter passes, each scaled by the same
# counter's reading for a plain 2^30-byte copy (profiles/hbm_traffic_counters.txt).  The masked figure
# belongs to the seeded lengths of make_config2 (2356 valid rows).
TRAFFIC_ROW_MASKED = 716.4e6 + 0.13e6
TRAFFIC_ROW_ALL = 1245.0e6 + 0.13e6
TRAFFIC_FUSED_CFG3 = 1847e6 + 6.8e6
TRAFFIC_DECODE_64 = 39.2e6 + 0.30e6 + 0.23e6   # sampler: main-kernel fetch, combine fetch, partials written
TRAFFIC_FUSED_SMALL_64 = 326.0e6 + 0.52e6      # sweep kernel: fetch + partials written (profiles/fused_lmhead_small_kernel_decode_64tokens.txt)
TRAFFIC_LORA_06B = 812.1e6 + 763.4e6            # merge kernel: fetch + write (profiles/lora_merge_kernel_qwen3_0.6b_update.txt)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


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


def time_steps(fn, steps, warmup):
    """Average milliseconds per step over `steps` back-to-back launches, by HIP events recorded on
    the stream the kernels run on (torch's current stream, which the library launches into)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall_ms


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

    # correctness gate on what is being timed: spike rows must score the closed form's ballpark
    step(True)
    torch.cuda.synchronize()
    got = lp.clone()
    assert torch.isfinite(got).all() and (got <= 1e-5).all()
    assert (got[valid == 0] == 0).all()

    ms_mask, wall_mask = time_steps(lambda: step(True), steps, warmup) if variant in ("both", "mask") else (float("nan"),) * 2
    ms_all, wall_all = time_steps(lambda: step(False), steps, warmup) if variant in ("both", "all") else (float("nan"),) * 2
    bytes_mask = n_valid * V * 2
    bytes_all = rows * V * 2
    out = {
        "n_valid": n_valid, "rows": rows,
        "ms_mask": ms_mask, "ms_all": ms_all, "wall_ms_mask": wall_mask,
        "gbs_mask": bytes_mask / (ms_mask * 1e-3) / 1e9, "gbs_all": bytes_all / (ms_all * 1e-3) / 1e9,
        "bytes_mask": bytes_mask, "bytes_all": bytes_all,
    }
    del logits, flat
    torch.cuda.empty_cache()
    return out


def bench_fused(dev, steps, warmup, n=4096, H=1024):
    """Fused lm_head + log-softmax on [n, H] x [V, H]: config 3 by default; n = 64 is the decode-step batch,
    where W is streamed once and the kernel is HBM-bound."""
    import torch
    import tome_amd
    from tome_amd import _lib
    lib = tome_amd.load_library()
    g = torch.Generator(device=dev).manual_seed(4321)
    hidden = torch.randn((n, H), device=dev, generator=g).to(torch.bfloat16)
    weight = (torch.randn((V, H), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    targets = torch.randint(0, V, (n,), device=dev, generator=g).to(torch.int32)
    lp = torch.empty(n, dtype=torch.float32, device=dev)
    ws_bytes = lib.tome_fused_lmhead_logprob_workspace(n, H, V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def step():
        _lib.check(lib.tome_fused_lmhead_logprob(hidden.data_ptr(), weight.data_ptr(), n, H, V, H, H,
                                                 targets.data_ptr(), None, 1.0, lp.data_ptr(), None, None, None,
                                                 ws.data_ptr(), ws_bytes, stream))
    step()
    torch.cuda.synchronize()
    assert torch.isfinite(lp).all() and (lp <= 1e-5).all()
    ms, wall = time_steps(step, steps, warmup)
    flop = 2.0 * n * H * V
    return {"tokens": n, "H": H, "ms": ms, "wall_ms": wall, "tflops": flop / (ms * 1e-3) / 1e12, "flop": flop}


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
    ms, wall = time_steps(step, steps, warmup)
    return {"rows": rows, "top_k": k, "ms": ms, "bytes": rows * V * 4}


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
    ms, wall = time_steps(step, steps, warmup)
    return {"ms": ms, "wall_ms": wall, "bytes": n_bytes, "jobs": len(jobs), "rank": rank}


def cpu_baseline(sample_rows=1024, budget_s=12.0):
    """NumPy fp32 restatement of local_compute_logprobs (mlx-impl/node.py:400-404) on a bounded
    sample of the config-2 workload: `sample_rows` rows of bf16 logits, upcast included."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(99)
    x = (rng.standard_normal((sample_rows, V)) * 3.0).astype(np.float32)
    t = rng.integers(0, V, size=sample_rows).astype(np.int32)
    x[np.arange(sample_rows), t] += 15.0
    bits = oracle.bf16_round(x)
    oracle.local_compute_logprobs_f32(bits[:8], t[:8], 1.0)   # warm-up
    times = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end and len(times) < 40:
        t0 = time.perf_counter()
        oracle.local_compute_logprobs_f32(bits, t, 1.0)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    out = {"value": sample_rows / med, "unit": "token-logprobs/s", "cores": 1, "kind": "port",
           "sample": f"{sample_rows} rows x {V} bf16 logits (config-2 distribution), NumPy fp32 restatement of "
                     f"node.py:400-404, median of {len(times)} passes"}
    # multi-core figure: the same arithmetic in scalar C with OpenMP over rows
    try:
        from oracle import cport
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        cport.local_compute_logprobs_c(bits[:8], t[:8], 1.0)
        ts = []
        for _ in range(10):
            t0 = time.perf_counter()
            cport.local_compute_logprobs_c(bits, t, 1.0)
            ts.append(time.perf_counter() - t0)
        out["multicore"] = {"value": sample_rows / min(ts), "cores": threads, "kind": "port",
                            "sample": "same rows, scalar C + OpenMP restatement (oracle/metal_logsoftmax.c)"}
    except Exception as e:  # the C port is optional for the baseline
        log("cpu multicore baseline skipped:", e)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", choices=["row", "fused", "small", "decode", "lora"], default=None)
    ap.add_argument("--row-variant", choices=["both", "mask", "all"], default="both",
                    help="time config 2 with its padding mask, without it, or both (profiling runs pick one)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, so a counter run can scale FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this path is measured on ONE GPU (rows are independent; more GPUs would each run "
            "this same kernel on their own share of the tokens). --gpus must be 1.")
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
    row = bench_row(dev, args.steps, args.warmup, args.row_variant) if args.only in (None, "row") else None
    # the fused step is ~10x longer than a row step: half the launches keep the run short; the clocks
    # still settle (a few tens of milliseconds of back-to-back launches are needed for that)
    fused = bench_fused(dev, max(5, args.steps // 2), max(2, args.warmup // 2)) if args.only in (None, "fused") else None
    small = bench_fused(dev, args.steps, args.warmup, n=64) if args.only in (None, "small") else None
    decode = bench_decode(dev, args.steps, args.warmup) if args.only in (None, "decode") else None
    lora = bench_lora(dev, max(5, args.steps // 4), max(2, args.warmup // 4)) if args.only in (None, "lora") else None
    cpu = None if args.no_cpu else cpu_baseline()

    line = {
        "metric": "token-logprobs/sec + % HBM/MFMA peak at V=151936, Qwen3-0.6B shape",
        "unit": "token-logprobs/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "data": "synthetic", "dtype": "f32",
    }
    if row is not None and args.row_variant == "all":
        row["ms_mask"], row["gbs_mask"], row["bytes_mask"], row["n_valid"] = (row["ms_all"], row["gbs_all"],
                                                                              row["bytes_all"], row["rows"])
    if row is not None:
        line.update({
            "value": row["n_valid"] / (row["ms_mask"] * 1e-3),
            "ms_per_step": row["ms_mask"],
            "config": {"workload": "config 2: row log-softmax + target gather, bf16 logits [8x512, 151936], "
                                   "padding mask lengths~U[64,512], fp32 out",
                       "rows": row["rows"], "valid_rows": row["n_valid"], "vocab": V, "temperature": 1.0},
            "roofline": {"bound": "hbm", "achieved": row["gbs_mask"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": row["gbs_mask"] / HBM_PEAK_GBS,
                         "traffic": TRAFFIC_ROW_ALL if args.row_variant == "all" else TRAFFIC_ROW_MASKED,
                         "kernel": "row_logprob_kernel<bf16>", "bytes_per_launch": row["bytes_mask"]},
        })
        if args.row_variant == "all":
            line["config"]["workload"] = line["config"]["workload"].replace(
                "padding mask lengths~U[64,512]", "padding mask NOT applied (all 4096 rows read)")
        if args.row_variant == "both":
            line["all_rows"] = {"value": row["rows"] / (row["ms_all"] * 1e-3), "ms_per_step": row["ms_all"],
                                "config": {"workload": "config 2 without the padding mask: all 4096 rows read"},
                                "roofline": {"bound": "hbm", "achieved": row["gbs_all"], "peak": HBM_PEAK_GBS,
                                             "unit": "GB/s", "frac": row["gbs_all"] / HBM_PEAK_GBS, "traffic": TRAFFIC_ROW_ALL,
                                             "bytes_per_launch": row["bytes_all"]}}
    if fused is not None:
        f = {"value": fused["tokens"] / (fused["ms"] * 1e-3), "unit": "token-logprobs/s", "ms_per_step": fused["ms"],
             "dtype": "bf16 x bf16 -> f32",
             "config": {"workload": "config 3: fused lm_head + log-softmax, hidden [4096,1024] x W [151936,1024] bf16",
                        "tokens": fused["tokens"], "hidden": fused["H"], "vocab": V},
             "roofline": {"bound": "mfma", "achieved": fused["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                          "unit": "TFLOP/s", "frac": fused["tflops"] / MFMA_BF16_PEAK_TFLOPS, "traffic": TRAFFIC_FUSED_CFG3,
                          "kernel": "fused_lmhead_dma_kernel", "flop_per_launch": fused["flop"]}}
        if row is None:
            line.update({"value": f["value"], "ms_per_step": f["ms_per_step"], "config": f["config"],
                         "roofline": f["roofline"], "dtype": "f32"})
        else:
            line["fused_lmhead"] = f
    if small is not None:
        nbytes = V * small["H"] * 2 + small["tokens"] * small["H"] * 2
        gbs = nbytes / (small["ms"] * 1e-3) / 1e9
        d = {"value": small["tokens"] / (small["ms"] * 1e-3), "unit": "token-logprobs/s", "ms_per_step": small["ms"],
             "dtype": "bf16 x bf16 -> f32",
             "config": {"workload": "fused lm_head + log-softmax at a decode-step batch: hidden [64,1024] x W [151936,1024] bf16",
                        "tokens": small["tokens"], "hidden": small["H"], "vocab": V},
             "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                          "traffic": TRAFFIC_FUSED_SMALL_64, "kernel": "fused_lmhead_small_kernel", "bytes_per_launch": nbytes}}
        if row is None and fused is None:
            line.update({"value": d["value"], "unit": d["unit"], "ms_per_step": d["ms_per_step"], "config": d["config"],
                         "roofline": d["roofline"]})
        else:
            line["fused_lmhead_decode_batch"] = d
    if decode is not None:
        gbs = decode["bytes"] / (decode["ms"] * 1e-3) / 1e9
        d = {"value": decode["rows"] / (decode["ms"] * 1e-3), "unit": "sampled tokens/s",
             "ms_per_step": decode["ms"], "dtype": "f32",
             "config": {"workload": "one decode step: top-k sampling + log-prob + argmax, "
                                    "fp32 logits [64, 151936] (config 1's shape), top_k 20",
                        "rows": decode["rows"], "top_k": decode["top_k"], "vocab": V},
             "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": gbs / HBM_PEAK_GBS, "traffic": TRAFFIC_DECODE_64,
                          "kernel": "row_sample_kernel<f32> + row_sample_combine_kernel",
                          "bytes_per_launch": decode["bytes"]}}
        if row is None and fused is None:
            line.update({"value": d["value"], "unit": d["unit"], "ms_per_step": d["ms_per_step"], "config": d["config"],
                         "roofline": d["roofline"]})
        else:
            line["decode_sampler"] = d
    if lora is not None:
        gbs = lora["bytes"] / (lora["ms"] * 1e-3) / 1e9
        d = {"value": lora["jobs"] / (lora["ms"] * 1e-3), "unit": "weight matrices merged/s", "ms_per_step": lora["ms"],
             "dtype": "bf16",
             "config": {"workload": "UpdateWeights at Qwen3-0.6B's shape: 28 layers x (qkv, gate_up, down), LoRA rank 8",
                        "matrices": lora["jobs"], "rank": lora["rank"]},
             "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                          "traffic": TRAFFIC_LORA_06B, "kernel": "lora_merge_kernel<1>", "bytes_per_launch": lora["bytes"]}}
        if row is None and fused is None and decode is None:
            line.update({"value": d["value"], "unit": d["unit"], "ms_per_step": d["ms_per_step"], "config": d["config"],
                         "roofline": d["roofline"], "dtype": "bf16"})
        else:
            line["lora_merge"] = d
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
