"""Loads tests/golden/logprob_golden.npz and rebuilds the seeded full-vocabulary inputs."""
import os

import numpy as np

import oracle

V_QWEN3 = 151936
_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "logprob_golden.npz")


def load():
    return np.load(_PATH, allow_pickle=False)


def seeded_case(g, name):
    """(x, targets, T, expected dict) for the cases stored as a seed (see make_golden.py)."""
    seed, rows, scale = int(g[f"{name}_seed"]), int(g[f"{name}_rows"]), float(g[f"{name}_scale"])
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows, V_QWEN3)) * scale).astype(np.float32)
    t = rng.integers(0, V_QWEN3, size=rows).astype(np.int32)
    if bool(g[f"{name}_bf16"]):
        x[np.arange(rows), t] += 15
        x = oracle.bf16_round(x)
    exp = {k: g[f"{name}_{k}"] for k in ("lp", "lse", "ent", "argmax")}
    return x, t, float(g[f"{name}_T"]), exp
