"""Writes tests/golden/logprob_golden.npz: inputs and expected outputs for the token-log-prob path.

The reference holds no stored vectors for this path (its would-be goldens, test_inputs/*.npy, are
git-ignored and absent; mlx-impl/tests/test_components.py:46-55) and its Python cannot be imported
here (MLX missing), so the expected values are produced by routines that share no code with
oracle/: math.fsum brute force for small rows and torch.float64 log_softmax / matmul (library
routines) for the rest.  Large inputs are regenerated from the stored seed with
numpy.random.default_rng (PCG64), small ones are stored whole.

Run from the repo root:  python tests/golden/make_golden.py
"""
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
V_QWEN3 = 151936


def bf16_bits(x32: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(x32, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def bits_to_f64(b: np.ndarray) -> np.ndarray:
    return torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16).to(torch.float64).numpy()


def brute_row(row, t, T):
    z = [float(v) / T for v in row]
    m = max(z)
    e = [math.exp(v - m) for v in z]
    s = math.fsum(e)
    lse = m + math.log(s)
    ent = lse - math.fsum(ei * zi for ei, zi in zip(e, z)) / s
    return z[t] - lse, lse, ent


def torch_rows(x64: np.ndarray, t: np.ndarray, T: float):
    z = torch.from_numpy(x64) / T
    ls = torch.log_softmax(z, dim=-1)
    lp = ls.gather(-1, torch.from_numpy(t.astype(np.int64))[:, None])[:, 0]
    lse = torch.logsumexp(z, dim=-1)
    ent = -(ls.exp() * ls).sum(-1)
    return lp.numpy(), lse.numpy(), ent.numpy(), z.argmax(-1).numpy().astype(np.int32)


def main():
    out = {}
    rng = np.random.default_rng(20260303)
    # small fp32 rows, brute force; V chosen around the reference kernel's block/tail sizes scaled down
    for name, rows, V, T in [("s0", 4, 16, 1.0), ("s1", 3, 37, 0.7), ("s2", 2, 513, 1.5)]:
        x = (rng.standard_normal((rows, V)) * 2).astype(np.float32)
        t = rng.integers(0, V, size=rows).astype(np.int32)
        res = np.array([brute_row(x[r], int(t[r]), T) for r in range(rows)])
        out.update({f"{name}_x": x, f"{name}_t": t, f"{name}_T": np.float64(T), f"{name}_lp": res[:, 0],
                    f"{name}_lse": res[:, 1], f"{name}_ent": res[:, 2]})
    # bf16 rows with a +15 spike (config-2 distribution), stored whole, torch.float64 expected
    x = (rng.standard_normal((6, 4104)) * 3).astype(np.float32)
    spike = rng.integers(0, 4104, size=6)
    x[np.arange(6), spike] += 15
    b = bf16_bits(x)
    t = np.where(rng.random(6) < 0.5, spike, rng.integers(0, 4104, size=6)).astype(np.int32)
    lp, lse, ent, am = torch_rows(bits_to_f64(b), t, 1.0)
    out.update({"b0_bits": b, "b0_t": t, "b0_T": np.float64(1.0), "b0_lp": lp, "b0_lse": lse, "b0_ent": ent, "b0_argmax": am})
    # full-vocabulary rows regenerated from a seed (config 1: fp32 N(0, 2^2); config 2: bf16 N(0, 3^2) + spike)
    for name, seed, rows, scale, T, as_bf16 in [("c1", 101, 4, 2.0, 1.0, False), ("c2", 202, 4, 3.0, 1.0, True),
                                                 ("c2t", 303, 3, 3.0, 0.7, True)]:
        g = np.random.default_rng(seed)
        x = (g.standard_normal((rows, V_QWEN3)) * scale).astype(np.float32)
        t = g.integers(0, V_QWEN3, size=rows).astype(np.int32)
        if as_bf16:
            x[np.arange(rows), t] += 15
            x64 = bits_to_f64(bf16_bits(x))
        else:
            x64 = x.astype(np.float64)
        lp, lse, ent, am = torch_rows(x64, t, T)
        out.update({f"{name}_seed": np.int64(seed), f"{name}_rows": np.int64(rows), f"{name}_scale": np.float64(scale),
                    f"{name}_T": np.float64(T), f"{name}_bf16": np.bool_(as_bf16), f"{name}_lp": lp, f"{name}_lse": lse,
                    f"{name}_ent": ent, f"{name}_argmax": am})
    # lm_head: bf16 hidden / weight stored whole, torch.float64 matmul
    n, H, V, T = 24, 64, 300, 0.9
    h = bf16_bits(rng.standard_normal((n, H)).astype(np.float32))
    w = bf16_bits((rng.standard_normal((V, H)) * 0.3).astype(np.float32))
    t = rng.integers(0, V, size=n).astype(np.int32)
    logits = torch.from_numpy(bits_to_f64(h)) @ torch.from_numpy(bits_to_f64(w)).T
    lp, lse, ent, am = torch_rows(logits.numpy(), t, T)
    out.update({"f0_h": h, "f0_w": w, "f0_t": t, "f0_T": np.float64(T), "f0_lp": lp, "f0_lse": lse, "f0_ent": ent,
                "f0_argmax": am})
    np.savez_compressed(os.path.join(HERE, "logprob_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "logprob_golden.npz"))


if __name__ == "__main__":
    main()
