"""Writes tests/golden/lora_golden.npz: inputs and expected outputs of the LoRA merge of UpdateWeights
(mlx-impl/node.py:128,137): out = bf16(base + bf16(bf16(scale) * bf16(lora_B @ lora_A))).

The reference holds no stored vectors for it and cannot be imported here (MLX missing), so the expected
bit patterns come from a route that shares no code with oracle/: exact rational arithmetic
(fractions.Fraction) for the product, the scaling and the sum, and a round-to-nearest-even to bf16 that
compares exact distances to the neighbouring bf16 values.  WHERE the reference rounds (after the matmul,
after the scalar multiply with the scalar cast to bf16 first, after the add) is MLX's published behaviour
for bf16 arrays and Python scalars; these vectors pin the arithmetic given those three roundings.

Run from the repo root:  python tests/golden/make_lora_golden.py
"""
import os
from fractions import Fraction

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def bits_of(x32: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(x32, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def value_of(bits: int) -> Fraction:
    return Fraction(float(torch.tensor([bits], dtype=torch.int32).to(torch.int16).view(torch.bfloat16).to(torch.float64)[0]))


def round_bf16(fr: Fraction) -> int:
    """Nearest bf16 bit pattern to an exact rational, ties to the even pattern."""
    if fr == 0:
        return 0
    near = int(torch.tensor([float(fr)], dtype=torch.float64).to(torch.bfloat16).view(torch.int16)[0]) & 0xFFFF
    best = None
    for cand in (near - 1, near, near + 1):
        cand &= 0xFFFF
        if (cand & 0x7F80) == 0x7F80:          # inf / nan patterns are never the answer here
            continue
        key = (abs(value_of(cand) - fr), cand & 1)
        if best is None or key < best[0]:
            best = (key, cand)
    return best[1]


def merge(base, a, b, scale):
    rows, cols = base.shape
    rank = a.shape[0]
    s = value_of(round_bf16(Fraction(float(np.float32(scale)))))
    out = np.zeros((rows, cols), dtype=np.uint16)
    for i in range(rows):
        for j in range(cols):
            d = sum((value_of(int(b[i, k])) * value_of(int(a[k, j])) for k in range(rank)), Fraction(0))
            d = value_of(round_bf16(d))
            d2 = value_of(round_bf16(s * d))
            out[i, j] = round_bf16(value_of(int(base[i, j])) + d2)
    return out


def main():
    rng = np.random.default_rng(20260304)
    out = {}
    for name, rows, cols, rank, scale, sb, sl in [("m0", 6, 16, 8, 2.5, 0.05, 0.1), ("m1", 5, 24, 12, 2.51, 0.02, 0.3),
                                                  ("m2", 9, 8, 16, -0.3, 1.0, 1.0), ("m3", 4, 32, 4, 1.0, 0.001, 0.05)]:
        base = bits_of(rng.standard_normal((rows, cols)) * sb)
        a = bits_of(rng.standard_normal((rank, cols)) * sl)
        b = bits_of(rng.standard_normal((rows, rank)) * sl)
        out.update({f"{name}_base": base, f"{name}_a": a, f"{name}_b": b, f"{name}_scale": np.float64(scale),
                    f"{name}_out": merge(base, a, b, scale)})
    np.savez_compressed(os.path.join(HERE, "lora_golden.npz"), **out)
    print("wrote lora_golden.npz:", sorted(out))


if __name__ == "__main__":
    main()
