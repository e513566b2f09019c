"""Writes tests/golden/cats_mlp_small.npz: small seeded CATS MLP cases with the outputs of the C oracle.

Provenance: the reference ships no golden vectors for this path (its own test file prints and saves, it asserts
nothing), so these are NOT reference outputs.  They are the CPU oracle's outputs, frozen: a regression anchor that
catches an accidental change of the oracle's arithmetic or rounding points, and a fixed set of vectors for the GPU
kernels.  What pins the oracle itself are the closed-form and brute-force checks in tests/test_oracle.py.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import cats_oracle as oracle  # noqa: E402
from tests.util import make_mlp  # noqa: E402

CASES = [  # name, H, I, B, dtype, quantile of |a| used as threshold
    ("f16_b1", 64, 96, 1, torch.float16, 0.5),
    ("f16_b3", 72, 100, 3, torch.float16, 0.7),
    ("bf16_b2", 64, 96, 2, torch.bfloat16, 0.5),
    ("f32_b2", 64, 40, 2, torch.float32, 0.3),
]


def bits(t: torch.Tensor) -> np.ndarray:
    """Storage bits as unsigned integers (npz has no bfloat16)."""
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32).numpy().astype(np.uint32)
    return t.contiguous().view(torch.int16).numpy().astype(np.uint16)


def main():
    oracle.build()
    out = {}
    for name, H, I, B, dtype, q in CASES:
        m = make_mlp(H, I, B, dtype, seed=1000 + H + I + B)
        a_abs = oracle.c_gate(m["x"], m["wg"], -1.0)[0].float().abs().flatten()
        t = float(torch.quantile(a_abs, q))
        ref = oracle.c_mlp(m["x"], m["wg"], m["wu"], m["wd"], t)
        for k in ("x", "wg", "wu", "wd"):
            out[f"{name}/{k}"] = bits(m[k])
        out[f"{name}/t"] = np.float64(t)
        out[f"{name}/a"] = bits(ref["a"])
        out[f"{name}/flag"] = ref["flag"].numpy().astype(np.uint8)
        out[f"{name}/y"] = bits(ref["y"])
    path = Path(__file__).resolve().parent / "cats_mlp_small.npz"
    np.savez_compressed(path, **out)
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
