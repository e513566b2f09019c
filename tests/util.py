"""Shared recipes for the parity tests: seeded synthetic MLPs in the shapes and distributions the benchmark
configurations name, threshold calibration, and the tolerances the parity bar states."""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

# output tolerance vs the dense-masked reference formula
TOL = {
    torch.float16: dict(rtol=1e-2, atol=2e-3),
    torch.bfloat16: dict(rtol=1e-2, atol=2e-3),
    torch.float32: dict(rtol=1e-5, atol=1e-5),
}
# tolerance on the activation a itself: one rounding step of the storage type plus accumulation-order noise
A_TOL = {
    torch.float16: dict(rtol=2e-3, atol=1e-4),
    torch.bfloat16: dict(rtol=1.6e-2, atol=1e-3),
    torch.float32: dict(rtol=1e-5, atol=1e-6),
}


def make_mlp(H, I, B, dtype, seed, dist="normal", heavy_tail=False, corr=0.0):
    """Weights and inputs on the CPU.

    dist "normal": W ~ N(0, 0.02^2), x ~ N(0, 1) (benchmark configs);  "uniform": everything U(-0.5, 0.5)
    (the reference's own test recipe, flash_gemv/test/test_fuse_gemv_cmp.py:173-187).
    heavy_tail: gate rows scaled by exp(N(0, 0.5^2)).  corr: pairwise correlation between the B rows of x.
    """
    g = torch.Generator().manual_seed(seed)
    if dist == "normal":
        wg = torch.randn(I, H, generator=g) * 0.02
        wu = torch.randn(I, H, generator=g) * 0.02
        wd = torch.randn(H, I, generator=g) * 0.02
        if corr > 0:
            common = torch.randn(1, H, generator=g)
            own = torch.randn(B, H, generator=g)
            x = math.sqrt(corr) * common + math.sqrt(1 - corr) * own
        else:
            x = torch.randn(B, H, generator=g)
    else:
        wg = torch.rand(I, H, generator=g) - 0.5
        wu = torch.rand(I, H, generator=g) - 0.5
        wd = torch.rand(H, I, generator=g) - 0.5
        x = torch.rand(B, H, generator=g) - 0.5
    if heavy_tail:
        wg = wg * torch.exp(torch.randn(I, 1, generator=g) * 0.5)
    cast = lambda t: t.to(dtype).contiguous()
    return dict(x=cast(x), wg=cast(wg), wu=cast(wu), wd=cast(wd), wdt=cast(wd).t().contiguous())


def calibrate(wg, sparsities, n_vec=256, seed=1234):
    """Thresholds at exact percentiles of |SiLU(X wg^T)| over n_vec seeded N(0,1) vectors, computed in fp32."""
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(n_vec, wg.shape[1], generator=g)
    act = F.silu(X @ wg.float().t()).abs().flatten()
    out = []
    for s in sparsities:
        if s <= 0:
            out.append(-1.0)
        else:
            k = min(max(int(round(s * act.numel())), 1), act.numel())
            out.append(float(torch.kthvalue(act, k).values))
    return out


def dev(d, device="cuda"):
    return {k: v.to(device) for k, v in d.items()}


def load_golden():
    """tests/golden/cats_mlp_small.npz as {case: dict of CPU tensors + t}.  The file holds storage bits (npz has no
    bfloat16); the dtype is in the case name."""
    from pathlib import Path

    import numpy as np

    z = np.load(Path(__file__).resolve().parent / "golden" / "cats_mlp_small.npz")
    cases = {}
    for key in z.files:
        name, field = key.split("/")
        cases.setdefault(name, {})[field] = z[key]
    out = {}
    for name, c in cases.items():
        dtype = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[name.split("_")[0]]

        def dec(arr, dtype=dtype):
            if dtype == torch.float32:
                return torch.from_numpy(arr.astype("int64").astype("uint32").view("int32").copy()).view(torch.float32)
            return torch.from_numpy(arr.view("int16").copy()).view(dtype)

        d = {k: dec(c[k]) for k in ("x", "wg", "wu", "wd", "a", "y")}
        d["flag"] = torch.from_numpy(c["flag"].copy()).bool()
        d["t"] = float(c["t"])
        d["wdt"] = d["wd"].t().contiguous()
        d["dtype"] = dtype
        out[name] = d
    return out
