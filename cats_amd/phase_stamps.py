"""Where the time of the single-pass MLP kernel goes, workgroup by workgroup.

``python -m cats_amd.phase_stamps [--batch 1] [--sparsity 0.5] [--calls 24]`` loads the stamped twin of the kernel
library (``cats_amd/lib/libcats_gemv_timing.so``, built by ``python -m cats_amd.build --timing`` with ``-DCATS_TIMING``), runs
``cats_mlp`` on the Llama-2-7B layer shape over rotating weight sets and prints, over all workgroups of all calls,
when each phase boundary was reached (microseconds after the first workgroup of the call started; the stamp is the
100 MHz ``wall_clock64`` counter, so one tick is 10 ns):

  start    thread 0 enters the kernel
  staged   x is in LDS (after the staging barrier)
  rows     the last row wave has published its last neuron (gate, threshold, up)
  down     down wave 0 has consumed its last live neuron
  stored   down wave 0 has issued its partial-sum stores

The stamps cost a few stores per workgroup; the stamped library is a measuring tool and nothing else loads it.
"""
from __future__ import annotations

import argparse
import ctypes

import torch
import torch.nn.functional as F

from . import capi
from .build import TIMING_LIB

H, I = 4096, 11008
SLOTS = 8  # stamps per workgroup in the buffer the kernel writes


def quantiles(v: torch.Tensor) -> str:
    q = torch.quantile(v.double(), torch.tensor([0.0, 0.1, 0.5, 0.9, 1.0], dtype=torch.float64))
    return "  ".join(f"{float(x):6.2f}" for x in q)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=1, choices=(1, 2))
    ap.add_argument("--sparsity", type=float, default=0.5)
    ap.add_argument("--calls", type=int, default=24)
    ap.add_argument("--sets", type=int, default=8)
    ap.add_argument("--workgroups-per-cu", type=int, default=1,
                    help="2 for a library built with CATS_HIP_DEFINES=-DCATS_FUSED_WAVES=8 (the stamp buffer has a line per workgroup)")
    args = ap.parse_args()

    if not TIMING_LIB.exists():
        raise SystemExit(f"{TIMING_LIB} is missing: build it with `python -m cats_amd.build`")
    capi.use_library(TIMING_LIB)
    L = capi.lib()
    L.cats_timing_buffer_fused.argtypes = [ctypes.c_void_p]
    L.cats_timing_buffer_fused.restype = None

    dev = "cuda"
    B = args.batch
    g = torch.Generator(device=dev).manual_seed(0)
    sets = [tuple((torch.randn(I, H, generator=g, device=dev) * 0.02).half() for _ in range(3)) for _ in range(args.sets)]
    x = torch.randn(B, H, generator=g, device=dev).half()
    calib = torch.randn(256, H, generator=g, device=dev)
    act = F.silu(calib @ sets[0][0].float().t()).abs().flatten()
    t = -1.0 if args.sparsity <= 0 else float(torch.kthvalue(act.cpu(), int(args.sparsity * act.numel())).values)
    ws = capi.Workspace(B, H, I)
    y = torch.empty(B, H, dtype=torch.float16, device=dev)
    grid = torch.cuda.get_device_properties(0).multi_processor_count * max(1, args.workgroups_per_cu)
    stamps = torch.zeros(grid * SLOTS, dtype=torch.int64, device=dev)

    for i in range(16):                                   # warm-up without stamps
        capi.mlp(x, *sets[i % args.sets], t, ws, y=y)
    torch.cuda.synchronize()
    L.cats_timing_buffer_fused(ctypes.c_void_p(stamps.data_ptr()))
    rows = []
    for i in range(args.calls):
        stamps.zero_()
        capi.mlp(x, *sets[i % args.sets], t, ws, y=y)
        torch.cuda.synchronize()
        r = stamps.cpu().view(grid, SLOTS)
        r = r[r[:, 0] > 0]                                # workgroups that ran
        ticks = r[:, :5].double()
        us = (ticks - ticks[:, 0].min()) * 0.01
        rows.append(torch.cat([us, r[:, 6:7].double()], dim=1))
    L.cats_timing_buffer_fused(None)
    allr = torch.cat(rows)

    print(f"single-pass kernel, Llama shape {H}->{I}, fp16, batch {B}, target sparsity {args.sparsity}: "
          f"{args.calls} calls x {rows[0].shape[0]} workgroups")
    print("microseconds after the first workgroup's start      min     p10  median     p90     max")
    for k, name in enumerate(("start", "staged", "rows", "down", "stored")):
        print(f"  {name:48s} {quantiles(allr[:, k])}")
    print(f"  {'live neurons per workgroup':48s} {quantiles(allr[:, 5])}")
    last = torch.stack([r[:, 4].max() for r in rows])
    med = torch.stack([r[:, 4].median() for r in rows])
    print(f"per call: last workgroup stored at {float(last.mean()):.2f} us (mean over calls), the median workgroup at "
          f"{float(med.mean()):.2f} us")
    live = allr[:, 5]
    for k, name in ((2, "last neuron published"), (3, "end of the down pass")):
        end = allr[:, k]
        c = torch.corrcoef(torch.stack([end, live]))[0, 1].item()
        slope = float(((end - end.mean()) * (live - live.mean())).sum() / ((live - live.mean()) ** 2).sum())
        print(f"{name} against live neurons of the workgroup: correlation {c:.2f}, {slope:.3f} us per live neuron")
    xcd = torch.arange(rows[0].shape[0]) % 8
    per_xcd = [float(torch.stack([r[xcd == k, 3].mean() for r in rows]).mean()) for k in range(8)]
    print("mean end of the down pass by blockIdx % 8 (workgroups are dealt round-robin over the 8 XCDs): "
          + "  ".join(f"{v:.2f}" for v in per_xcd))


if __name__ == "__main__":
    main()
