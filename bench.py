#!/usr/bin/env python3
"""Benchmark of the CATS sparse-MLP decode path on one MI355X.

A "step" is one CATS MLP call (gate GEMV + SiLU + threshold + sparse up + sparse down, then the reduction over
the workgroups' partial sums) on a Llama-2-7B-shaped layer (4096 -> 11008), fp16, batch 1, threshold at the 50th percentile of |SiLU(gate)| --
the configuration the headline metric is quoted on.  Inputs are resident in HBM before the timed region.
Steps rotate over several independent weight sets whose total size exceeds the 256 MB memory-side cache,
so every step streams its weights from HBM.

Prints ONE JSON line: per-layer latency (value, us: plain stream launches of the fp16-output call; the HIP-graph
replay and the one-launch fp32-accumulate contract beside it), achieved HBM bandwidth on touched bytes, the same
for sparsities 0/30/50/70/90 %, the dense fp16 GEMV MLP (stock PyTorch-ROCm F.linear) on the same GPU, the read-stream
bandwidth the GPU reaches (`stream_ceiling`), a `roofline` object for the dominant kernel and a `cpu_baseline` object
(the dense-masked PyTorch CATS MLP on this box's host cores).  `--decode` adds the 32-layer decode loop (tokens/s,
CATS vs dense).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
# HBM bytes per launch of the dominant kernel at 50 % sparsity, from rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a copy of
# known size.  The record names the kernel sources it was measured on (a hash); if they have changed since, the figure
# is stale and `roofline.traffic` is reported as null.
TRAFFIC_RECORD = ROOT / "profiles" / "cats_mlp_llama7b_fp16_b1_s50_hbm_traffic.json"
H, I = 4096, 11008
SPARSITIES = [0.0, 0.3, 0.5, 0.7, 0.9]


def touched_bytes(sz, B, k):
    """Algorithmic bytes of one CATS MLP call: all of W_gate, k rows each of W_up and W_down^T, x, y, a, the int32
    index list and the count."""
    return sz * H * I + 2 * sz * H * k + sz * B * (2 * H + I) + 4 * k + 4


def stage_bytes(sz, B, k, grid=256):
    """Bytes per launch of the two kernels of the single-pass path: (streaming kernel, reduction, partial sums).
    Streaming: the algorithmic bytes of the whole call (touched_bytes: the streaming kernel is the one that moves them);
    the fp32 partial sums it leaves per workgroup are this design's own overhead and are returned separately, not
    counted as algorithmic.  Reduction: those partial sums and y."""
    partials = grid * B * H * 4
    stream = touched_bytes(sz, B, k)
    reduce = partials + sz * B * H
    return stream, reduce, partials


def csrc_hash():
    """sha256 over the kernel sources, in name order: ties a committed counter reading to the code it was taken on."""
    import hashlib

    h = hashlib.sha256()
    for f in sorted((ROOT / "cats_amd" / "csrc").iterdir()):
        if f.suffix in (".h", ".hip", ".cpp"):
            h.update(f.name.encode())
            h.update(f.read_bytes())
    return h.hexdigest()[:16]


def measured_traffic():
    """(bytes or None, note) from the committed counter record, None if it was taken on other kernel sources."""
    try:
        rec = json.loads(TRAFFIC_RECORD.read_text())
    except (OSError, ValueError):
        return None, f"no counter record at {TRAFFIC_RECORD.name}"
    if rec.get("csrc_hash") != csrc_hash():
        return None, f"counter record {TRAFFIC_RECORD.name} was taken on other kernel sources ({rec.get('csrc_hash')} != {csrc_hash()})"
    return int(rec["fetch_bytes"] + rec["write_bytes"]), f"{TRAFFIC_RECORD.name}: {rec.get('kernel')}"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--sets", type=int, default=8, help="independent weight sets rotated through (cache defeat)")
    ap.add_argument("--sparsity", type=float, default=0.5)
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip everything but the headline configuration")
    ap.add_argument("--extra", default="mistral,batch,70b,entry",
                    help="which of the other measurements to run: mistral (bf16, heavy-tailed), batch (2/4/8), 70b (8192->28672), "
                         "entry (each drop-in entry point alone)")
    ap.add_argument("--batches", default="2,4,8,16", help="with --extra batch: the batch sizes to run")
    ap.add_argument("--entries", default="", help="with --extra entry: comma-separated entry points to time (default: all)")
    ap.add_argument("--no-graph", action="store_true", help="time plain stream launches only")
    ap.add_argument("--decode", action="store_true", help="(default) run the 32-layer decode loop (config 5)")
    ap.add_argument("--no-decode", action="store_true", help="skip the 32-layer decode loop")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run one 256 MiB device-to-device copy first: a kernel of known traffic for scaling rocprof counters")
    ap.add_argument("--print-csrc-hash", action="store_true", help="print the hash of the kernel sources (for a new counter record) and exit")
    ap.add_argument("--contract", choices=("both", "y_out", "y_f32"), default="both",
                    help="profiling aid: run the timed loops of one output contract only, so that a kernel trace or a counter run holds "
                         "launches of one kind (y_f32: value is then the fp32-accumulate call and config.contract says so)")
    ap.add_argument("--path", type=int, default=0, help="1 = keep the call on the separate gate+up and sparse-down kernels")
    ap.add_argument("--gate-variant", type=int, default=0)
    ap.add_argument("--down-groups", type=int, default=0)
    ap.add_argument("--down-block", type=int, default=0)
    args = ap.parse_args()
    if args.print_csrc_hash:
        print(csrc_hash())
        return
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path needs no collective); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import torch.nn.functional as F

    from cats_amd import capi

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    L = capi.lib()  # raises if the HIP library is missing: no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    dtype, sz, B = torch.float16, 2, 1
    capi.set_tuning(args.gate_variant, args.down_groups, args.down_block, args.path)

    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- synthetic layer sets --------------------------------------------------------------------------------
    g = torch.Generator(device="cuda").manual_seed(0)
    sets = []
    for _ in range(args.sets):
        wg = (torch.randn(I, H, generator=g, device=dev) * 0.02).to(dtype)
        wu = (torch.randn(I, H, generator=g, device=dev) * 0.02).to(dtype)
        wd = (torch.randn(H, I, generator=g, device=dev) * 0.02).to(dtype)
        sets.append(dict(wg=wg, wu=wu, wd=wd, wdt=wd.t().contiguous()))
    x = torch.randn(B, H, generator=g, device=dev).to(dtype)
    # thresholds: exact percentiles of |SiLU(X wg^T)| over 256 seeded calibration vectors (first set; the sets
    # are identically distributed)
    X = torch.randn(256, H, generator=g, device=dev)
    act = F.silu(X @ sets[0]["wg"].float().t()).abs().flatten()
    thr = {}
    for s in SPARSITIES + [args.sparsity]:
        thr[s] = -1.0 if s <= 0 else float(torch.kthvalue(act.cpu(), max(1, int(round(s * act.numel())))).values)
    del X, act

    ws = capi.Workspace(B, H, I)
    y = torch.empty(B, H, dtype=dtype, device=dev)
    count = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    y32 = torch.zeros(B, H, dtype=torch.float32, device=dev)

    def mlp_args(st, t, cnt=None, f32=False):
        return (p(x), p(st["wg"]), p(st["wu"]), p(st["wdt"]), None if f32 else p(y), p(y32) if f32 else None, None, cnt, B, H, I,
                capi.F16, ctypes.c_float(t), p(ws.buf), ws.nbytes, stream)

    def active_count(t):
        ks = []
        for st in sets:
            capi.check(L.cats_mlp(*mlp_args(st, t, p(count))), "cats_mlp")
            ks.append(int(count.item()))
        return sum(ks) / len(ks)

    def time_region(fn_step, steps, warmup):
        """EXACTLY `steps` calls between two events on the launch stream, synchronised on both sides."""
        for i in range(warmup):
            fn_step(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn_step(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps  # us per step

    def time_cats(t, steps, warmup, stage=0, f32=False, zero_fill=False):
        """stage 0: the whole call; 1 / 2: one of its two launches alone, back to back (cats_mlp_stage).
        f32: the fp32-accumulate contract (one launch, atomics into the caller's buffer); zero_fill: with the fill
        kernel that contract asks the caller for in front of every call."""
        prepared = [mlp_args(st, t, f32=f32) for st in sets]
        n = len(prepared)
        if stage:
            stage_args = [(stage,) + a[:5] + a[8:] for a in prepared]  # no y_f32 / flag_out / count_out
            fn = lambda i: L.cats_mlp_stage(*stage_args[i % n])
        elif zero_fill:
            def fn(i):
                y32.zero_()
                return L.cats_mlp(*prepared[i % n])
        else:
            fn = lambda i: L.cats_mlp(*prepared[i % n])
        capi.check(fn(0), "cats_mlp (first timed-configuration call)")
        us = time_region(fn, steps, warmup)
        capi.check(fn(0), "cats_mlp (after the timed region)")
        return us

    def per_rep_stats(t, reps):
        """Every call between its own pair of events (the reference's bench/utils.py:44-58 times one call per rep and
        reports the geometric mean; its cache flush is the weight-set rotation here)."""
        prepared = [mlp_args(st, t) for st in sets]
        n = len(prepared)
        for i in range(n * 4):
            L.cats_mlp(*prepared[i % n])
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        torch.cuda.synchronize()
        for i, (e0, e1) in enumerate(ev):
            e0.record()
            L.cats_mlp(*prepared[i % n])
            e1.record()
        torch.cuda.synchronize()
        us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in ev)
        import math

        gmean = math.exp(sum(math.log(max(u, 1e-3)) for u in us) / len(us))
        return dict(reps=reps, median_us=round(us[len(us) // 2], 2), gmean_us=round(gmean, 2), min_us=round(us[0], 2),
                    p90_us=round(us[int(0.9 * (len(us) - 1))], 2), max_us=round(us[-1], 2),
                    note="one call per event pair; event records sit inside each interval, so these run above the block mean")

    def time_cats_graph(t, steps, warmup):
        """The same steps replayed from a HIP graph holding one step per weight set."""
        prepared = [mlp_args(st, t) for st in sets]
        n = len(prepared)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            sargs = [a[:-1] + (ctypes.c_void_p(side.cuda_stream),) for a in prepared]
            for a in sargs:
                L.cats_mlp(*a)
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                cap = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for a in prepared:
                    capi.check(L.cats_mlp(*(a[:-1] + (cap,))), "cats_mlp (capture)")
        torch.cuda.synchronize()
        reps, wreps = max(1, steps // n), max(1, warmup // n)
        us = time_region(lambda i: graph.replay(), reps, wreps) / n
        return us, reps * n

    def time_dense(steps, warmup):
        n = len(sets)

        def step(i):
            st = sets[i % n]
            return F.linear(F.silu(F.linear(x, st["wg"])) * F.linear(x, st["wu"]), st["wd"])

        return time_region(step, steps, warmup)

    # ---- headline: 50 % sparsity ---------------------------------------------------------------------------------
    t50 = thr[args.sparsity]
    k50 = active_count(t50)
    only32 = args.contract == "y_f32"
    us_eager = time_cats(t50, args.steps, args.warmup, f32=only32)
    if args.no_graph or only32:
        us_graph, graph_steps = None, 0
    else:
        us_graph, graph_steps = time_cats_graph(t50, args.steps, args.warmup)
    # Per-kernel launch durations: at least 400 launches and 50 warm-up launches each, whatever --steps says.  The first
    # launch after the synchronisation that opens a timed region pays the launch latency in full; over 20 launches that
    # adds a microsecond to a 32 us kernel, over 400 it does not (the rocprofv3 trace of the same command agrees with
    # the long figure).  `value` itself is timed over exactly --steps calls.
    kernel_steps, kernel_warmup = max(args.steps, 400), max(args.warmup, 50)
    if only32:  # one launch: the call is the kernel
        us_k1, us_k2, rep_stats = us_eager, float("nan"), None
    else:
        us_k1 = time_cats(t50, kernel_steps, kernel_warmup, stage=1)
        us_k2 = time_cats(t50, kernel_steps, kernel_warmup, stage=2)
        rep_stats = per_rep_stats(t50, min(400, max(50, args.steps)))
    us_dense = time_dense(args.steps, args.warmup)
    if args.contract == "y_out":
        us_f32 = us_f32_zero = float("nan")
    else:
        us_f32 = us_eager if only32 else time_cats(t50, args.steps, args.warmup, f32=True)
        us_f32_zero = time_cats(t50, args.steps, args.warmup, f32=True, zero_fill=True)
    # value is the plain stream-launch time of the call the decode path makes (fp16 y, two launches, bitwise
    # reproducible); the graph replay and the one-launch fp32-accumulate contract are reported beside it
    us, launch, steps_timed = us_eager, "stream", args.steps
    tb = touched_bytes(sz, B, k50)
    ceiling = stream_ceiling(torch, capi, tb)
    single_pass = args.path != 1
    partial_bytes = 0
    if single_pass:
        b_k1, b_k2, partial_bytes = stage_bytes(sz, B, k50)
        k1_name = "cats::mlp_fused_kernel<F16,B=1> (gate GEMV + SiLU + threshold + sparse up + sparse down into per-workgroup partial sums)"
        k2_name = "cats::reduce_partials_kernel<F16> (sum of the 256 partial sums, rounding, y)"
    else:
        b_k1 = sz * H * I + sz * H * k50 + sz * B * H + I // 8 + 4 * B * k50
        b_k2 = sz * H * k50 + 4 * B * k50 + I // 8 + sz * B * H
        k1_name = "cats::rows_kernel<F16,B=1,kGateUp> (gate GEMV + SiLU + threshold + sparse up)"
        k2_name = "cats::down_kernel<F16,B=1> (sparse neuron-major down)"
    traffic, traffic_note = measured_traffic() if (single_pass and abs(args.sparsity - 0.5) < 1e-9) else (None, "measured for the default path at 50 % only")

    sweep = []
    if not args.no_sweep:
        ssteps, swarm = max(200, args.steps // 4), max(50, args.warmup // 4)
        for s in SPARSITIES:
            k = active_count(thr[s])
            u = time_cats(thr[s], ssteps, swarm)
            u32 = time_cats(thr[s], ssteps, swarm, f32=True) if args.contract != "y_out" else float("nan")
            b = touched_bytes(sz, B, k)
            sweep.append(dict(target_sparsity=s, sparsity=round(1 - k / I, 4), us=round(u, 2), touched_MB=round(b / 1e6, 1),
                              GBps=round(b / u * 1e-3, 1), hbm_frac=round(b / u * 1e-3 / HBM_PEAK_GBPS, 4),
                              speedup_vs_dense=round(us_dense / u, 3), us_f32_accumulate=round(u32, 2),
                              hbm_frac_f32_accumulate=round(b / u32 * 1e-3 / HBM_PEAK_GBPS, 4)))

    out = {
        "metric": "CATS-MLP us/layer + achieved HBM GB/s (touched bytes); batch-1 decode tok/s",
        "value": round(us, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": steps_timed,
        "warmup": args.warmup,
        "ms_per_step": round(us / 1e3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "Llama-2-7B-shaped CATS MLP 4096->11008, fp16, batch 1, threshold at the 50th percentile of |SiLU(gate)|",
                   "hidden": H, "intermediate": I, "batch": B, "target_sparsity": args.sparsity,
                   "achieved_sparsity": round(1 - k50 / I, 4), "active_neurons": round(k50, 1), "weight_sets": args.sets,
                   "launch": launch, "contract": "y_f32 (fp32 accumulate, one launch)" if only32 else "y_out (fp16, two launches)"},
        "touched_bytes": int(tb),
        "achieved_GBps_touched": round(tb / us * 1e-3, 1),
        "hbm_frac_touched": round(tb / us * 1e-3 / HBM_PEAK_GBPS, 4),
        "us_stream_launch": round(us_eager, 3),
        "us_hipgraph": None if us_graph is None else round(us_graph, 3),
        "hipgraph_steps": graph_steps,
        "f32_accumulate": {
            "what": "cats_mlp with y_f32 (the contract of the reference's fuse_gemv_gemv_gemv / flag_gemv_gemv_atomic: the caller "
                    "zeroes an fp32 (B, H) buffer, the call adds into it): one launch, fp32 atomics, no reduction launch; summation "
                    "order and so the last bits vary from run to run",
            "us": round(us_f32, 3),
            "hbm_frac_touched": round(tb / us_f32 * 1e-3 / HBM_PEAK_GBPS, 4),
            "us_with_zero_fill": round(us_f32_zero, 3),
            "hbm_frac_touched_with_zero_fill": round(tb / us_f32_zero * 1e-3 / HBM_PEAK_GBPS, 4),
            "plain_read_time_over_call_time": round(ceiling["same_bytes_as_one_call"]["us"] / us_f32, 4),
        },
        "stream_ceiling": ceiling,
        "frac_of_stream_ceiling": round(tb / us * 1e-3 / ceiling["GBps"], 4),
        "plain_read_of_the_same_bytes_us": ceiling["same_bytes_as_one_call"]["us"],
        "plain_read_time_over_call_time": round(ceiling["same_bytes_as_one_call"]["us"] / us, 4),
        "dense_fp16_us": round(us_dense, 3),
        "dense_GBps": round(3 * sz * H * I / us_dense * 1e-3, 1),
        "speedup_vs_dense": round(us_dense / us, 3),
        "per_rep": rep_stats,
        "roofline": {
            "bound": "hbm",
            "kernel": k1_name,
            "achieved": round(b_k1 / us_k1 * 1e-3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(b_k1 / us_k1 * 1e-3 / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_note,
            "bytes_per_launch": int(b_k1),
            "design_overhead_bytes": int(partial_bytes),
            "bytes_note": "bytes_per_launch are the algorithmic bytes of the call (weights touched, x, y, a, index list, count); "
                          "design_overhead_bytes are the per-workgroup fp32 partial sums this design writes and reads on top, "
                          "not counted in achieved / frac",
            "us_per_launch": round(us_k1, 3),
            "frac_of_stream_ceiling": round(b_k1 / us_k1 * 1e-3 / ceiling["GBps"], 4),
            "second_kernel": {"kernel": k2_name, "bytes_per_launch": int(b_k2), "us_per_launch": round(us_k2, 3),
                              "achieved": round(b_k2 / us_k2 * 1e-3, 1), "frac": round(b_k2 / us_k2 * 1e-3 / HBM_PEAK_GBPS, 4)},
            "kernel_launches_timed": kernel_steps,
            "note": "per-kernel times are back-to-back launches of that kernel alone (launch gap included; at least 400 of them, so that the one launch latency after the opening synchronisation does not weigh on them), timed with events on the launch stream; value is the whole call over exactly `steps` calls",
        },
        "sweep": sweep,
    }

    extra = set() if args.no_extra else {e.strip() for e in args.extra.split(",") if e.strip()}
    if extra & {"mistral", "batch", "70b"}:
        del sets
        torch.cuda.empty_cache()
        out["other_configs"] = other_configs(torch, F, capi, L, max(200, args.steps // 4), max(50, args.warmup // 4), extra,
                                             [int(b) for b in args.batches.split(",") if b.strip()], args.contract)

    if "entry" in extra:
        out["entry_points"] = entry_points(torch, F, capi, max(200, args.steps // 4), max(50, args.warmup // 4),
                                           {e.strip() for e in args.entries.split(",") if e.strip()})

    if not args.no_decode:
        from cats_amd import decoder

        out["decode"] = decoder.bench_decode(prompt_len=128, gen_len=256, sparsity=0.5)

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch, F, thr[0.5] if 0.5 in thr else t50)
        if not args.no_decode:
            from cats_amd import decoder

            # the same greedy loop with the dense-masked PyTorch CATS MLP in fp32 on the host cores: 4 of the 32 layers,
            # 7 timed tokens, per-token time scaled to 32 layers
            out["cpu_baseline"]["decode"] = decoder.cpu_decode_baseline(num_layers=4, gen_len=8, prompt_len=16, sparsity=0.5,
                                                                         threads=out["cpu_baseline"]["cores"])

    def no_nan(v):  # figures of a contract that was not run
        if isinstance(v, float) and v != v:
            return None
        if isinstance(v, dict):
            return {k: no_nan(w) for k, w in v.items()}
        if isinstance(v, list):
            return [no_nan(w) for w in v]
        return v

    print(json.dumps(no_nan(out)))


def stream_ceiling(torch, capi, call_bytes, gib=1, reps=40):
    """Read-stream bandwidth this GPU reaches: cats_probe_read (read-only, the same 128-bit streaming loads as the weight
    rows) over a 1 GiB buffer, four times the 256 MB memory-side cache, timed with events on the launch stream.  And the
    same kernel over exactly the bytes one headline call touches (slices of the buffer in turn, so nothing is cached):
    the time a perfectly balanced, dependency-free read of those bytes takes as one launch -- a launch's fixed cost
    weighs more on 181 MB than on 1 GiB."""
    buf = torch.empty(gib << 30, dtype=torch.uint8, device="cuda")
    buf.fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")

    def timed(fn, n):
        for i in range(5):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    us = timed(lambda i: capi.probe_read(buf, sink), reps)
    nbytes = buf.numel()
    nb = int(call_bytes) // 16 * 16
    slices = [buf[i * nb:(i + 1) * nb] for i in range(nbytes // nb)]
    us_call = timed(lambda i: capi.probe_read(slices[i % len(slices)], sink), 10 * reps)
    del buf, slices
    torch.cuda.empty_cache()
    return {"GBps": round(nbytes / us * 1e-3, 1), "frac_of_peak": round(nbytes / us * 1e-3 / HBM_PEAK_GBPS, 4), "bytes": nbytes,
            "us_per_pass": round(us, 2), "kernel": "read_probe_kernel (cats_probe_read): read-only, nothing written",
            "same_bytes_as_one_call": {"bytes": nb, "us": round(us_call, 2), "GBps": round(nb / us_call * 1e-3, 1),
                                       "frac_of_peak": round(nb / us_call * 1e-3 / HBM_PEAK_GBPS, 4)}}


def other_configs(torch, F, capi, L, steps, warmup, which, batches=(2, 4, 8, 16), contract="both"):
    """The remaining single-layer configurations: Mistral-7B shape in bf16 with heavy-tailed gate rows (50 / 70 %), and
    the Llama fp16 layer at batch 2 / 4 / 8 with pairwise-correlated rows (per-row masks, union gathering), and the
    Llama-70B-shaped layer at batch 1."""
    import math

    dev = torch.device("cuda:0")
    res = []

    def run(name, Hh, Ii, B, dtype, code, sparsities, heavy_tail=False, corr=0.0, nsets=6, batch_entry_points=False):
        g = torch.Generator(device="cuda").manual_seed(1)
        sz = 2
        sets = []
        for _ in range(nsets):
            wg = torch.randn(Ii, Hh, generator=g, device=dev) * 0.02
            if heavy_tail:
                wg = wg * torch.exp(torch.randn(Ii, 1, generator=g, device=dev) * 0.5)
            wu = torch.randn(Ii, Hh, generator=g, device=dev) * 0.02
            wd = torch.randn(Hh, Ii, generator=g, device=dev) * 0.02
            sets.append(dict(wg=wg.to(dtype), wu=wu.to(dtype), wd=wd.to(dtype), wdt=wd.to(dtype).t().contiguous()))
            del wg, wu, wd
        if corr > 0:
            x = (math.sqrt(corr) * torch.randn(1, Hh, generator=g, device=dev) + math.sqrt(1 - corr) * torch.randn(B, Hh, generator=g, device=dev)).to(dtype)
        else:
            x = torch.randn(B, Hh, generator=g, device=dev).to(dtype)
        X = torch.randn(256, Hh, generator=g, device=dev)
        act = F.silu(X @ sets[0]["wg"].float().t()).abs().flatten().cpu()
        ws = capi.Workspace(B, Hh, Ii)
        y = torch.empty(B, Hh, dtype=dtype, device=dev)
        y32 = torch.zeros(B, Hh, dtype=torch.float32, device=dev)
        count = torch.zeros(1, dtype=torch.int32, device=dev)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        p = lambda t: ctypes.c_void_p(t.data_ptr())

        def timed(fn):
            for i in range(warmup):
                fn(i)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(steps):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / steps

        us_dense = timed(lambda i: F.linear(F.silu(F.linear(x, sets[i % nsets]["wg"])) * F.linear(x, sets[i % nsets]["wu"]), sets[i % nsets]["wd"]))
        for s in sparsities:
            t = float(torch.kthvalue(act, max(1, int(round(s * act.numel())))).values)
            ks = []
            for st in sets:
                capi.check(L.cats_mlp(p(x), p(st["wg"]), p(st["wu"]), p(st["wdt"]), p(y), None, None, p(count), B, Hh, Ii, code, ctypes.c_float(t),
                                      p(ws.buf), ws.nbytes, stream), "cats_mlp")
                ks.append(int(count.item()))
            k = sum(ks) / len(ks)
            prepared = [(p(x), p(st["wg"]), p(st["wu"]), p(st["wdt"]), p(y), None, None, None, B, Hh, Ii, code, ctypes.c_float(t), p(ws.buf), ws.nbytes, stream)
                        for st in sets]
            us = timed(lambda i: L.cats_mlp(*prepared[i % nsets])) if contract != "y_f32" else float("nan")
            # the fp32-accumulate contract (adds into the caller's fp32 buffer; one launch at 1..2 rows)
            prepared32 = [a[:4] + (None, p(y32)) + a[6:] for a in prepared]
            us32 = timed(lambda i: L.cats_mlp(*prepared32[i % nsets])) if contract != "y_out" else float("nan")
            tb = sz * Hh * Ii + 2 * sz * Hh * k + sz * B * (2 * Hh + Ii) + 4 * k + 4
            line = dict(config=name, batch=B, row_sparsity_target=s, union_sparsity=round(1 - k / Ii, 4), us=round(us, 2),
                        touched_MB=round(tb / 1e6, 1), GBps=round(tb / us * 1e-3, 1), hbm_frac=round(tb / us * 1e-3 / HBM_PEAK_GBPS, 4),
                        dense_us=round(us_dense, 2), speedup_vs_dense=round(us_dense / us, 3), us_f32_accumulate=round(us32, 2),
                        hbm_frac_f32_accumulate=round(tb / us32 * 1e-3 / HBM_PEAK_GBPS, 4))
            if batch_entry_points:
                # the same batch through the two other whole-MLP contracts of the reference: gate activations given
                # (gemv_gemv_triton; reads W_up and W_down^T rows only) and W_down in nn.Linear's layout, read whole
                # (flag_gemv_gemv_inner, which the reference instantiates for 1, 2, 8 and 16 rows)
                acts = [capi.gate_flag(x, st["wg"], t)[0] for st in sets]
                line["us_up_down_given_gate"] = round(timed(lambda i: capi.up_down(x, acts[i % nsets], sets[i % nsets]["wu"], sets[i % nsets]["wdt"], t, ws)), 2)
                line["us_rowmajor_down"] = round(timed(lambda i: capi.mlp_rowmajor_down(x, sets[i % nsets]["wg"], sets[i % nsets]["wu"], sets[i % nsets]["wd"], t, ws)), 2)
                del acts
            res.append(line)
        del sets
        torch.cuda.empty_cache()

    if "mistral" in which:
        run("mistral7b_bf16_heavy_tail", 4096, 14336, 1, torch.bfloat16, capi.BF16, [0.5, 0.7], heavy_tail=True)
    if "batch" in which:
        for B in batches:
            run(f"llama7b_fp16_batch{B}_corr0.5", 4096, 11008, B, torch.float16, capi.F16, [0.5], corr=0.5, batch_entry_points=contract == "both")
    if "70b" in which:
        # the larger shape the reference smoke-tests (flash_gemv/test/test_fuse_gemv_cmp.py:662-676): 1.4 GB per weight set
        run("llama70b_fp16", 8192, 28672, 1, torch.float16, capi.F16, [0.5], nsets=2)
    return res


def entry_points(torch, F, capi, steps, warmup, only=()):
    """Latency of each drop-in entry point alone on the headline layer (Llama shape, fp16, batch 1, 50 % sparsity),
    with the algorithmic bytes it has to move.  Weight sets rotate as in the headline run."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(2)
    nsets, sz = 6, 2
    sets = []
    for _ in range(nsets):
        wg = (torch.randn(I, H, generator=g, device=dev) * 0.02).half()
        wu = (torch.randn(I, H, generator=g, device=dev) * 0.02).half()
        wd = (torch.randn(H, I, generator=g, device=dev) * 0.02).half()
        sets.append(dict(wg=wg, wu=wu, wd=wd, wdt=wd.t().contiguous()))
    x = torch.randn(1, H, generator=g, device=dev).half()
    X = torch.randn(256, H, generator=g, device=dev)
    act = F.silu(X @ sets[0]["wg"].float().t()).abs().flatten().cpu()
    t = float(torch.kthvalue(act, int(0.5 * act.numel())).values)
    ws = capi.Workspace(1, H, I)
    # per-set inputs of the later stages, produced by the earlier ones
    for st in sets:
        st["a"], st["flag"] = capi.gate_flag(x, st["wg"], t)
        st["z"] = capi.up_flag(x, st["wu"], st["a"], st["flag"])
        # the same active set as a sorted index list with compact activations / intermediates (the DejaVu-style interface)
        st["idx"] = torch.nonzero(st["flag"][0]).flatten()
        st["a_c"] = st["a"][0][st["idx"]].contiguous()
        st["z_c"] = st["z"][:, st["idx"]].contiguous()
        st["wg_t"] = st["wg"].t().contiguous()
    k = sum(int(st["flag"].sum()) for st in sets) / nsets
    nw = torch.ones(H, dtype=torch.float16, device=dev)
    # fuse_gemv_cmp: device part only (the reference's op also copies the count to the host, which is a stream sync)
    vals = torch.empty(I, dtype=torch.float16, device=dev)
    idx = torch.empty(I, dtype=torch.int64, device=dev)
    cnt = torch.zeros(1, dtype=torch.int32, device=dev)
    out32 = torch.zeros(1, H, dtype=torch.float32, device=dev)
    L = capi.lib()
    import flash_gemv as fg

    pv = lambda t_: ctypes.c_void_p(t_.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def compact(st):
        capi.check(L.cats_gate_compact(pv(x), pv(st["wg"]), pv(vals), pv(idx), pv(cnt), H, I, capi.F16, ctypes.c_float(t), pv(ws.buf),
                                       ws.nbytes, stream), "cats_gate_compact")

    def timed(fn):
        for i in range(warmup):
            fn(sets[i % nsets])
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn(sets[i % nsets])
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    full, act_rows = sz * H * I, sz * H * k
    table = [
        ("cats_gate_flag", "fuse_gemv_flag / _local / _batch", full, lambda st: capi.gate_flag(x, st["wg"], t)),
        ("cats_gate_compact", "fuse_gemv_cmp (ordered index list + count, device part)", full, compact),
        ("cats_up_flag", "fuse_flag_gemv_local, gather_gemv_elemul_flag_3d", act_rows, lambda st: capi.up_flag(x, st["wu"], st["a"], st["flag"])),
        ("cats_down_flag", "atomic_gemv, gather_transposed_gemv_flag_3d", act_rows, lambda st: capi.down_flag(st["z"], st["wdt"], st["flag"], ws)),
        ("cats_up_index", "gather_gemv, gather_gemv_elemul_indirect_index_2d (sorted index list)", act_rows,
         lambda st: capi.up_index(x, st["wu"], st["idx"], None, st["a_c"])),
        ("cats_down_index", "gather_transposed_gemv, gather_transposed_gemv_indirect_index_2d (sorted index list)", act_rows,
         lambda st: capi.down_index(st["z_c"], st["wdt"], st["idx"], ws)),
        ("flash_gemv.flag_gemv_gemv_dejavu", "the reference's index-list composite: torch gate GEMV + SiLU + nonzero (host sync), index-list up and down",
         full + 2 * act_rows, lambda st: fg.flag_gemv_gemv_dejavu(x, st["wg_t"], st["wu"], st["wdt"], t)),
        ("cats_up_down", "gemv_gemv_triton (gate activations given)", 2 * act_rows, lambda st: capi.up_down(x, st["a"], st["wu"], st["wdt"], t, ws)),
        ("cats_gate_up", "fuse_gemv_flag_gemv", full + act_rows, lambda st: capi.gate_up(x, st["wg"], st["wu"], t)),
        ("cats_mlp", "the whole MLP into an fp16 y (no single reference op; what flash_gemv.cats_mlp and CatsMLP sp_method 3 call)",
         full + 2 * act_rows, lambda st: capi.mlp(x, st["wg"], st["wu"], st["wdt"], t, ws)),
        ("cats_mlp (y_f32)", "the C call behind flag_gemv_gemv_atomic / fuse_gemv_gemv_gemv / fuse_gemv_flag_gemv_gemv: adds into an fp32 y",
         full + 2 * act_rows, lambda st: capi.mlp(x, st["wg"], st["wu"], st["wdt"], t, ws, y_f32=out32)),
        ("cats_mlp_norm_residual", "norm -> mlp -> residual of the decoder layer", full + 2 * act_rows,
         lambda st: capi.mlp_norm_residual(x, nw, 1e-5, st["wg"], st["wu"], st["wdt"], t, ws)),
        ("cats_mlp_norm_residual_norm", "the same plus the next layer's input norm from the finishing launch", full + 2 * act_rows,
         lambda st: capi.mlp_norm_residual_norm(x, nw, 1e-5, st["wg"], st["wu"], st["wdt"], t, nw, 1e-5, ws)),
        ("cats_mlp_rowmajor_down", "flag_gemv_gemv, flag_gemv_gemv_inner*", 2 * full + act_rows, lambda st: capi.mlp_rowmajor_down(x, st["wg"], st["wu"], st["wd"], t, ws)),
    ]
    # the registered torch ops and the Python composites, called as a user of the reference's package calls them
    x3 = x.reshape(1, 1, H)
    act_fn = torch.nn.SiLU()
    flag1 = torch.zeros(1, I, dtype=torch.bool, device=dev)

    def zeroed(op):
        def call(st):
            out32.zero_()   # the contract of these ops: the caller zeroes the fp32 output
            return op(st)
        return call

    def module_call(method):
        from cats_amd.mlp import CatsMLP

        mods = []
        for st in sets:
            m = CatsMLP(H, I, dead_threshold=t, dtype=torch.float16, device="meta")
            m.gate_proj.weight = torch.nn.Parameter(st["wg"], requires_grad=False)
            m.up_proj.weight = torch.nn.Parameter(st["wu"], requires_grad=False)
            m.down_proj.weight = torch.nn.Parameter(st["wd"], requires_grad=False)
            m.is_profile, m.sp_method, m.wdown_t = True, method, st["wdt"]
            st[f"mod{method}"] = m
        return lambda st: st[f"mod{method}"](x3)

    table += [
        ("torch.ops.flash_gemv.flag_gemv_gemv_atomic", "same op of the reference (flash_gemv.py:30-31); fp32 output, accumulate",
         full + 2 * act_rows, lambda st: fg.flag_gemv_gemv_atomic(x, st["wg"], st["wu"], st["wdt"], out32, t)),
        ("out.zero_() + torch.ops.flash_gemv.flag_gemv_gemv_atomic", "the same with the zero fill its contract asks of the caller",
         full + 2 * act_rows, zeroed(lambda st: fg.flag_gemv_gemv_atomic(x, st["wg"], st["wu"], st["wdt"], out32, t))),
        ("torch.ops.flash_gemv.fuse_gemv_gemv_gemv", "same op of the reference (flash_gemv.py:15-16); fp32 output, accumulate",
         full + 2 * act_rows, lambda st: fg.fuse_gemv_gemv_gemv(x, st["wg"], st["wu"], st["wdt"], out32, t)),
        ("torch.ops.flash_gemv.fuse_gemv_flag_gemv_gemv", "same op of the reference (flash_gemv.py:12-13); also writes the flags",
         full + 2 * act_rows, lambda st: fg.fuse_gemv_flag_gemv_gemv(x, st["wg"], st["wu"], st["wdt"], out32, flag1, t)),
        ("torch.ops.flash_gemv.flag_gemv_gemv_inner", "same op of the reference (flash_gemv.py:36-37; sp_method 1): HF-layout dense down",
         2 * full + act_rows, lambda st: fg.flag_gemv_gemv_inner(x3, st["wg"], st["wu"], st["wd"], t)),
        ("SiLU(x @ Wgate) + flash_gemv.gemv_gemv_triton", "the reference microbenchmark's 'Triton' column as it times it "
         "(bench/profile_llama7B.py:16-18): torch gate GEMV and SiLU, then the sparse up / down call; this is the sp_method 2 path",
         full + 2 * act_rows, lambda st: fg.gemv_gemv_triton(x3, act_fn(torch.matmul(x3, st["wg_t"])), st["wu"], st["wdt"], t)),
        ("CatsMLP.forward sp_method 1", "module call (ugly_utils.py:877-886)", 2 * full + act_rows, module_call(1)),
        ("CatsMLP.forward sp_method 2", "module call (ugly_utils.py:887-894)", full + 2 * act_rows, module_call(2)),
        ("CatsMLP.forward sp_method 3", "module call: the whole MLP in the HIP kernels", full + 2 * act_rows, module_call(3)),
    ]
    res = []
    for name, replaces, nbytes, fn in table:
        if only and name not in only:
            continue
        us = timed(fn)
        res.append(dict(entry_point=name, replaces=replaces, us=round(us, 2), weight_MB=round(nbytes / 1e6, 1),
                        GBps=round(nbytes / us * 1e-3, 1), hbm_frac=round(nbytes / us * 1e-3 / HBM_PEAK_GBPS, 4)))
    del sets
    torch.cuda.empty_cache()
    return res


def cpu_baseline(torch, F, t):
    """The dense-masked PyTorch CATS MLP (the reference's sp_method 0 branch) in fp32 on the host cores."""
    from oracle import cats_oracle

    ncores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = min(ncores, int(os.environ.get("OMP_NUM_THREADS", ncores)))
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    wg = torch.randn(I, H, generator=g) * 0.02
    wu = torch.randn(I, H, generator=g) * 0.02
    wd = torch.randn(H, I, generator=g) * 0.02
    x = torch.randn(1, 1, H, generator=g)
    for _ in range(3):
        cats_oracle.torch_cats_mlp(x, wg, wu, wd, t)
    times = []
    t_end = time.perf_counter() + 12.0
    while len(times) < 20 or (time.perf_counter() < t_end and len(times) < 400):
        t0 = time.perf_counter()
        cats_oracle.torch_cats_mlp(x, wg, wu, wd, t)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    cpu = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                cpu = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": round(med * 1e6, 1), "unit": "us/layer", "cores": threads, "kind": "port",
            "sample": f"{len(times)} calls of the fp32 dense-masked PyTorch CATS MLP (4096->11008, batch 1), median; cpu: {cpu}",
            "GBps_dense_bytes": round(3 * 4 * H * I / med * 1e-9, 1)}


if __name__ == "__main__":
    main()
