"""A Llama-2-7B-architecture decoder around the CATS MLP, for the end-to-end decode measurement.

The reference never defines the decoder itself: it subclasses the HF Llama / Mistral models and only swaps
``layer.mlp`` (experiments/models/sparse_silu/ugly_utils.py:119-131).  What is restated here are the conventions
its tree spells out: decoder layer order ``h += attn(input_layernorm(h)); h += mlp(post_attention_layernorm(h))``
(ugly_utils.py:1016-1057), rotate-half RoPE and eager attention with an fp32 softmax
(experiments/models/sparse_mistral/sparse_silu.py:280-312, 756-832), and the timing rule of the patched
``generate()``: tokens 2..N only, tok/s = (N - 1) / elapsed (experiments/time_util_nofile.py:2902-2904, 2984-2994).
Everything except the MLP uses stock PyTorch-ROCm ops, so dense-vs-CATS differences isolate the MLP path.
The decode step is shape-static (fixed-size KV cache, position kept on the device) so it can be replayed from a
HIP graph.
"""
from __future__ import annotations

import math
import time
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from .mlp import CatsMLP


@dataclass
class DecoderConfig:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_layers: int = 32
    num_heads: int = 32
    vocab_size: int = 32000
    rms_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_len: int = 512

    @property
    def head_dim(self):
        return self.hidden_size // self.num_heads


class RMSNorm(nn.Module):
    def __init__(self, dim, eps, dtype, device):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype, device=device))
        self.eps = eps

    def forward(self, x):
        v = x.float()
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * v.to(x.dtype)


def rotate_half(x):
    d = x.shape[-1] // 2
    return torch.cat((-x[..., d:], x[..., :d]), dim=-1)


class Attention(nn.Module):
    def __init__(self, cfg: DecoderConfig, dtype, device):
        super().__init__()
        Hd = cfg.hidden_size
        kw = dict(bias=False, dtype=dtype, device=device)
        self.cfg = cfg
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = (nn.Linear(Hd, Hd, **kw) for _ in range(4))
        self.k_cache = None
        self.v_cache = None

    def reset_cache(self, batch, dtype, device):
        c = self.cfg
        self.k_cache = torch.zeros(batch, c.num_heads, c.max_len, c.head_dim, dtype=dtype, device=device)
        self.v_cache = torch.zeros_like(self.k_cache)

    def forward(self, h, cos, sin, positions, mask):
        """h (B, q, H); cos/sin (q, head_dim); positions (q,) int64 cache slots; mask (q, max_len) additive."""
        c = self.cfg
        B, q, _ = h.shape
        shp = (B, q, c.num_heads, c.head_dim)
        qh = self.q_proj(h).view(shp).transpose(1, 2)
        kh = self.k_proj(h).view(shp).transpose(1, 2)
        vh = self.v_proj(h).view(shp).transpose(1, 2)
        qh = qh * cos + rotate_half(qh) * sin
        kh = kh * cos + rotate_half(kh) * sin
        self.k_cache.index_copy_(2, positions, kh)
        self.v_cache.index_copy_(2, positions, vh)
        att = torch.matmul(qh, self.k_cache.transpose(2, 3)) / math.sqrt(c.head_dim) + mask
        att = torch.softmax(att, dim=-1, dtype=torch.float32).to(h.dtype)
        out = torch.matmul(att, self.v_cache).transpose(1, 2).reshape(B, q, c.hidden_size)
        return self.o_proj(out)


class DecoderLayer(nn.Module):
    def __init__(self, cfg, dtype, device):
        super().__init__()
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_eps, dtype, device)
        self.self_attn = Attention(cfg, dtype, device)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_eps, dtype, device)
        self.mlp = CatsMLP(cfg.hidden_size, cfg.intermediate_size, dtype=dtype, device=device)
        self.fuse_norm_residual = False  # decode only: post-attention norm and residual inside the two MLP launches
        self.fuse_next_norm = False      # and the norm the next layer starts with written by the same launches

    def forward(self, h, cos, sin, positions, mask, normed=None, next_norm=None):
        """normed: input_layernorm(h) if the previous layer's MLP launches already wrote it.  next_norm: the RMSNorm
        module that will consume this layer's output; with fuse_next_norm the return value is (h, next_norm(h))."""
        if normed is None:
            normed = self.input_layernorm(h)
        h = h + self.self_attn(normed, cos, sin, positions, mask)
        if self.fuse_norm_residual and h.shape[1] == 1 and self.mlp.is_profile and self.mlp.sp_method == 3:
            n = self.post_attention_layernorm
            if self.fuse_next_norm and next_norm is not None:
                return self.mlp.forward_norm_residual_norm(h, n.weight, n.eps, next_norm.weight, next_norm.eps)
            return self.mlp.forward_norm_residual(h, n.weight, n.eps)
        return h + self.mlp(self.post_attention_layernorm(h))


class LlamaDecoder(nn.Module):
    """Random-init decoder-only transformer in the Llama-2 layout (no biases, untied lm_head)."""

    def __init__(self, cfg: DecoderConfig, dtype=torch.float16, device="cuda", seed=0, init_std=0.02):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device)
        self.layers = nn.ModuleList(DecoderLayer(cfg, dtype, device) for _ in range(cfg.num_layers))
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_eps, dtype, device)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False, dtype=dtype, device=device)
        g = torch.Generator(device=device).manual_seed(seed)
        with torch.no_grad():
            for name, p in self.named_parameters():
                if p.dim() == 2:
                    p.copy_((torch.randn(p.shape, generator=g, device=device, dtype=torch.float32) * init_std).to(dtype))
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, device=device).float() / cfg.head_dim))
        ang = torch.outer(torch.arange(cfg.max_len, device=device).float(), inv)
        emb = torch.cat((ang, ang), dim=-1)
        self.register_buffer("cos_table", emb.cos().to(dtype), persistent=False)
        self.register_buffer("sin_table", emb.sin().to(dtype), persistent=False)

    def reset_cache(self, batch=1):
        dev = self.embed_tokens.weight.device
        for layer in self.layers:
            layer.self_attn.reset_cache(batch, self.dtype, dev)

    def forward(self, tokens, positions):
        """tokens (B, q) int64; positions (q,) int64 -> logits (B, q, vocab).  Causal over cache slots <= position."""
        cfg = self.cfg
        h = self.embed_tokens(tokens)
        cos, sin = self.cos_table[positions], self.sin_table[positions]
        slots = torch.arange(cfg.max_len, device=tokens.device)
        mask = torch.zeros(positions.numel(), cfg.max_len, dtype=self.dtype, device=tokens.device)
        mask.masked_fill_(slots[None, :] > positions[:, None], float("-inf"))
        normed = None
        for i, layer in enumerate(self.layers):
            next_norm = self.layers[i + 1].input_layernorm if i + 1 < len(self.layers) else self.norm
            out = layer(h, cos, sin, positions, mask, normed, next_norm)
            h, normed = out if isinstance(out, tuple) else (out, None)
        return self.lm_head(normed if normed is not None else self.norm(h))

    # ---- MLP mode switches ----
    def set_mlp_mode(self, mode: str):
        """"dense": plain SwiGLU.  "cats_torch": dense-masked PyTorch.  "cats": the two-launch HIP path.
        "cats_rowmajor": flag_gemv_gemv_inner* (HF-layout down).  "cats_split": torch gate + HIP sparse up / down.
        "cats_fused": "cats" with the post-attention norm and the residual add inside the two MLP launches.
        "cats_fused_next": "cats_fused" whose launches also write the next layer's input norm (the final norm after the
        last layer), so a decode step runs no stand-alone norm after the first layer's."""
        for layer in self.layers:
            m = layer.mlp
            layer.fuse_norm_residual = mode in ("cats_fused", "cats_fused_next")
            layer.fuse_next_norm = mode == "cats_fused_next"
            if layer.fuse_norm_residual:
                m.prepare_decode(3)
                continue
            if mode == "dense":
                m.is_profile, m.kill_sparse_swish_outputs = False, False
            elif mode == "cats_torch":
                m.is_profile, m.sp_method = True, 0
            elif mode in ("cats", "cats_split", "cats_rowmajor"):
                m.prepare_decode({"cats": 3, "cats_split": 2, "cats_rowmajor": 1}[mode])
            else:
                raise ValueError(mode)

    @torch.no_grad()
    def calibrate(self, sparsity: float, n_seq: int = 64, seq_len: int = 128, seed: int = 1, chunk: int = 8):
        """Per-layer thresholds at an exact percentile of |SiLU(gate)| over n_seq seeded random-token sequences, run
        through the dense model (the reference collects its histograms before thresholds are set)."""
        dev = self.embed_tokens.weight.device
        g = torch.Generator(device=dev).manual_seed(seed)
        acts = [[] for _ in self.layers]
        hooks = []
        for i, layer in enumerate(self.layers):
            hooks.append(layer.mlp.gate_proj.register_forward_hook(
                lambda mod, inp, out, i=i: acts[i].append(F.silu(out).abs().flatten().float()[::4].clone())))
        self.set_mlp_mode("dense")
        positions = torch.arange(seq_len, device=dev)
        for s in range(0, n_seq, chunk):
            toks = torch.randint(0, self.cfg.vocab_size, (min(chunk, n_seq - s), seq_len), generator=g, device=dev)
            self.reset_cache(toks.shape[0])
            self.forward(toks, positions)
        for h in hooks:
            h.remove()
        thresholds = []
        for i, layer in enumerate(self.layers):
            a = torch.cat(acts[i])
            k = max(1, int(round(sparsity * a.numel())))
            t = float(torch.kthvalue(a, k).values) if sparsity > 0 else -1.0
            layer.mlp.dead_threshold = t
            thresholds.append(t)
            acts[i] = None
        return thresholds

    @torch.no_grad()
    def generate_greedy(self, prompt, gen_len: int, use_graph: bool = True):
        """Greedy decode; returns (tokens (gen_len,), seconds for tokens 2..gen_len).  The first generated token
        comes from the prefill and is not timed (experiments/time_util_nofile.py:2902-2904)."""
        dev = prompt.device
        P = prompt.shape[1]
        assert P + gen_len <= self.cfg.max_len
        self.reset_cache(1)
        logits = self.forward(prompt, torch.arange(P, device=dev))
        tok = logits[:, -1].argmax(-1, keepdim=True)                     # token 1
        out = torch.zeros(gen_len, dtype=torch.int64, device=dev)
        out[0] = tok[0, 0]
        pos = torch.full((1,), P, dtype=torch.int64, device=dev)
        step_idx = torch.ones(1, dtype=torch.int64, device=dev)

        def step():
            lg = self.forward(tok, pos)
            nxt = lg[:, -1].argmax(-1, keepdim=True)
            tok.copy_(nxt)
            out.index_copy_(0, step_idx, nxt[0])
            pos.add_(1)
            step_idx.add_(1)

        graph = None
        if use_graph:
            snap = [t.clone() for t in (tok, pos, step_idx, out)]
            caches = [(l.self_attn.k_cache.clone(), l.self_attn.v_cache.clone()) for l in self.layers]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()                                                   # warm-up on the capture stream (allocations)
                side.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            for t, s in zip((tok, pos, step_idx, out), snap):            # rewind the two steps spent on capture
                t.copy_(s)
            for l, (k, v) in zip(self.layers, caches):
                l.self_attn.k_cache.copy_(k)
                l.self_attn.v_cache.copy_(v)
            del caches
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(gen_len - 1):
            if graph is not None:
                graph.replay()
            else:
                step()
        e1.record()
        torch.cuda.synchronize()
        return out.clone(), e0.elapsed_time(e1) * 1e-3


    @torch.no_grad()
    def decode_forced(self, prompt, forced):
        """Prefill, then feed the tokens of `forced` (n,) one per step whatever the model would have chosen.  Returns the
        fp32 logits of the n + 1 predictions (after the prompt and after each forced token), on the CPU.  Two MLP modes
        run over the same token sequence can be compared step by step this way; free-running greedy decoding cannot,
        because one flipped argmax changes every later input."""
        dev = prompt.device
        P = prompt.shape[1]
        n = int(forced.numel())
        assert P + n <= self.cfg.max_len
        self.reset_cache(1)
        out = [self.forward(prompt, torch.arange(P, device=dev))[0, -1].float().cpu()]
        for i in range(n):
            lg = self.forward(forced[i].view(1, 1), torch.full((1,), P + i, dtype=torch.int64, device=dev))
            out.append(lg[0, -1].float().cpu())
        return torch.stack(out)


def compare_modes(model, prompt, n_tokens=32, modes=("cats_torch", "cats", "cats_fused", "cats_fused_next")):
    """Agreement of the MLP modes on one model: the first mode decodes n_tokens greedily (eager); every mode is then
    run over that same token sequence and its per-step predictions are compared with the first mode's.
    Returns {mode: {"argmax_agreement": fraction of the n_tokens + 1 steps with the same top token,
                    "max_logit_diff": largest |logit difference| over all steps, "logit_scale": largest |logit|}}
    and the union sparsity the kernel path achieved per layer during its pass (from the kernel's own counts).

    A deep random-init network amplifies any difference in a mask bit: a neuron whose activation sits within a rounding
    step of the threshold may be kept by one gate GEMV and dropped by another that adds in a different order, and 32
    layers later logits have moved.  The entry "cats_torch_nudged" measures that floor on the reference itself: the
    dense-masked PyTorch MLP with every threshold raised by 0.1 %, against the same MLP with the thresholds as calibrated.
    What the kernels compute per call is checked without this amplification by layerwise_parity()."""
    model.set_mlp_mode(modes[0])
    ref_tokens, _ = model.generate_greedy(prompt, n_tokens, use_graph=False)
    ref = None
    res = {}
    sparsity = None

    def score(lg):
        # per-step distance from the reference run: rounding-level differences start small and grow as flipped mask bits
        # accumulate in the KV cache; a defect in one layer's arithmetic would be large from the first step on
        by_step = (lg - ref).abs().amax(-1)
        return {"argmax_agreement": round(float((lg.argmax(-1) == ref.argmax(-1)).float().mean()), 4),
                "max_logit_diff": round(float((lg - ref).abs().max()), 5), "logit_scale": round(float(ref.abs().max()), 4),
                "max_logit_diff_by_step": [round(float(v), 4) for v in by_step[:: max(1, by_step.numel() // 8)]]}

    for mode in modes:
        model.set_mlp_mode(mode)
        collect = mode == "cats"
        if collect:
            for layer in model.layers:
                layer.mlp.activate_stats(is_collect_histogram=False)
        lg = model.decode_forced(prompt, ref_tokens)
        if collect:
            sparsity = [layer.mlp.decode_union_sparsity() for layer in model.layers]
            for layer in model.layers:
                layer.mlp.deactivate_stats()
        if ref is None:
            ref = lg
            # the reference mode must reproduce its own greedy tokens when they are fed back to it
            res["self_consistent"] = bool(torch.equal(lg[:-1].argmax(-1), ref_tokens.cpu()))
            continue
        res[mode] = score(lg)
    model.set_mlp_mode(modes[0])
    saved = [layer.mlp.dead_threshold for layer in model.layers]
    for layer, t in zip(model.layers, saved):
        layer.mlp.dead_threshold = t * 1.001
    res[modes[0] + "_nudged"] = score(model.decode_forced(prompt, ref_tokens))
    for layer, t in zip(model.layers, saved):
        layer.mlp.dead_threshold = t
    return res, sparsity


@torch.no_grad()
def layerwise_parity(model, prompt, n_tokens=8, rtol=1e-2, atol=2e-3):
    """Every CATS MLP call of a decode run, checked in place: the dense-masked PyTorch model decodes n_tokens greedily
    and the input of each layer's MLP is recorded at every step; the HIP path is then run on exactly those inputs.
    Per call: y against the reference formula down(where(flag, a, 0) * up(x)) evaluated by PyTorch on the kernel's own
    gate activations and flags (identical gate values, so no mask tie can enter), to rtol / atol; the kernel's flags
    against |a| > t on its own activations, bit for bit; and against PyTorch's own gate GEMV, where they may differ
    only for activations within a rounding step of t (counted, and the largest distance from t reported)."""
    import flash_gemv

    model.set_mlp_mode("cats_torch")
    inputs = [[] for _ in model.layers]
    hooks = [layer.mlp.register_forward_pre_hook(lambda mod, args, i=i: inputs[i].append(args[0].detach().clone()) if args[0].shape[1] == 1 else None)
             for i, layer in enumerate(model.layers)]
    model.generate_greedy(prompt, n_tokens, use_graph=False)
    for h in hooks:
        h.remove()
    calls = bad = flips = flagged = own_rule_violations = 0
    worst = 0.0
    far = 0.0
    for layer, xs in zip(model.layers, inputs):
        m = layer.mlp
        t = float(m.dead_threshold)
        wdt = m.wdown_t if m.wdown_t is not None else m.down_proj.weight.detach().t().contiguous()
        for x in xs:
            y, flag, _ = flash_gemv.cats_mlp_stats(x, m.gate_proj.weight, m.up_proj.weight, wdt, t)
            a = torch.empty(1, 1, m.intermediate_size, dtype=x.dtype, device=x.device)
            f2 = torch.zeros(1, 1, m.intermediate_size, dtype=torch.bool, device=x.device)
            flash_gemv.fuse_gemv_flag_local(x, m.gate_proj.weight, a, f2, t)
            flag = flag.view_as(f2)
            own_rule_violations += int((flag != (a.abs() > t)).sum()) + int((flag != f2).sum())
            want = m.down_proj(torch.where(flag, a, torch.zeros_like(a)) * m.up_proj(x))
            err = (y.view_as(want).float() - want.float()).abs()
            ratio = float((err / (atol + rtol * want.float().abs())).max())
            worst = max(worst, ratio)
            bad += ratio > 1.0
            a_t = F.silu(m.gate_proj(x))
            diff = flag != (a_t.abs() > t)
            flips += int(diff.sum())
            if int(diff.sum()):
                far = max(far, float((a_t.float().abs() - t).abs()[diff].max()))
            flagged += flag.numel()
            calls += 1
    return {"mlp_calls_checked": calls, "calls_outside_tolerance": int(bad), "worst_error_over_tolerance": round(worst, 4),
            "tolerance": {"rtol": rtol, "atol": atol}, "flags_not_matching_own_activations": own_rule_violations,
            "mask_bits_differing_from_torch_gate": flips, "mask_bits_total": flagged, "largest_distance_from_threshold_of_a_differing_bit": far}


def bench_decode(prompt_len=128, gen_len=256, sparsity=0.5, num_layers=32, seed=0, use_graph=True, cfg=None):
    """Config 5: random-init fp16 Llama-2-7B architecture, batch 1, uniform-random prompt, greedy decode.
    Returns tok/s for the dense MLP and the CATS MLP (HIP path) and their ratio."""
    cfg = cfg or DecoderConfig(num_layers=num_layers, max_len=prompt_len + gen_len)
    t0 = time.time()
    model = LlamaDecoder(cfg, torch.float16, "cuda", seed=seed).eval()
    thresholds = model.calibrate(sparsity)
    g = torch.Generator(device="cuda").manual_seed(seed + 7)
    prompt = torch.randint(0, cfg.vocab_size, (1, prompt_len), generator=g, device="cuda")
    res = {"layers": cfg.num_layers, "prompt_len": prompt_len, "gen_len": gen_len, "target_sparsity": sparsity,
           "launch": "hipgraph" if use_graph else "stream", "setup_s": None}
    toks = {}
    for mode in ("dense", "cats", "cats_fused", "cats_fused_next"):
        model.set_mlp_mode(mode)
        model.generate_greedy(prompt, min(gen_len, 8), use_graph=False)          # warm-up (workspaces, kernels)
        out, secs = model.generate_greedy(prompt, gen_len, use_graph=use_graph)
        toks[mode] = out
        res[f"{mode}_tok_s"] = round((gen_len - 1) / secs, 2)
        res[f"{mode}_ms_per_token"] = round(secs / (gen_len - 1) * 1e3, 4)
    res["speedup"] = round(res["cats_tok_s"] / res["dense_tok_s"], 3)
    res["speedup_fused"] = round(res["cats_fused_tok_s"] / res["dense_tok_s"], 3)
    res["speedup_fused_next"] = round(res["cats_fused_next_tok_s"] / res["dense_tok_s"], 3)
    res["mean_threshold"] = round(sum(thresholds) / len(thresholds), 5)
    # correctness of what was just timed, untimed: the kernel modes against the dense-masked PyTorch MLP (the reference's
    # sp_method 0) over the same 32 greedy tokens, and the sparsity the kernels actually met while decoding them
    n_cmp = min(32, gen_len)
    agree, sparsity = compare_modes(model, prompt, n_cmp)
    res["layerwise_parity"] = layerwise_parity(model, prompt, 8)
    res["token_agreement"] = {"tokens": n_cmp + 1, "reference_mode": "cats_torch (dense-masked PyTorch MLP, sp_method 0)", **agree,
                              "free_running_common_prefix": {m: int((torch.cumprod((toks[m][:n_cmp] == toks["cats"][:n_cmp]).long(), 0)).sum())
                                                             for m in ("cats_fused", "cats_fused_next")}}
    res["achieved_sparsity"] = {"mean": round(sum(sparsity) / len(sparsity), 4), "min": round(min(sparsity), 4), "max": round(max(sparsity), 4),
                                "per_layer": [round(v, 4) for v in sparsity],
                                "definition": "1 - neurons fetched / I per MLP call, averaged over the compared decode steps (batch 1: union = row sparsity)"}
    res["setup_s"] = round(time.time() - t0, 1)
    return res


@torch.no_grad()
def cpu_decode_baseline(num_layers=4, gen_len=8, prompt_len=16, sparsity=0.5, threads=None):
    """The same greedy loop with the dense-masked PyTorch CATS MLP in fp32 on the host cores, on a reduced model
    (num_layers of the 32 layers, a short prompt, gen_len tokens); the per-token time is scaled to 32 layers."""
    if threads:
        torch.set_num_threads(threads)
    cfg = DecoderConfig(num_layers=num_layers, max_len=prompt_len + gen_len)
    model = LlamaDecoder(cfg, torch.float32, "cpu", seed=0).eval()
    model.calibrate(sparsity, n_seq=2, seq_len=prompt_len, chunk=2)
    model.set_mlp_mode("cats_torch")
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, cfg.vocab_size, (1, prompt_len), generator=g)
    model.reset_cache(1)
    logits = model.forward(prompt, torch.arange(prompt_len))
    tok = logits[:, -1].argmax(-1, keepdim=True)
    t0 = time.perf_counter()
    for i in range(gen_len - 1):
        logits = model.forward(tok, torch.tensor([prompt_len + i]))
        tok = logits[:, -1].argmax(-1, keepdim=True)
    per_tok = (time.perf_counter() - t0) / (gen_len - 1)
    # the whole measured per-token time (embedding and lm_head included) is scaled by 32 / num_layers: a little
    # pessimistic for the CPU, which is the baseline here
    return {"tok_s_32_layers_extrapolated": round(1.0 / (per_tok * 32 / num_layers), 3), "measured_layers": num_layers,
            "measured_tokens": gen_len - 1, "ms_per_token_measured": round(per_tok * 1e3, 2), "threads": torch.get_num_threads()}
