"""CATS MLP modules: the host-side mirror of ``LlamaSparseSiluMLP`` / ``MistralSparseSiluMLP``
(experiments/models/sparse_silu/ugly_utils.py:476-566, 807-960) for the decode path, plus the model surgery and
threshold helpers that sit around them (``apply_sparse_silu_mlp`` :119-131, ``get_threshold`` :236-245,
``set_sparse_threshold`` :257-273, ``save_act_hist`` / ``load_act_hist`` :399-433, ``activate_stats`` :846-850).

Same attribute switches as the reference, poked onto the module by the harness
(experiments/bench_sparse_inference_llama.py:66-77): ``is_profile``, ``sp_method``, ``wdown_t``,
``dead_threshold``, ``is_stats``, ``is_collect_histogram``, ``kill_sparse_swish_outputs``.

``sp_method`` when ``is_profile`` and the input is a decode step (``x.shape[1] == 1``):
  0  dense-masked PyTorch (the reference's own fallback and the parity oracle's formula)
  1  ``flash_gemv.flag_gemv_gemv_inner{,_fp32,_bf16}`` on the HF-layout down weight (dense down)
  2  ``flash_gemv.gemv_gemv_triton``: gate in torch, sparse up / down in HIP over ``wdown_t``
  3  ``flash_gemv.cats_mlp``: everything in two HIP launches over ``wdown_t`` (no reference counterpart: the
     reference has no single call with the gate fused in and neuron-major down weights)
Prefill (``x.shape[1] > 1``) always takes the dense-masked branch, as in the reference (:900-904).
"""
from __future__ import annotations

import os
import time
from typing import Iterable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

NUM_BINS = 1000


def histogram_bins(num_bins: int = NUM_BINS) -> torch.Tensor:
    """[-inf, linspace(-1, 1, num_bins - 2), +inf] (ugly_utils.py:829-831)."""
    inner = torch.linspace(-1, 1, num_bins - 2)
    return torch.cat([torch.tensor([-torch.inf]), inner, torch.tensor([torch.inf])])


def get_threshold(bin_edges: torch.Tensor, histogram_counts: torch.Tensor, sparsity_level: float):
    """ugly_utils.py:236-245.  Normalises ``histogram_counts`` in place like the reference and returns the left edge
    of the first bin whose cumulative mass exceeds ``sparsity_level`` (a 0-dim tensor)."""
    assert len(bin_edges.shape) == len(histogram_counts.shape) == 1, "bin_edges and histogram are expected to be 1-dimensional."
    histogram_counts /= histogram_counts.sum()
    threshold_idx = torch.searchsorted(histogram_counts.cumsum(0), sparsity_level, side="right")
    return bin_edges[threshold_idx]


class SparseSiLU(nn.SiLU):
    """SiLU followed by a symmetric dead zone: values with |a| <= threshold become 0 (ugly_utils.py:80-92)."""

    def __init__(self, threshold):
        super().__init__()
        self.set_new_threshold(threshold)

    def set_new_threshold(self, threshold):
        self.threshold = threshold
        self.m = nn.Threshold(float(threshold), 0)

    def forward(self, x):
        act = super().forward(x)
        return self.m(act) - self.m(-act)


class CatsMLP(nn.Module):
    """SwiGLU MLP with CATS thresholding.  ``gate_proj`` / ``up_proj`` / ``down_proj`` are bias-free ``nn.Linear``
    layers in the HF layout, so an existing ``LlamaMLP`` / ``MistralMLP`` can hand its three projections over."""

    def __init__(self, hidden_size: int, intermediate_size: int, dead_threshold: float = 0.0, dtype=None, device=None):
        super().__init__()
        kw = dict(bias=False, dtype=dtype, device=device)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, **kw)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, **kw)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, **kw)
        self.act_fn = nn.SiLU()
        # switches (same names as the reference)
        self.is_profile = False
        self.sp_method = 0
        self.wdown_t: Optional[torch.Tensor] = None
        self.kill_sparse_swish_outputs = False
        self.dead_threshold = dead_threshold
        self.sparse_act_fn = SparseSiLU(threshold=dead_threshold)
        # running statistics
        self.is_stats = False
        self.is_collect_histogram = False
        self.dead_percentage = 0
        self.agg_sparsity = 0
        self.visit_counts = 0
        self.count = 0
        self.t = 0
        # kernel path while is_stats: [neurons fetched, calls] as one device int64 pair.  Both are added to on the device,
        # so a HIP-graph replay of the decode step counts the call as well as the neurons.
        self.decode_fetched: Optional[torch.Tensor] = None
        self.histogram_bins = histogram_bins()
        self.pre_act_hist_counts = torch.zeros(NUM_BINS - 1)
        self.post_act_hist_counts = torch.zeros(NUM_BINS - 1)

    # ---- statistics (ugly_utils.py:846-860) ----
    def activate_stats(self, is_collect_histogram: bool = True):
        self.is_stats = True
        self.dead_percentage = 0
        self.visit_counts = 0
        self.decode_fetched = None
        self.is_collect_histogram = is_collect_histogram

    def deactivate_stats(self):
        self.is_stats = False

    def decode_union_sparsity(self) -> Optional[float]:
        """1 - (neurons fetched per call) / I over the kernel-path calls made while is_stats; None if there were none.
        This is what the reference's microbenchmark reports as sparsity (flash_gemv/bench/profile_llama7B.py:56,72)."""
        if self.decode_fetched is None:
            return None
        fetched, calls = (int(v) for v in self.decode_fetched.tolist())
        if calls == 0:
            return None
        return 1.0 - fetched / (calls * self.intermediate_size)

    def collect_stats(self, pre_activation, post_activation):
        start_time = time.time()
        pre_activation = pre_activation.float().cpu().detach()
        post_activation = post_activation.float().cpu().detach()
        self.pre_act_hist_counts += torch.histogram(pre_activation, bins=self.histogram_bins)[0]
        self.post_act_hist_counts += torch.histogram(torch.abs(post_activation), bins=self.histogram_bins)[0]
        self.t += time.time() - start_time

    # ---- decode-path preparation (bench_sparse_inference_llama.py:76) ----
    def prepare_decode(self, sp_method: int = 3):
        """Turn on the kernel path: one-time neuron-major copy of the down weight for methods 2 and 3."""
        self.is_profile = True
        self.sp_method = sp_method
        if sp_method in (2, 3):
            self.wdown_t = self.down_proj.weight.detach().t().contiguous()
        return self

    def forward_norm_residual(self, h, norm_weight, eps):
        """``h + self(norm_weight * rms_norm(h, eps))`` for the decode kernel path (sp_method 3): the post-attention
        norm is applied while the gate kernel stages h, the residual is added where the down kernel writes."""
        if not (self.is_profile and self.sp_method == 3 and h.shape[1] == 1):
            raise RuntimeError("CatsMLP.forward_norm_residual: decode path only (prepare_decode(3), one token per row)")
        if self.wdown_t is None:
            raise RuntimeError("CatsMLP: sp_method 3 needs wdown_t (call prepare_decode() once after loading weights)")
        import flash_gemv

        return flash_gemv.cats_mlp_norm_residual(h, norm_weight, float(eps), self.gate_proj.weight, self.up_proj.weight,
                                                 self.wdown_t, float(self.dead_threshold))

    def forward_norm_residual_norm(self, h, norm_weight, eps, next_norm_weight, next_eps):
        """``(out, next)``: ``out`` as forward_norm_residual, ``next = next_norm_weight * rms_norm(out, next_eps)`` -- the
        norm the following layer (or the model's final norm) would start with, written by the same two launches."""
        if not (self.is_profile and self.sp_method == 3 and h.shape[1] == 1):
            raise RuntimeError("CatsMLP.forward_norm_residual_norm: decode path only (prepare_decode(3), one token per row)")
        if self.wdown_t is None:
            raise RuntimeError("CatsMLP: sp_method 3 needs wdown_t (call prepare_decode() once after loading weights)")
        import flash_gemv

        return flash_gemv.cats_mlp_norm_residual_norm(h, norm_weight, float(eps), self.gate_proj.weight, self.up_proj.weight,
                                                      self.wdown_t, float(self.dead_threshold), next_norm_weight, float(next_eps))

    def _dense_masked(self, x):
        post_act = self.act_fn(self.gate_proj(x))
        dead_neurons = post_act.abs() <= self.dead_threshold
        post_act[dead_neurons] = 0
        return self.down_proj(post_act * self.up_proj(x))

    def forward(self, x, sp_mask: torch.Tensor = None):
        if sp_mask is not None:  # ugly_utils.py:872-875
            return self.down_proj(self.sparse_act_fn(self.gate_proj(x) * sp_mask) * self.up_proj(x))

        if self.is_profile:
            if x.shape[1] == 1 and self.sp_method in (1, 2, 3):
                import flash_gemv  # raises if the HIP op library is missing: there is no fallback for these methods

                t = float(self.dead_threshold)
                if self.sp_method == 1:
                    fn = {torch.float16: flash_gemv.flag_gemv_gemv_inner, torch.bfloat16: flash_gemv.flag_gemv_gemv_inner_bf16,
                          torch.float32: flash_gemv.flag_gemv_gemv_inner_fp32}[x.dtype]
                    return fn(x, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, t)
                if self.wdown_t is None:
                    raise RuntimeError("CatsMLP: sp_method 2/3 need wdown_t (call prepare_decode() once after loading weights)")
                if self.sp_method == 2:
                    return flash_gemv.gemv_gemv_triton(x, self.act_fn(self.gate_proj(x)), self.up_proj.weight, self.wdown_t, t)
                if self.is_stats:
                    # decode-time sparsity bookkeeping (the reference's agg_sparsity, ugly_utils.py:929-937, for the
                    # kernel path): the kernel reports how many neurons it fetched -- the union over the rows -- and
                    # the running total stays on the device, so nothing here waits for the GPU
                    y, _, fetched = flash_gemv.cats_mlp_stats(x, self.gate_proj.weight, self.up_proj.weight, self.wdown_t, t)
                    if self.decode_fetched is None or self.decode_fetched.device != fetched.device:
                        self.decode_fetched = torch.zeros(2, dtype=torch.int64, device=fetched.device)
                    self.decode_fetched[0] += fetched.reshape(())
                    self.decode_fetched[1] += 1
                    return y
                return flash_gemv.cats_mlp(x, self.gate_proj.weight, self.up_proj.weight, self.wdown_t, t)
            return self._dense_masked(x)

        # training / evaluation path (ugly_utils.py:922-946), statistics and histogram collection included
        self.count += 1
        pre_act = self.gate_proj(x)
        post_act = self.act_fn(pre_act)
        if self.kill_sparse_swish_outputs:
            dead_neurons = post_act.abs() <= self.dead_threshold
            dead_percentage = dead_neurons.float().mean()
            agg_sparsity = dead_neurons.all(dim=0).float().mean()
            if self.is_stats:
                self.dead_percentage = (self.dead_percentage * self.visit_counts + dead_percentage) / (self.visit_counts + 1)
                self.agg_sparsity = (self.agg_sparsity * self.visit_counts + agg_sparsity) / (self.visit_counts + 1)
                self.visit_counts += 1
                if self.is_collect_histogram:
                    self.collect_stats(pre_act, post_act)
            post_act[dead_neurons] = 0
        return self.down_proj(post_act * self.up_proj(x))


# ---- model-level helpers ------------------------------------------------------------------------------------------

def _layers(model) -> Iterable[nn.Module]:
    inner = getattr(model, "model", model)
    return inner.layers


def apply_cats_mlp(model, dead_threshold: float = 0.0):
    """Swap every ``layer.mlp`` for a CatsMLP that shares its three projections (ugly_utils.py:119-131)."""
    for layer in _layers(model):
        old = layer.mlp
        if isinstance(old, CatsMLP):
            continue
        w = old.gate_proj.weight
        new = CatsMLP(w.shape[1], w.shape[0], dead_threshold=dead_threshold, dtype=w.dtype, device="meta")
        new.gate_proj, new.up_proj, new.down_proj = old.gate_proj, old.up_proj, old.down_proj
        layer.mlp = new
    return model


def activate_stats(model, is_collect_histogram: bool = True):
    for layer in _layers(model):
        if isinstance(layer.mlp, CatsMLP):
            layer.mlp.activate_stats(is_collect_histogram)
            layer.mlp.kill_sparse_swish_outputs = True


def deactivate_stats(model):
    for layer in _layers(model):
        if isinstance(layer.mlp, CatsMLP):
            layer.mlp.deactivate_stats()


def set_sparse_threshold(model, sparsity_level: float):
    """Per-layer threshold from each layer's |SiLU(gate)| histogram (ugly_utils.py:257-273)."""
    for layer in _layers(model):
        mlp = layer.mlp
        if isinstance(mlp, CatsMLP) and mlp.is_stats:
            mlp.dead_threshold = get_threshold(mlp.histogram_bins, mlp.post_act_hist_counts, sparsity_level)
            mlp.sparse_act_fn.set_new_threshold(mlp.dead_threshold)


def set_thresholds(model, thresholds):
    """Apply a ``config.thresholds`` list (experiments/pretrain_sparse_model.py:434-435; ugly_utils.py:786-792)."""
    for layer, t in zip(_layers(model), thresholds):
        if isinstance(layer.mlp, CatsMLP):
            layer.mlp.dead_threshold = t
            layer.mlp.sparse_act_fn.set_new_threshold(t)
            layer.mlp.kill_sparse_swish_outputs = True


def get_thresholds(model):
    return [float(layer.mlp.dead_threshold) for layer in _layers(model) if isinstance(layer.mlp, CatsMLP)]


def save_act_hist(model, filename: str):
    """``{layer_index: (bins, pre_counts, post_counts)}`` via torch.save -- the reference's format (ugly_utils.py:399-413)."""
    d = os.path.dirname(filename)
    if d:
        os.makedirs(d, exist_ok=True)
    act_dict = {}
    for i, layer in enumerate(_layers(model)):
        if isinstance(layer.mlp, CatsMLP) and layer.mlp.is_stats:
            act_dict[i] = (layer.mlp.histogram_bins, layer.mlp.pre_act_hist_counts, layer.mlp.post_act_hist_counts)
    torch.save(act_dict, filename)


def load_act_hist(model, filename: str):
    """Inverse of save_act_hist (ugly_utils.py:416-433).  The file holds tensors only, so it is read with
    ``weights_only=True``."""
    assert os.path.exists(filename), f"{filename} does not exist when loading pre/post-activation histogram of the CATS MLP."
    act_dict = torch.load(filename, weights_only=True)
    for i, layer in enumerate(_layers(model)):
        if isinstance(layer.mlp, CatsMLP) and layer.mlp.is_stats:
            layer.mlp.histogram_bins, layer.mlp.pre_act_hist_counts, layer.mlp.post_act_hist_counts = act_dict[i]


def prepare_decode(model, sp_method: int = 3):
    """``is_profile`` / ``sp_method`` / ``wdown_t`` on every CATS MLP (bench_sparse_inference_llama.py:66-77)."""
    for layer in _layers(model):
        if isinstance(layer.mlp, CatsMLP):
            layer.mlp.prepare_decode(sp_method)
    return model
