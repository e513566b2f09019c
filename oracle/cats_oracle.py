"""CPU oracle for the CATS sparse-MLP decode path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this
module; the product (``cats_amd/``, ``flash_gemv/``) never does and fails loudly without its HIP library.

Two independent restatements live here:

* ``torch_*`` -- the reference's PyTorch formulas on CPU tensors, line for line what
  ``experiments/models/sparse_silu/ugly_utils.py:895-899`` (dense-masked MLP), ``:80-92`` (SparseSiLU),
  ``:236-245`` (get_threshold), ``:829-831`` (histogram bins) and ``flash_gemv/flash_gemv/__init__.py:38-48``
  (flags) compute.  Every factor is a torch library routine (``F.linear``, ``F.silu``, ``abs``, ``<=``).
* ``c_*`` -- ctypes bindings of ``cats_oracle.c``, a plain-C restatement with explicit rounding points and
  double accumulation.  It does not use torch for arithmetic, so it cross-checks the formulas above and is
  the checker for dtype-exact questions (mask bits on identical gate values).

Parity status: the reference ships no golden vectors for this path; both restatements are pinned by the
closed forms and brute-force checks in ``tests/test_oracle.py``.  ``torch_rms_norm`` restates a routine of the
reference's dependency ``transformers``; it is pinned against the installed library's ``LlamaRMSNorm`` and against
closed forms there too.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libcats_oracle.so"
_lib = None

DTYPE_CODE = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def build(force: bool = False) -> Path:
    """Compile cats_oracle.c with gcc (seconds)."""
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < (_HERE / "cats_oracle.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(_HERE), "-B"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(str(_LIB_PATH))
        vp, i32, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.oracle_f32_to_f16.argtypes = [f32]; L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]; L.oracle_f16_to_f32.restype = f32
        L.oracle_f32_to_bf16.argtypes = [f32]; L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]; L.oracle_bf16_to_f32.restype = f32
        L.oracle_round.argtypes = [i32, f32]; L.oracle_round.restype = f32
        L.oracle_silu.argtypes = [f32]; L.oracle_silu.restype = f32
        L.oracle_gate.argtypes = [vp, vp, i32, i32, i32, i32, f32, vp, vp]; L.oracle_gate.restype = None
        L.oracle_mlp.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, vp, vp, vp, vp, vp]; L.oracle_mlp.restype = None
        L.oracle_sparse_up.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, vp, vp]; L.oracle_sparse_up.restype = None
        L.oracle_sparse_down.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]; L.oracle_sparse_down.restype = None
        L.oracle_compact.argtypes = [vp, i32, vp]; L.oracle_compact.restype = i32
        L.oracle_get_threshold.argtypes = [vp, vp, i32, f32, vp]; L.oracle_get_threshold.restype = f32
        L.oracle_histogram.argtypes = [vp, ctypes.c_size_t, vp, i32, vp]; L.oracle_histogram.restype = None
        _lib = L
    return _lib


def _cpu(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to("cpu").contiguous()


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


# ----------------------------------------------------------------------------------------------------------
# torch restatement (reference formulas on CPU tensors)
# ----------------------------------------------------------------------------------------------------------

def torch_cats_mlp(x, wgate, wup, wdown, threshold):
    """ugly_utils.py:895-899.  x (..., H); wgate, wup (I, H); wdown (H, I) -- nn.Linear layouts.  Returns (y, post_act
    before masking, dead mask)."""
    post_act = F.silu(F.linear(x, wgate))
    dead_neurons = post_act.abs() <= threshold
    act = post_act.clone()
    act[dead_neurons] = 0
    return F.linear(act * F.linear(x, wup), wdown), post_act, dead_neurons


def torch_dense_mlp(x, wgate, wup, wdown):
    """Plain SwiGLU MLP (HF LlamaMLP.forward): down(silu(gate(x)) * up(x))."""
    return F.linear(F.silu(F.linear(x, wgate)) * F.linear(x, wup), wdown)


def torch_rms_norm(h, weight, eps):
    """The post-attention norm of the decoder layer the reference patches (ugly_utils.py:1038 calls the HF module).
    The module lives in the reference's dependency transformers (pinned 4.36.2 in requirements.txt:40), class
    LlamaRMSNorm / MistralRMSNorm; its published forward is restated here: fp32 mean of squares, rsqrt(mean + eps),
    cast back to the input dtype, then the weight multiplies in that dtype."""
    v = h.to(torch.float32)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return weight * v.to(h.dtype)


def torch_layer_tail(h, norm_weight, eps, wgate, wup, wdown, threshold):
    """residual = h; h = norm(h); h = residual + mlp(h)  (ugly_utils.py:1036-1057, dense-masked MLP of :895-899)."""
    y, _, _ = torch_cats_mlp(torch_rms_norm(h, norm_weight, eps), wgate, wup, wdown, threshold)
    return h + y


def torch_gather_gemv(x, weight, idx, bias=None, activation="id", scale=None):
    """Index-list up projection, the reference's formula y = activation(x @ weight[idx, :].T + bias[idx])
    (flash_gemv/flash_gemv/kernels.py:645-652, activations :46-66 of the kernel's epilogue: relu, squared relu, swish),
    optionally times the compact gate activations (gather_gemv_elemul_indirect_index_2d, kernels.py:1242-1250).
    Evaluated in fp32 with one rounding to x.dtype at the end, as the Triton kernels accumulate and store."""
    xf, wf = _cpu(x).float(), _cpu(weight).float()
    idx = _cpu(idx).long()
    y = xf @ wf[idx, :].t()
    if bias is not None:
        y = y + _cpu(bias).float()[idx]
    if activation == "relu":
        y = torch.relu(y)
    elif activation == "squared_relu":
        y = torch.relu(y) ** 2
    elif activation == "swish":
        y = y * torch.sigmoid(y)
    elif activation != "id":
        raise ValueError(activation)
    if scale is not None:
        y = y * _cpu(scale).float().view(1, -1)
    return y.to(x.dtype)


def torch_gather_transposed_gemv(x, weight, idx, bias=None):
    """Index-list down projection, the reference's formula y = weight[idx, :]^T @ x + bias (kernels.py:1028-1034): every
    entry of idx contributes x[:, m] * weight[idx[m], :], so duplicate entries add up (the reference adds with atomics,
    kernels.py:842-850).  fp32 with one rounding to x.dtype at the end (kernels.py:1061-1094)."""
    xf, wf = _cpu(x).float(), _cpu(weight).float()
    idx = _cpu(idx).long()
    y = xf @ wf[idx, :]
    if bias is not None:
        y = y + _cpu(bias).float().view(1, -1)
    return y.to(x.dtype)


def torch_flags(x_1, threshold):
    """flash_gemv/flash_gemv/__init__.py:41,46 -- computed in x_1's dtype, the scalar is cast to it."""
    return torch.abs(x_1) > threshold


def torch_sparse_silu(x, threshold):
    """SparseSiLU.forward, ugly_utils.py:80-92: nn.Threshold keeps values strictly greater than the threshold."""
    act = F.silu(x)
    m = torch.nn.Threshold(threshold, 0)
    return m(act) - m(-act)


def histogram_bins(num_bins: int = 1000) -> torch.Tensor:
    """ugly_utils.py:829-831: [-inf, linspace(-1, 1, num_bins - 2), +inf] -> num_bins edges, num_bins - 1 bins."""
    inner = torch.linspace(-1, 1, num_bins - 2)
    return torch.cat([torch.tensor([-torch.inf]), inner, torch.tensor([torch.inf])])


def torch_get_threshold(bin_edges, histogram_counts, sparsity_level):
    """ugly_utils.py:236-245 (normalises a copy; the reference normalises in place)."""
    counts = histogram_counts.clone().float()
    counts /= counts.sum()
    idx = torch.searchsorted(counts.cumsum(0), torch.tensor(float(sparsity_level)), side="right")
    return bin_edges[idx]


def percentile_threshold(abs_act: torch.Tensor, sparsity: float) -> float:
    """Threshold at an exact percentile of |SiLU(gate)| (the calibration the benchmark configs name).  sparsity
    0 means "nothing is cut": any negative threshold does that, -1.0 is what the reference sweeps
    (flash_gemv/bench/final_profile_llama7B.sh:3)."""
    if sparsity <= 0.0:
        return -1.0
    flat = abs_act.float().flatten()
    k = int(round(sparsity * flat.numel()))
    k = min(max(k, 1), flat.numel())
    return float(torch.kthvalue(flat, k).values)


# ----------------------------------------------------------------------------------------------------------
# C restatement
# ----------------------------------------------------------------------------------------------------------

def c_round(dtype: torch.dtype, v: float) -> float:
    return float(lib().oracle_round(DTYPE_CODE[dtype], v))


def c_gate(x, wgate, threshold):
    """Returns (a (B, I) in dtype, flags (B, I) bool)."""
    x, wgate = _cpu(x), _cpu(wgate)
    H = x.shape[-1]
    B = x.numel() // H
    I = wgate.shape[0]
    a = torch.empty(B, I, dtype=x.dtype)
    flag = torch.empty(B, I, dtype=torch.uint8)
    lib().oracle_gate(_ptr(x), _ptr(wgate), B, H, I, DTYPE_CODE[x.dtype], float(threshold), _ptr(a), _ptr(flag))
    return a, flag.bool()


def c_mlp(x, wgate, wup, wdown, threshold, a_in=None, flag_in=None):
    """Dense-masked MLP; wdown (H, I).  With a_in / flag_in the gate stage is replaced by the given values.
    Returns dict(y (B, H), a (B, I), flag (B, I) bool, z (B, I))."""
    x, wgate, wup, wdown = _cpu(x), _cpu(wgate), _cpu(wup), _cpu(wdown)
    H = x.shape[-1]
    B = x.numel() // H
    I = wup.shape[0]
    assert wdown.shape == (H, I)
    y = torch.empty(B, H, dtype=x.dtype)
    a = torch.empty(B, I, dtype=x.dtype)
    z = torch.empty(B, I, dtype=x.dtype)
    flag = torch.empty(B, I, dtype=torch.uint8)
    if a_in is not None:
        a_in = _cpu(a_in).reshape(B, I).to(x.dtype).contiguous()
        flag_in = _cpu(flag_in).reshape(B, I).to(torch.uint8).contiguous()
    lib().oracle_mlp(_ptr(x), _ptr(wgate), _ptr(wup), _ptr(wdown), B, H, I, DTYPE_CODE[x.dtype], float(threshold),
                     _ptr(a_in), _ptr(flag_in), _ptr(y), _ptr(a), _ptr(flag), _ptr(z))
    return {"y": y, "a": a, "flag": flag.bool(), "z": z}


def c_sparse_up(x, wup, a, flag):
    """Returns fp32 (B, I)."""
    x, wup, a = _cpu(x), _cpu(wup), _cpu(a)
    flag = _cpu(flag).to(torch.uint8).contiguous()
    H = x.shape[-1]
    B = x.numel() // H
    I = wup.shape[0]
    out = torch.empty(B, I, dtype=torch.float32)
    lib().oracle_sparse_up(_ptr(x), _ptr(wup), _ptr(a), _ptr(flag), B, H, I, DTYPE_CODE[x.dtype], _ptr(out), None)
    return out


def c_sparse_down(z, wdown_t, flag):
    """Returns fp32 (B, H), starting from zero."""
    z, wdown_t = _cpu(z), _cpu(wdown_t)
    flag = _cpu(flag).to(torch.uint8).contiguous()
    I, H = wdown_t.shape
    B = z.numel() // I
    y = torch.zeros(B, H, dtype=torch.float32)
    lib().oracle_sparse_down(_ptr(z), _ptr(wdown_t), _ptr(flag), B, H, I, DTYPE_CODE[z.dtype], _ptr(y))
    return y


def c_compact(flag_row):
    flag_row = _cpu(flag_row).to(torch.uint8).flatten().contiguous()
    idx = torch.empty(flag_row.numel(), dtype=torch.int64)
    n = lib().oracle_compact(_ptr(flag_row), flag_row.numel(), _ptr(idx))
    return idx[:n].clone(), n


def c_get_threshold(bin_edges, counts, sparsity):
    edges = _cpu(bin_edges).float().contiguous()
    c = _cpu(counts).float().clone().contiguous()
    index = ctypes.c_int(0)
    t = lib().oracle_get_threshold(_ptr(edges), _ptr(c), c.numel(), float(sparsity), ctypes.byref(index))
    return float(t), index.value


def c_histogram(values, edges):
    v = _cpu(values).float().flatten().contiguous()
    e = _cpu(edges).float().contiguous()
    out = torch.empty(e.numel() - 1, dtype=torch.float32)
    lib().oracle_histogram(_ptr(v), v.numel(), _ptr(e), e.numel() - 1, _ptr(out))
    return out


def f16_bits_table() -> np.ndarray:
    """All 65536 fp16 bit patterns widened by the C oracle (for the exhaustive conversion test)."""
    L = lib()
    return np.array([L.oracle_f16_to_f32(i) for i in range(65536)], dtype=np.float32)
