"""HIP-backed stand-ins for the reference's Triton wrappers (flash_gemv/flash_gemv/kernels.py).

Same function names, argument order, shape checks and return dtypes; the bodies call the gfx950 kernels
through ``torch.ops.flash_gemv`` -- nothing here imports Triton.

Flag-based pair (the path the reference publishes numbers for):
  gather_gemv_elemul_flag_3d      kernels.py:208-254   sparse up,   z = x_1 * (x . wup[j]) where flagged
  gather_transposed_gemv_flag_3d  kernels.py:416-462   sparse down, y = sum_j z[j] * weight[j, :]
Index-list (DejaVu-style) family (kernels.py:639-695, 1022-1094, 1236-1334): the kernels read the index list and
fetch exactly the listed weight rows (cats_up_index / cats_down_index); inputs and outputs stay compact, aligned
with the list.
"""
from typing import Optional

import torch


def gather_gemv_elemul_flag_3d(x: torch.Tensor, x_1: torch.Tensor, wup: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """z[b, 0, j] = x_1[b, 0, j] * (x[b, 0, :] . wup[j, :]) where idx[b, 0, j] (bool flags) is set, else 0.

    x (B, 1, H); x_1 (B, 1, I); wup (I, H); idx flags (B, 1, I).  Row j of wup is read iff any batch row flags it.
    Returns (B, 1, I) in x.dtype (the reference accumulates in fp32 and casts, kernels.py:236,254).
    """
    Z, N = wup.shape
    beam_width, seq_len, _ = x.shape
    assert seq_len == 1
    assert 1 <= beam_width <= 8  # reference: <= 4 (kernels.py:227)
    x = x.contiguous()
    x_1 = x_1.contiguous()
    if wup.stride(1) > 1:
        wup = wup.contiguous()
    assert x.dtype == wup.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {wup.dtype}"
    return torch.ops.flash_gemv.cats_up_flag(x, x_1, wup, idx.contiguous())


def gather_transposed_gemv_flag_3d(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """y[b, 0, :] = sum over flagged j of x[b, 0, j] * weight[j, :].

    x (B, 1, I); weight (I, H) neuron-major; idx flags (B, 1, I).  Returns (B, 1, H) in weight.dtype
    (fp32 accumulation, kernels.py:438-462).
    """
    Z, N = weight.shape
    beam_width, seq_len, _ = x.shape
    assert x.shape[2] == Z
    x = x.contiguous()
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    return torch.ops.flash_gemv.cats_down_flag(x, weight, idx.contiguous())


_ACTIVATIONS = {"id": 0, "relu": 1, "squared_relu": 2, "swish": 3}


def gather_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor, bias: Optional[torch.Tensor] = None,
                activation: str = "id") -> torch.Tensor:
    """y = activation(x @ weight[idx, :].T + bias[idx]); x (batch, N), weight (Z, N), idx (M,) -> (batch, M).

    The kernel reads the list and fetches exactly those rows (reference kernels.py:484-695): fp32 accumulation, bias,
    activation, one rounding at the store."""
    assert activation in _ACTIVATIONS
    Z, N = weight.shape
    batch, _ = x.shape
    assert x.shape == (batch, N)
    assert 1 <= batch <= 8  # reference: 1..4 (kernels.py:658)
    x = x.contiguous()
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (Z,), "Incompatible dimensions in between weight and bias"
        assert x.dtype == bias.dtype, f"Input and bias must have the same dtype, got {x.dtype} and {bias.dtype}"
    return torch.ops.flash_gemv.cats_up_index(x, weight, idx.contiguous(), bias, None, _ACTIVATIONS[activation])


def gather_transposed_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ weight[idx, :] + bias; x (batch, M), weight (Z, N), idx (M,) -> (batch, N) in x.dtype (kernels.py:1022-1094).
    Duplicate entries of idx add up, as they do with the reference's atomic adds."""
    Z, N = weight.shape
    (M,) = idx.shape
    batch, _ = x.shape
    assert x.shape == (batch, M)
    x = x.contiguous()
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (N,), "Incompatible dimensions in between weight and bias"
        assert x.dtype == bias.dtype, f"Input and bias must have the same dtype, got {x.dtype} and {bias.dtype}"
    return torch.ops.flash_gemv.cats_down_index(x, weight, idx.contiguous(), bias)


def gather_gemv_elemul_indirect_index_2d(x: torch.Tensor, x_1: torch.Tensor, Wup: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """y = x_1 * (x @ Wup[idx, :].T); x (1, N), x_1 (M,) compact activations, idx (M,) -> (1, M) (kernels.py:1236-1274):
    the multiply happens in fp32 inside the kernel, before the one rounding."""
    _, N = Wup.shape
    beam_width, _ = x.shape
    (M,) = idx.shape
    assert x.shape[1] == N
    assert beam_width == 1
    if Wup.stride(1) > 1:
        Wup = Wup.contiguous()
    return torch.ops.flash_gemv.cats_up_index(x.contiguous(), Wup, idx.contiguous(), None, x_1.contiguous().view(-1), 0)


def gather_transposed_gemv_indirect_index_2d(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """y = x @ weight[idx, :]; x (beam, M), idx (M,) -> (beam, N) in x.dtype (kernels.py:1276-1325)."""
    (M,) = idx.shape
    assert x.shape[1] == M
    return gather_transposed_gemv(x.contiguous(), weight, idx)


def mistral_mlp_partial_sparse(x, x_1, Wup, Wdownt, idx):
    x = gather_gemv(x, Wup, idx) * x_1
    x = gather_transposed_gemv(x, Wdownt, idx)
    return x


def mistral_mlp_sparse_direct_index_2d(x, x_1, Wup, Wdownt, idx):
    x_2 = gather_gemv_elemul_indirect_index_2d(x, x_1, Wup, idx)
    return gather_transposed_gemv_indirect_index_2d(x_2, Wdownt, idx)
