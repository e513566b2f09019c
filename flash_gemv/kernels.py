"""HIP-backed stand-ins for the reference's Triton wrappers (flash_gemv/flash_gemv/kernels.py).

Same function names, argument order, shape checks and return dtypes; the bodies call the gfx950 kernels
through ``torch.ops.flash_gemv`` -- nothing here imports Triton.

Flag-based pair (the path the reference publishes numbers for):
  gather_gemv_elemul_flag_3d      kernels.py:208-254   sparse up,   z = x_1 * (x . wup[j]) where flagged
  gather_transposed_gemv_flag_3d  kernels.py:416-462   sparse down, y = sum_j z[j] * weight[j, :]
Index-list (DejaVu-style) family (kernels.py:639-695, 1022-1094, 1236-1334): the sorted index list is
scattered into a flag row and the same two kernels run; results are gathered back to the list order.
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


def _flags_from_index(idx: torch.Tensor, rows: int, width: int) -> torch.Tensor:
    flags = torch.zeros(rows, width, dtype=torch.bool, device=idx.device)
    flags[:, idx] = True
    return flags


def gather_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor, bias: Optional[torch.Tensor] = None,
                activation: str = "id") -> torch.Tensor:
    """y = activation(x @ weight[idx, :].T + bias[idx]); x (batch, N), weight (Z, N), idx (M,) -> (batch, M)."""
    assert activation in ["id", "relu", "squared_relu", "swish"]
    Z, N = weight.shape
    batch, _ = x.shape
    assert x.shape == (batch, N)
    assert 1 <= batch <= 8  # reference: 1..4 (kernels.py:658)
    x = x.contiguous()
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
    flags = _flags_from_index(idx, batch, Z)
    ones = torch.ones(batch, Z, dtype=x.dtype, device=x.device)
    y = torch.ops.flash_gemv.cats_up_flag(x, ones, weight, flags)[:, idx]
    if bias is not None:
        assert bias.shape == (Z,), "Incompatible dimensions in between weight and bias"
        y = y + bias[idx]
    if activation == "relu":
        y = torch.relu(y)
    elif activation == "squared_relu":
        y = torch.relu(y) ** 2
    elif activation == "swish":
        y = torch.nn.functional.silu(y)
    return y


def gather_transposed_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ weight[idx, :] + bias; x (batch, M), weight (Z, N), idx (M,) -> (batch, N)."""
    Z, N = weight.shape
    batch, M = x.shape
    assert idx.shape == (M,)
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
    flags = _flags_from_index(idx, batch, Z)
    dense = torch.zeros(batch, Z, dtype=x.dtype, device=x.device)
    dense[:, idx] = x
    y = torch.ops.flash_gemv.cats_down_flag(dense, weight, flags)
    if bias is not None:
        y = y + bias
    return y


def gather_gemv_elemul_indirect_index_2d(x: torch.Tensor, x_1: torch.Tensor, Wup: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """y = x_1 * (x @ Wup[idx, :].T); x (1, N), x_1 (M,) compact activations, idx (M,) -> (1, M)."""
    _, N = Wup.shape
    beam_width, _ = x.shape
    assert x.shape[1] == N
    assert beam_width == 1
    return gather_gemv(x, Wup, idx) * x_1


def gather_transposed_gemv_indirect_index_2d(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """y = x @ weight[idx, :]; x (beam, M), idx (M,) -> (beam, N) in x.dtype."""
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
