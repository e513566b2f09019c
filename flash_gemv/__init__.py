"""flash_gemv -- the CATS sparse-MLP decode ops, backed by hand-written gfx950 HIP kernels.

Drop-in for the reference package of the same name (flash_gemv/flash_gemv/__init__.py): the same 14
``torch.ops.flash_gemv.*`` ops, the same Python wrappers and the same four composites.  Importing it loads
``_C.so`` from this directory (as the reference does, __init__.py:29-36) and fails loudly if that library is
missing -- there is no PyTorch fallback.  Triton is not imported.

Layout conventions (they differ between entry points, as in the reference):
  ``flag_gemv_gemv_triton`` / ``flag_gemv_gemv_dejavu`` / ``flag_gemv_gemv_fuse_dejavu`` take ``Wgate`` as
  (H, I) and compute ``x @ Wgate``; every ``torch.ops`` gate op takes (I, H).  ``Wup`` is (I, H) and
  ``Wdownt`` is neuron-major (I, H) everywhere in this file.
"""
import importlib.machinery
import os.path as osp

import torch

library = "_C"
spec = importlib.machinery.PathFinder().find_spec(library, [osp.dirname(__file__)])
if spec is not None:
    torch.ops.load_library(spec.origin)
else:
    raise ImportError(
        f"Could not find module '{library}' in {osp.dirname(__file__)}: build it with `python -m cats_amd.build`"
    )

from .flash_gemv import (  # noqa: E402
    fuse_gemv_cmp,
    fuse_gemv_flag,
    fuse_gemv_flag_gemv,
    fuse_gemv_flag_gemv_gemv,
    fuse_gemv_gemv_gemv,
    fuse_gemv_flag_batch,
    fuse_gemv_flag_local,
    fuse_flag_gemv_local,
    atomic_gemv,
    flag_gemv_gemv_atomic,
    flag_gemv_gemv,
    flag_gemv_gemv_inner,
    flag_gemv_gemv_inner_fp32,
    flag_gemv_gemv_inner_bf16,
)
from .kernels import (  # noqa: E402
    gather_gemv_elemul_flag_3d,
    gather_transposed_gemv_flag_3d,
    mistral_mlp_partial_sparse,
    mistral_mlp_sparse_direct_index_2d,
)

__version__ = "0.0.1"


def flag_gemv_gemv_triton(x, Wgate, Wup, Wdownt, threshold):
    """Gate in torch (``x @ Wgate``, Wgate (H, I)), then sparse up / down (reference __init__.py:38-43)."""
    act_fn = torch.nn.SiLU()
    x_1 = act_fn(torch.matmul(x, Wgate))
    # flags = |x_1| > threshold, sparse up, sparse down: one call (the flags are derived where x_1 is read)
    return gemv_gemv_triton(x, x_1, Wup, Wdownt, threshold)


def gemv_gemv_triton(x, x_1, Wup, Wdownt, threshold):
    """Sparse up / down given the gate activations x_1 (reference __init__.py:45-48).  The flags |x_1| > threshold are
    derived inside the up kernel (same strict comparison, threshold rounded to x_1's dtype as torch does)."""
    return torch.ops.flash_gemv.cats_up_down(x, x_1.contiguous(), Wup, Wdownt, threshold)


def flag_gemv_gemv_dejavu(x, Wgate, Wup, Wdownt, threshold):
    """Index-list baseline: x (1, H) 2-D (reference __init__.py:50-54)."""
    act_fn = torch.nn.SiLU()
    x_1 = act_fn(torch.matmul(x, Wgate))
    (_, idx) = torch.nonzero(torch.abs(x_1) > threshold, as_tuple=True)
    return mistral_mlp_partial_sparse(x, x_1[0][idx], Wup, Wdownt, idx)


def flag_gemv_gemv_fuse_dejavu(x, Wgate, Wup, Wdownt, threshold):
    """Index-list variant with the element-wise multiply fused into up (reference __init__.py:56-60)."""
    act_fn = torch.nn.SiLU()
    x_1 = act_fn(torch.matmul(x, Wgate))
    (_, idx) = torch.nonzero(torch.abs(x_1) > threshold, as_tuple=True)
    return mistral_mlp_sparse_direct_index_2d(x, x_1[0][idx], Wup, Wdownt, idx)


def cats_mlp(x, Wgate, Wup, Wdownt, threshold):
    """Whole CATS MLP in two HIP launches: gate + SiLU + threshold + sparse up, then sparse down.

    x (B, 1, H) or (B, H); Wgate, Wup, Wdownt all (I, H) (Wdownt neuron-major).  No reference counterpart as a
    single call: it is flag_gemv_gemv_triton with the gate GEMV fused in and (I, H) gate weights.
    """
    return torch.ops.flash_gemv.cats_mlp(x, Wgate, Wup, Wdownt, threshold)


def cats_mlp_norm_residual(h, norm_weight, eps, Wgate, Wup, Wdownt, threshold):
    """h + CATS_MLP(norm_weight * rms_norm(h, eps)) in the same two launches as cats_mlp.

    The three module calls at the end of the reference's decoder layer (residual = h; h = post_attention_layernorm(h);
    h = residual + mlp(h), experiments/models/sparse_silu/ugly_utils.py:1036-1057) for decode, batch * seq <= 16.
    """
    return torch.ops.flash_gemv.cats_mlp_norm_residual(h, norm_weight, eps, Wgate, Wup, Wdownt, threshold)


def cats_mlp_norm_residual_norm(h, norm_weight, eps, Wgate, Wup, Wdownt, threshold, next_norm_weight, next_eps):
    """(out, next): out as cats_mlp_norm_residual, next = next_norm_weight * rms_norm(out, next_eps) from the same two
    launches -- the input_layernorm of the following decoder layer (ugly_utils.py:1016-1057), or the final norm."""
    return torch.ops.flash_gemv.cats_mlp_norm_residual_norm(h, norm_weight, eps, Wgate, Wup, Wdownt, threshold, next_norm_weight, next_eps)


def cats_mlp_stats(x, Wgate, Wup, Wdownt, threshold):
    """cats_mlp that also returns the (B, I) bool flags and the number of neurons fetched (int32 tensor)."""
    return torch.ops.flash_gemv.cats_mlp_stats(x, Wgate, Wup, Wdownt, threshold)


__all__ = [
    "fuse_gemv_cmp",
    "fuse_gemv_flag",
    "fuse_gemv_flag_gemv",
    "fuse_gemv_flag_gemv_gemv",
    "fuse_gemv_gemv_gemv",
    "fuse_gemv_flag_batch",
    "fuse_gemv_flag_local",
    "fuse_flag_gemv_local",
    "atomic_gemv",
    "flag_gemv_gemv_atomic",
    "flag_gemv_gemv",
    "flag_gemv_gemv_inner",
    "flag_gemv_gemv_inner_fp32",
    "flag_gemv_gemv_inner_bf16",
    "flag_gemv_gemv_triton",
    "gemv_gemv_triton",
    "flag_gemv_gemv_fuse_dejavu",
    "flag_gemv_gemv_dejavu",
    "gather_gemv_elemul_flag_3d",
    "gather_transposed_gemv_flag_3d",
    "mistral_mlp_partial_sparse",
    "mistral_mlp_sparse_direct_index_2d",
    "cats_mlp",
    "cats_mlp_stats",
    "cats_mlp_norm_residual",
    "cats_mlp_norm_residual_norm",
]
