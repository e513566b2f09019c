"""Python entry points of the registered ops: one callable per ``torch.ops.flash_gemv.<name>``, with the
reference's names, positional argument order and in-place conventions
(flash_gemv/flash_gemv/flash_gemv.py:3-43; registration in flash_gemv/csrc/fuse_gemv_cmp.cpp:87-102).

The callables are generated from the table below so that signature, documentation and dispatch target
sit in one place.  B = batch rows, H = hidden, I = intermediate; decode inputs are (B, 1, H) or (B, H).
``flag`` tensors are torch.bool.  Differences from the reference, all on the safe side: gate / up outputs
need no pre-zeroing (every element is written), shapes are not hard-wired to 4096 x 14336, and bad
arguments raise ``RuntimeError`` instead of ``exit(-1)``.
"""
import inspect

import torch

# name -> (parameters, what it computes)
_OPS = {
    "fuse_gemv_cmp": (
        ("input", "weight", "output", "idx", "threshold"),
        "Gate GEMV + SiLU + |a| > t for one row; writes the active activations compactly to output[:n] and their "
        "ascending neuron indices to idx[:n] (int64); returns n.  weight (I, H).",
    ),
    "fuse_gemv_flag": (
        ("input", "weight", "output", "flag", "threshold"),
        "Gate GEMV + SiLU; output (B, I) activations, flag (B, I) = |a| > t.  weight (I, H).",
    ),
    "fuse_gemv_flag_gemv": (
        ("input", "wgate", "wup", "output", "flag", "threshold"),
        "Gate then sparse up: output (B, I) = a * (x . wup[j]) where flagged, else 0.",
    ),
    "fuse_gemv_flag_gemv_gemv": (
        ("input", "wgate", "wup", "wdown", "output", "flag", "threshold"),
        "Whole MLP, wdown neuron-major (I, H); fp32 output (B, H) is accumulated into (zero it first).",
    ),
    "fuse_gemv_gemv_gemv": (
        ("input", "wgate", "wup", "wdown", "output", "threshold"),
        "Whole MLP, wdown neuron-major (I, H); fp32 output (B, H) is accumulated into (zero it first).",
    ),
    "fuse_gemv_flag_batch": (
        ("input", "weight", "output", "flag", "threshold"),
        "Batched form of fuse_gemv_flag.",
    ),
    "fuse_gemv_flag_local": (
        ("input", "weight", "output", "flag", "threshold"),
        "Shape-generic form of fuse_gemv_flag.",
    ),
    "fuse_flag_gemv_local": (
        ("input", "weight", "output", "flag"),
        "Sparse up in place: output holds the gate activations on entry and a * (x . weight[j]) (0 where not "
        "flagged) on return.  weight (I, H); rows without a flag in any batch row are not read.",
    ),
    "atomic_gemv": (
        ("input", "weight", "output", "flag"),
        "Sparse down: fp32 output (B, H) += sum over flagged j of input[b, j] * weight[j, :]; weight (I, H).",
    ),
    "flag_gemv_gemv_atomic": (
        ("input", "wgate", "wup", "wdown", "output", "threshold"),
        "Whole MLP with the sparse neuron-major down; fp32 output is accumulated into (zero it first).",
    ),
    "flag_gemv_gemv": (
        ("input", "wgate", "wup", "wdown", "output", "threshold"),
        "Whole MLP with the HF-layout wdown (H, I): dense down over the zero-filled intermediate; output (B, H).",
    ),
    "flag_gemv_gemv_inner": (
        ("input", "wgate", "wup", "wdown", "threshold"),
        "fp16 whole MLP, wdown (H, I); returns a new tensor shaped like input.",
    ),
    "flag_gemv_gemv_inner_fp32": (
        ("input", "wgate", "wup", "wdown", "threshold"),
        "fp32 whole MLP, wdown (H, I); returns a new tensor shaped like input.",
    ),
    "flag_gemv_gemv_inner_bf16": (
        ("input", "wgate", "wup", "wdown", "threshold"),
        "bf16 whole MLP, wdown (H, I); returns a new tensor shaped like input.",
    ),
}


def _entry_point(name, params, doc):
    def call(*args, **kwargs):
        bound = signature.bind(*args, **kwargs)
        return getattr(torch.ops.flash_gemv, name)(*bound.args)

    signature = inspect.Signature([inspect.Parameter(p, inspect.Parameter.POSITIONAL_OR_KEYWORD) for p in params])
    call.__name__ = call.__qualname__ = name
    call.__doc__ = doc
    call.__signature__ = signature
    return call


for _name, (_params, _doc) in _OPS.items():
    globals()[_name] = _entry_point(_name, _params, _doc)

__all__ = list(_OPS)
