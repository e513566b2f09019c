"""CPU-side checks of the drop-in boundary: the C-ABI library loads, exports every symbol the header declares,
validates arguments without touching a GPU, and the flash_gemv package registers the reference's op surface."""
import ctypes
import inspect
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "cats_gemv.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cats_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cats_amd import capi

    L = capi.lib()
    syms = declared_symbols()
    assert set(syms) == set(capi.SYMBOLS), "capi.SYMBOLS and include/cats_gemv.h disagree"
    for s in syms:
        assert hasattr(L, s), f"{s} is declared but not exported"
    assert L.cats_version() >= 100


def test_argument_validation_needs_no_gpu():
    """Every check happens before any HIP call, so the status codes can be exercised on a CPU-only host."""
    from cats_amd import capi

    L = capi.lib()
    buf = (ctypes.c_char * 4096)()
    base = ctypes.addressof(buf)
    p = ctypes.c_void_p((base + 255) // 256 * 256)      # 256-aligned fake pointer, never dereferenced on the host
    odd = ctypes.c_void_p(p.value + 2)
    big = 1 << 30
    assert L.cats_gate_flag(p, p, p, p, 1, 64, 96, 9, 0.1, None) == 1            # dtype
    assert L.cats_gate_flag(p, p, p, p, 0, 64, 96, 0, 0.1, None) == 4            # batch
    assert L.cats_gate_flag(p, p, p, p, 17, 64, 96, 0, 0.1, None) == 4
    assert L.cats_gate_flag(p, p, p, p, 1, 0, 96, 0, 0.1, None) == 2             # shape
    assert L.cats_gate_flag(p, p, p, p, 1, 60, 96, 0, 0.1, None) == 3            # row pitch 120 B
    assert L.cats_gate_flag(p, p, p, p, 1, 62, 96, 2, 0.1, None) == 3            # fp32 row pitch 248 B
    assert L.cats_gate_flag(odd, p, p, p, 1, 64, 96, 0, 0.1, None) == 3          # misaligned x
    assert L.cats_gate_flag(None, p, p, p, 1, 64, 96, 0, 0.1, None) == 5         # null
    assert L.cats_gate_flag(p, p, None, None, 1, 64, 96, 0, 0.1, None) == 5      # no output requested
    assert L.cats_mlp(p, p, p, p, p, None, None, None, 1, 64, 96, 0, 0.1, None, 0, None) == 6     # no workspace
    assert L.cats_mlp(p, p, p, p, p, None, None, None, 1, 64, 96, 0, 0.1, p, 16, None) == 6      # too small
    assert L.cats_mlp(p, p, p, p, p, p, None, None, 1, 64, 96, 0, 0.1, p, big, None) == 5        # both outputs given
    assert L.cats_mlp(p, p, p, p, None, None, None, None, 1, 64, 96, 0, 0.1, p, big, None) == 5  # neither
    assert L.cats_mlp_rowmajor_down(p, p, p, p, p, 1, 64, 100, 0, 0.1, p, big, None) == 3        # wdown rows 200 B
    assert L.cats_down_flag(p, p, p, None, None, 1, 64, 96, 0, p, big, None) == 5
    for code in range(8):
        assert capi.status_string(code) != "unknown status"
    assert capi.status_string(99) == "unknown status"


def test_workspace_size_depends_on_layer_shape_only():
    from cats_amd import capi

    L = capi.lib()
    a = L.cats_workspace_bytes(1, 4096, 11008)
    assert a == L.cats_workspace_bytes(8, 4096, 11008) and a % 256 == 0
    assert L.cats_workspace_bytes(1, 4096, 14336) > a
    assert L.cats_workspace_bytes(0, 4096, 11008) == 0


def test_flash_gemv_package_surface():
    import flash_gemv

    ops = ["fuse_gemv_cmp", "fuse_gemv_flag", "fuse_gemv_flag_gemv", "fuse_gemv_flag_gemv_gemv", "fuse_gemv_gemv_gemv",
           "fuse_gemv_flag_batch", "fuse_gemv_flag_local", "fuse_flag_gemv_local", "atomic_gemv", "flag_gemv_gemv_atomic",
           "flag_gemv_gemv", "flag_gemv_gemv_inner", "flag_gemv_gemv_inner_fp32", "flag_gemv_gemv_inner_bf16"]
    composites = ["flag_gemv_gemv_triton", "gemv_gemv_triton", "flag_gemv_gemv_fuse_dejavu", "flag_gemv_gemv_dejavu"]
    for name in ops + composites:
        assert callable(getattr(flash_gemv, name)), name
        assert name in flash_gemv.__all__
    assert all(isinstance(n, str) for n in flash_gemv.__all__)      # the reference lists function objects here
    for name in ops:
        assert hasattr(torch.ops.flash_gemv, name), f"torch.ops.flash_gemv.{name} is not registered"
    # positional signatures of the reference wrappers (flash_gemv/flash_gemv/flash_gemv.py:3-43)
    want = {
        "fuse_gemv_cmp": ["input", "weight", "output", "idx", "threshold"],
        "fuse_gemv_flag_gemv_gemv": ["input", "wgate", "wup", "wdown", "output", "flag", "threshold"],
        "fuse_flag_gemv_local": ["input", "weight", "output", "flag"],
        "atomic_gemv": ["input", "weight", "output", "flag"],
        "flag_gemv_gemv_inner_bf16": ["input", "wgate", "wup", "wdown", "threshold"],
        "gemv_gemv_triton": ["x", "x_1", "Wup", "Wdownt", "threshold"],
        "flag_gemv_gemv_triton": ["x", "Wgate", "Wup", "Wdownt", "threshold"],
    }
    for name, params in want.items():
        assert list(inspect.signature(getattr(flash_gemv, name)).parameters) == params, name
    import sys
    assert "triton" not in sys.modules, "importing flash_gemv must not import triton"


def test_torch_ops_reject_cpu_tensors():
    """No silent CPU fallback: the ops refuse tensors that are not on the GPU."""
    import flash_gemv

    x = torch.zeros(1, 1, 64, dtype=torch.float16)
    w = torch.zeros(96, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU"):
        flash_gemv.cats_mlp(x, w, w, w, 0.1)
    with pytest.raises(RuntimeError, match="GPU"):
        flash_gemv.flag_gemv_gemv_inner(x, w, w, w.t().contiguous(), 0.1)
    out, flag = torch.zeros(1, 1, 96, dtype=torch.float16), torch.zeros(96, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="GPU"):
        flash_gemv.fuse_gemv_flag_local(x, w, out, flag, 0.1)


def test_argument_validation_of_the_newer_entry_points():
    """cats_mlp_norm_residual_norm and cats_probe_read reject bad arguments before any HIP call."""
    from cats_amd import capi

    L = capi.lib()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.c_void_p((ctypes.addressof(buf) + 255) // 256 * 256)
    odd = ctypes.c_void_p(p.value + 4)
    big = 1 << 30
    nrn = L.cats_mlp_norm_residual_norm
    assert nrn(p, p, 1e-5, p, p, p, p, None, 1e-5, p, 1, 64, 96, 0, 0.1, p, big, None) == 5      # next norm weight missing
    assert nrn(p, p, 1e-5, p, p, p, p, p, 1e-5, None, 1, 64, 96, 0, 0.1, p, big, None) == 5      # next output missing
    assert nrn(p, p, 1e-5, p, p, p, p, odd, 1e-5, p, 1, 64, 96, 0, 0.1, p, big, None) == 3       # misaligned weight
    assert nrn(p, p, 1e-5, p, p, p, p, p, 1e-5, p, 1, 72, 96, 0, 0.1, p, big, None) == 2         # H % 32 != 0
    assert nrn(p, p, 1e-5, p, p, p, p, p, 1e-5, p, 17, 64, 96, 0, 0.1, p, big, None) == 4        # batch
    probe = L.cats_probe_read
    probe.argtypes, probe.restype = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p], ctypes.c_int
    assert probe(None, 64, p, None) == 5
    assert probe(p, 0, p, None) == 3
    assert probe(p, 24, p, None) == 3
    assert probe(odd, 64, p, None) == 3
