"""ctypes binding of the C ABI in ``include/cats_gemv.h`` (``cats_amd/lib/libcats_gemv.so``).

This is the same boundary the torch op library binds; it exists so tests, the benchmark and non-torch callers
can drive the kernels with raw device pointers.  Tensors are only used here as owners of device memory
(``data_ptr()``) and of the current stream -- no torch arithmetic happens on this path, and a missing library
raises ``ImportError`` (there is no fallback).
"""
from __future__ import annotations

import ctypes
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent / "lib" / "libcats_gemv.so"
_lib = None

F16, BF16, F32 = 0, 1, 2
DTYPE_CODE = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}

# every symbol include/cats_gemv.h declares
SYMBOLS = (
    "cats_version", "cats_status_string", "cats_workspace_bytes", "cats_workspace_init", "cats_gate_flag",
    "cats_gate_compact", "cats_read_count", "cats_up_flag", "cats_down_flag", "cats_gate_up", "cats_mlp",
    "cats_mlp_rowmajor_down", "cats_mlp_norm_residual", "cats_up_down", "cats_set_tuning", "cats_mlp_stage", "cats_mlp_noalloc", "cats_up_index", "cats_down_index",
    "cats_probe_read", "cats_mlp_norm_residual_norm",
)


class CatsError(RuntimeError):
    pass


def use_library(path) -> None:
    """Bind another build of the kernel library (the stamped one, say).  Only before the first call into it."""
    global _LIB_PATH
    if _lib is not None:
        raise RuntimeError("the kernel library is already loaded")
    _LIB_PATH = Path(path)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise ImportError(f"{_LIB_PATH} is missing: build it with `python -m cats_amd.build`")
        L = ctypes.CDLL(str(_LIB_PATH))
        vp, i32, f32, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
        L.cats_version.argtypes = []; L.cats_version.restype = i32
        L.cats_status_string.argtypes = [i32]; L.cats_status_string.restype = ctypes.c_char_p
        L.cats_workspace_bytes.argtypes = [i32, i32, i32]; L.cats_workspace_bytes.restype = sz
        L.cats_workspace_init.argtypes = [vp, sz, vp]; L.cats_workspace_init.restype = i32
        L.cats_gate_flag.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, f32, vp]; L.cats_gate_flag.restype = i32
        L.cats_gate_compact.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, f32, vp, sz, vp]; L.cats_gate_compact.restype = i32
        L.cats_read_count.argtypes = [vp, vp]; L.cats_read_count.restype = i32
        L.cats_up_flag.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]; L.cats_up_flag.restype = i32
        L.cats_down_flag.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, sz, vp]; L.cats_down_flag.restype = i32
        L.cats_gate_up.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp]; L.cats_gate_up.restype = i32
        L.cats_mlp.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, sz, vp]; L.cats_mlp.restype = i32
        L.cats_mlp_rowmajor_down.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, sz, vp]; L.cats_mlp_rowmajor_down.restype = i32
        L.cats_mlp_norm_residual.argtypes = [vp, vp, f32, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, sz, vp]
        L.cats_mlp_norm_residual.restype = i32
        if hasattr(L, "cats_mlp_norm_residual_norm"):  # absent from older builds of the library bound with use_library()
            L.cats_mlp_norm_residual_norm.argtypes = [vp, vp, f32, vp, vp, vp, vp, vp, f32, vp, i32, i32, i32, i32, f32, vp, sz, vp]
            L.cats_mlp_norm_residual_norm.restype = i32
        L.cats_up_down.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, sz, vp]; L.cats_up_down.restype = i32
        L.cats_mlp_stage.argtypes = [i32, vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, sz, vp]; L.cats_mlp_stage.restype = i32
        L.cats_mlp_noalloc.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp]; L.cats_mlp_noalloc.restype = i32
        L.cats_up_index.argtypes = [vp, vp, vp, i32, vp, vp, i32, vp, i32, i32, i32, i32, vp]; L.cats_up_index.restype = i32
        L.cats_down_index.argtypes = [vp, vp, vp, i32, vp, vp, i32, i32, i32, i32, vp, sz, vp]; L.cats_down_index.restype = i32
        L.cats_set_tuning.argtypes = [i32, i32, i32, i32]; L.cats_set_tuning.restype = i32
        _lib = L
    return _lib


def status_string(code: int) -> str:
    return lib().cats_status_string(code).decode()


def check(code: int, what: str) -> None:
    if code != 0:
        raise CatsError(f"{what}: {status_string(code)} (status {code})")


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _dims(x: torch.Tensor, w: torch.Tensor):
    H = x.shape[-1]
    return x.numel() // H, H, w.shape[0]


class Workspace:
    """Device scratch for the workspace-taking entry points; zero-filled once by the library."""

    def __init__(self, B: int, H: int, I: int, device="cuda"):
        self.nbytes = lib().cats_workspace_bytes(B, H, I)
        self.buf = torch.empty(self.nbytes, dtype=torch.uint8, device=device)
        check(lib().cats_workspace_init(_p(self.buf), self.nbytes, _stream(self.buf)), "cats_workspace_init")


def gate_flag(x, wgate, threshold, want_a=True, want_flag=True):
    B, H, I = _dims(x, wgate)
    a = torch.empty(B, I, dtype=x.dtype, device=x.device) if want_a else None
    flag = torch.empty(B, I, dtype=torch.bool, device=x.device) if want_flag else None
    check(lib().cats_gate_flag(_p(x), _p(wgate), _p(a), _p(flag), B, H, I, DTYPE_CODE[x.dtype], float(threshold), _stream(x)),
          "cats_gate_flag")
    return a, flag


def gate_compact(x, wgate, threshold, ws: Workspace):
    """Returns (vals (I,), idx (I,) int64, n) -- only the first n entries are meaningful."""
    B, H, I = _dims(x, wgate)
    vals = torch.zeros(I, dtype=x.dtype, device=x.device)
    idx = torch.full((I,), -1, dtype=torch.int64, device=x.device)
    count = torch.zeros(1, dtype=torch.int32, device=x.device)
    check(lib().cats_gate_compact(_p(x), _p(wgate), _p(vals), _p(idx), _p(count), H, I, DTYPE_CODE[x.dtype], float(threshold),
                                  _p(ws.buf), ws.nbytes, _stream(x)), "cats_gate_compact")
    n = lib().cats_read_count(_p(count), _stream(x))
    return vals, idx, n


def up_flag(x, wup, a, flag, out_f32=False):
    B, H, I = _dims(x, wup)
    out = torch.empty(B, I, dtype=torch.float32 if out_f32 else x.dtype, device=x.device)
    check(lib().cats_up_flag(_p(x), _p(wup), _p(a), _p(flag), _p(out), int(out_f32), B, H, I, DTYPE_CODE[x.dtype], _stream(x)),
          "cats_up_flag")
    return out


def down_flag(z, wdown_t, flag, ws: Workspace, accumulate_into=None):
    """accumulate_into: optional fp32 (B, H) tensor (atomic_gemv mode); otherwise returns (B, H) in dtype."""
    I, H = wdown_t.shape
    B = z.numel() // I
    if accumulate_into is not None:
        check(lib().cats_down_flag(_p(z), _p(wdown_t), _p(flag), _p(accumulate_into), None, B, H, I, DTYPE_CODE[z.dtype],
                                   _p(ws.buf), ws.nbytes, _stream(z)), "cats_down_flag")
        return accumulate_into
    y = torch.empty(B, H, dtype=z.dtype, device=z.device)
    check(lib().cats_down_flag(_p(z), _p(wdown_t), _p(flag), None, _p(y), B, H, I, DTYPE_CODE[z.dtype], _p(ws.buf), ws.nbytes,
                               _stream(z)), "cats_down_flag")
    return y


def gate_up(x, wgate, wup, threshold):
    B, H, I = _dims(x, wgate)
    out = torch.empty(B, I, dtype=x.dtype, device=x.device)
    flag = torch.empty(B, I, dtype=torch.bool, device=x.device)
    check(lib().cats_gate_up(_p(x), _p(wgate), _p(wup), _p(out), _p(flag), B, H, I, DTYPE_CODE[x.dtype], float(threshold), _stream(x)),
          "cats_gate_up")
    return out, flag


def mlp(x, wgate, wup, wdown_t, threshold, ws: Workspace, y=None, want_flag=False, want_count=False, y_f32=None):
    """Whole MLP (two launches).  Returns y, or (y, flag, count) tensors when asked for."""
    B, H, I = _dims(x, wgate)
    if y is None and y_f32 is None:
        y = torch.empty(B, H, dtype=x.dtype, device=x.device)
    flag = torch.empty(B, I, dtype=torch.bool, device=x.device) if want_flag else None
    count = torch.zeros(1, dtype=torch.int32, device=x.device) if want_count else None
    check(lib().cats_mlp(_p(x), _p(wgate), _p(wup), _p(wdown_t), _p(y) if y_f32 is None else None, _p(y_f32), _p(flag), _p(count),
                         B, H, I, DTYPE_CODE[x.dtype], float(threshold), _p(ws.buf), ws.nbytes, _stream(x)), "cats_mlp")
    out = y if y_f32 is None else y_f32
    if want_flag or want_count:
        return out, flag, count
    return out


ACTIVATIONS = {"id": 0, "relu": 1, "squared_relu": 2, "swish": 3}


def up_index(x, w, idx, bias=None, scale=None, activation="id"):
    """out[b, m] = scale[m] * act(x[b] . w[idx[m]] + bias[idx[m]]); idx int64 (M,).  Returns (B, M) in x.dtype."""
    B, H, Z = _dims(x, w)
    M = int(idx.numel())
    out = torch.empty(B, M, dtype=x.dtype, device=x.device)
    check(lib().cats_up_index(_p(x), _p(w), _p(idx), M, _p(bias), _p(scale), ACTIVATIONS[activation], _p(out), B, H, Z,
                              DTYPE_CODE[x.dtype], _stream(x)), "cats_up_index")
    return out


def down_index(z, wdown_t, idx, ws: Workspace, bias=None):
    """y[b] = sum_m z[b, m] * wdown_t[idx[m]] (+ bias); z (B, M) aligned with idx.  Returns (B, H) in z.dtype."""
    Z, H = wdown_t.shape
    M = int(idx.numel())
    B = z.shape[0]
    y = torch.empty(B, H, dtype=z.dtype, device=z.device)
    check(lib().cats_down_index(_p(z), _p(wdown_t), _p(idx), M, _p(bias), _p(y), B, H, Z, DTYPE_CODE[z.dtype], _p(ws.buf), ws.nbytes,
                                _stream(z)), "cats_down_index")
    return y


def mlp_noalloc(x, wgate, wup, wdown_t, threshold, y):
    """cats_mlp into the caller's y with the library's built-in scratch: no workspace, nothing allocated by the call."""
    B, H, I = _dims(x, wgate)
    check(lib().cats_mlp_noalloc(_p(x), _p(wgate), _p(wup), _p(wdown_t), _p(y), B, H, I, DTYPE_CODE[x.dtype], float(threshold),
                                 _stream(x)), "cats_mlp_noalloc")
    return y


def up_down(x, a, wup, wdown_t, threshold, ws: Workspace):
    """Sparse up + down given the gate activations a (B, I): flags = |a| > threshold are derived on the device."""
    B, H, I = _dims(x, wup)
    y = torch.empty(B, H, dtype=x.dtype, device=x.device)
    check(lib().cats_up_down(_p(x), _p(a), _p(wup), _p(wdown_t), _p(y), B, H, I, DTYPE_CODE[x.dtype], float(threshold), _p(ws.buf),
                             ws.nbytes, _stream(x)), "cats_up_down")
    return y


def mlp_norm_residual(h, norm_weight, eps, wgate, wup, wdown_t, threshold, ws: Workspace, out=None):
    """out = h + MLP(norm_weight * rms_norm(h)); pass out=h to update the hidden state in place."""
    B, H, I = _dims(h, wgate)
    if out is None:
        out = torch.empty(B, H, dtype=h.dtype, device=h.device)
    check(lib().cats_mlp_norm_residual(_p(h), _p(norm_weight), float(eps), _p(wgate), _p(wup), _p(wdown_t), _p(out), B, H, I,
                                       DTYPE_CODE[h.dtype], float(threshold), _p(ws.buf), ws.nbytes, _stream(h)),
          "cats_mlp_norm_residual")
    return out


def mlp_norm_residual_norm(h, norm_weight, eps, wgate, wup, wdown_t, threshold, next_norm_weight, next_eps, ws: Workspace, out=None):
    """(out, next_out): out = h + MLP(norm_weight * rms_norm(h)), next_out = next_norm_weight * rms_norm(out)."""
    B, H, I = _dims(h, wgate)
    if out is None:
        out = torch.empty(B, H, dtype=h.dtype, device=h.device)
    nxt = torch.empty(B, H, dtype=h.dtype, device=h.device)
    check(lib().cats_mlp_norm_residual_norm(_p(h), _p(norm_weight), float(eps), _p(wgate), _p(wup), _p(wdown_t), _p(out),
                                            _p(next_norm_weight), float(next_eps), _p(nxt), B, H, I, DTYPE_CODE[h.dtype],
                                            float(threshold), _p(ws.buf), ws.nbytes, _stream(h)), "cats_mlp_norm_residual_norm")
    return out, nxt


def mlp_rowmajor_down(x, wgate, wup, wdown, threshold, ws: Workspace):
    B, H, I = _dims(x, wgate)
    y = torch.empty(B, H, dtype=x.dtype, device=x.device)
    check(lib().cats_mlp_rowmajor_down(_p(x), _p(wgate), _p(wup), _p(wdown), _p(y), B, H, I, DTYPE_CODE[x.dtype], float(threshold),
                                       _p(ws.buf), ws.nbytes, _stream(x)), "cats_mlp_rowmajor_down")
    return y


def probe_read(src: torch.Tensor, sink: torch.Tensor):
    """One read-only streaming pass over src (any dtype, contiguous); sink: 4 bytes of device memory, normally untouched."""
    fn = lib().cats_probe_read
    fn.argtypes, fn.restype = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p], ctypes.c_int
    check(fn(_p(src), src.numel() * src.element_size(), _p(sink), _stream(src)), "cats_probe_read")


def set_tuning(gate_variant=0, down_groups=0, down_block=0, path=0):
    """path=1 keeps the whole-MLP entry points on the separate gate+up and sparse-down kernels at every batch size."""
    lib().cats_set_tuning(int(gate_variant), int(down_groups), int(down_block), int(path))
