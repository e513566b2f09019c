"""Build the gfx950 kernels and the torch op library in-tree.

Three shared objects come out of this:

* ``cats_amd/lib/libcats_gemv.so`` -- the HIP kernels behind the C ABI of ``include/cats_gemv.h``.
  No torch in it: plain pointers, sizes and a stream.
* ``flash_gemv/_C.so`` -- a thin ``TORCH_LIBRARY(flash_gemv, m)`` shim that unpacks tensors, picks the
  current HIP stream, owns a cached workspace and calls the C ABI.  It takes the place of the reference's
  ``flash_gemv/_C*.so`` (built there by ``flash_gemv/setup.py:51-97`` with nvcc).

* ``cats_amd/lib/libcats_gemv_timing.so`` -- the kernel library compiled with ``-DCATS_TIMING``: every workgroup
  stamps the wall clock at its phase boundaries into a caller-supplied buffer.  Only ``cats_amd.phase_stamps``
  loads it.

Run ``python -m cats_amd.build`` (hipcc cross-compiles for gfx950 without a GPU); ``--timing`` also builds the
stamped twin.  ``CATS_HIP_DEFINES`` in the environment adds compiler definitions to the kernel builds.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "cats_amd" / "csrc"
OBJ = ROOT / "build" / "obj"
LIB_DIR = ROOT / "cats_amd" / "lib"
KERNEL_LIB = LIB_DIR / "libcats_gemv.so"
TIMING_LIB = LIB_DIR / "libcats_gemv_timing.so"   # same kernels with per-workgroup wall-clock stamps (-DCATS_TIMING)
TORCH_LIB = ROOT / "flash_gemv" / "_C.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
HIP_FLAGS = [
    "-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(map(str, cmd))}\n{proc.stdout}\n{err}")
    if err.strip():
        print(err, file=sys.stderr)


def build_kernels(jobs: int = 4, timing: bool = False) -> Path:
    """The kernel library; with ``timing`` the instrumented twin that ``cats_amd.phase_stamps`` loads (never the product)."""
    obj = OBJ / "timing" if timing else OBJ
    out = TIMING_LIB if timing else KERNEL_LIB
    extra = ["-DCATS_TIMING"] if timing else []
    extra += os.environ.get("CATS_HIP_DEFINES", "").split()  # experiment switches, e.g. -DCATS_FUSED_POOL=1
    obj.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    units = [
        (CSRC / "cats_inst.hip", obj / "cats_inst_f16.o", ["-DCATS_DT=F16"]),
        (CSRC / "cats_inst.hip", obj / "cats_inst_bf16.o", ["-DCATS_DT=BF16"]),
        (CSRC / "cats_inst.hip", obj / "cats_inst_f32.o", ["-DCATS_DT=F32"]),
        (CSRC / "cats_api.hip", obj / "cats_api.o", []),
    ]
    cmds = [[HIPCC, *HIP_FLAGS, *extra, *defs, "-c", str(src), "-o", str(o)] for src, o, defs in units]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, cmds))
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(out), *[str(u[1]) for u in units]])
    return out


def build_torch_shim() -> Path:
    import torch
    from torch.utils import cpp_extension

    torch_lib = Path(torch.__file__).parent / "lib"
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    cmd = [
        HIPCC, "-O2", "-fPIC", "-std=c++17", "-shared", "-x", "c++",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DHIPBLAS_V2",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch.compiled_with_cxx11_abi())}",
        f"-I{ROOT / 'include'}", "-I/opt/rocm/include", *inc,
        str(CSRC / "cats_torch.cpp"), "-o", str(TORCH_LIB),
        f"-L{LIB_DIR}", "-lcats_gemv", f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
        "-L/opt/rocm/lib", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN/../cats_amd/lib", f"-Wl,-rpath,{torch_lib}",
    ]
    _run(cmd)
    return TORCH_LIB


def build_all(timing: bool = False) -> None:
    """The product: kernel library and torch op library.  ``timing`` adds the stamped twin (a measuring tool)."""
    print(f"[cats_amd.build] kernels  -> {build_kernels()}")
    print(f"[cats_amd.build] torch op -> {build_torch_shim()}")
    if timing:
        print(f"[cats_amd.build] stamped  -> {build_kernels(timing=True)}")


if __name__ == "__main__":
    build_all(timing="--timing" in sys.argv[1:])
