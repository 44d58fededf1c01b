"""Builds ``libsteptron_moe_gfx950.so`` from ``csrc/*.hip`` with hipcc (gfx950 only).

The library is built in-tree (``steptronoss_amd/lib/``) so that it travels with the
source tree; hipcc cross-compiles without a GPU.  Run ``python -m steptronoss_amd.build``.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_NAME = "libsteptron_moe_gfx950.so"
LIB_PATH = LIB_DIR / LIB_NAME

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(args):
    hipcc, src, obj = args
    cmd = [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    return src, proc.returncode, proc.stdout + proc.stderr


def build_library(verbose: bool = True, jobs: int = 8) -> Path:
    """Compile every ``csrc/*.hip`` and link the shared library; always recompiles."""
    hipcc = _hipcc()
    LIB_DIR.mkdir(exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    work = [(hipcc, src, obj_dir / (src.stem + ".o")) for src in sources()]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile, work))
    failed = False
    for src, code, out in results:
        harmless = "packed-fp32-ops' is not a recognized feature"
        shown = "\n".join(l for l in out.splitlines() if harmless not in l).strip()
        if verbose and shown:
            print(f"[hipcc {src.name}]\n{shown}", file=sys.stderr)
        if code != 0:
            failed = True
    if failed:
        raise RuntimeError("hipcc failed, see messages above")
    tmp = LIB_DIR / (LIB_NAME + ".tmp")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *[str(w[2]) for w in work]]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout + proc.stderr)
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({LIB_PATH.stat().st_size // 1024} KiB) from {len(work)} sources")
    return LIB_PATH


def build_host_check(verbose: bool = True) -> Path:
    """Compile ``tests/capi_host/host_check.cpp`` (a torch-free host of the C ABI, used by the GPU
    tests) into a small shared library next to its source, linked against the main library."""
    src = PKG.parent / "tests" / "capi_host" / "host_check.cpp"
    out = src.with_name("libstm_host_check.so")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [  # host code only: the plain C++ compiler, the HIP runtime API headers and library
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", f"-I{rocm}/include", str(src),
        "-o", str(out), f"-L{LIB_DIR}", "-lsteptron_moe_gfx950", "-Wl,-rpath,$ORIGIN/../../steptronoss_amd/lib",
        f"-L{rocm}/lib", "-lamdhip64", f"-Wl,-rpath,{rocm}/lib",
    ]  # fmt: skip
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("host check build failed:\n" + proc.stdout + proc.stderr)
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build_library()
    build_host_check()
