"""Builds libint4linear.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Run as ``python -m int4linear_amd.build``.  hipcc cross-compiles for gfx950 without a
GPU, so this works on a CPU-only machine.  The library lands in
``int4linear_amd/lib/libint4linear.so``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = PKG_DIR / "csrc" / "build"
LIB_PATH = LIB_DIR / "libint4linear.so"

HIP_SOURCES = ["api.hip", "kernels_simple.hip", "kernels_mfma.hip", "kernels_fp6.hip", "kernels_skinny.hip"]
CXX_SOURCES = ["packer_host.cpp"]

# Packed-FP32 VALU forms are switched off for every device compile of this project.
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# Per-file additions.  The decode kernels are a few microseconds long, and a wave's scalar loads
# of its kernel arguments are a memory round trip in front of its first instruction that does
# anything: there the first 14 dwords of the arguments arrive preloaded in scalar registers.
# (The compiler keeps a prologue that loads them the ordinary way, which firmware without the
# feature runs instead.)  The option is internal to LLVM: build_library() tries it on an empty
# kernel first and drops it if this hipcc does not take it (the kernels then load their
# arguments the ordinary way, a few tenths of a microsecond per launch).
EXTRA_HIP_FLAGS = {
    "kernels_skinny.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"],
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build int4linear_amd")
    return exe


def _accepted_flags(hipcc: str, flags: list[str]) -> list[str]:
    """`flags` if this hipcc compiles an empty device function with them, else none of them:
    options passed to LLVM with -mllvm are internal and may be gone in another release, and a
    missing one must cost its tuning, not the build."""
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        src = Path(tmp) / "probe.hip"
        src.write_text("__global__ void probe(int *p) { *p = 0; }\n")
        cmd = [hipcc, "--offload-arch=gfx950", "--cuda-device-only", *flags, "-c", str(src), "-o", str(Path(tmp) / "probe.o")]
        ok = subprocess.run(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL).returncode == 0
    if not ok:
        sys.stderr.write("int4linear_amd.build: hipcc rejects " + " ".join(flags) + "; building without\n")
    return flags if ok else []


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless.
    noise = ("is not a recognized feature", "warning generated", "warnings generated")
    out = "\n".join(l for l in proc.stdout.splitlines() if l and not any(n in l for n in noise))
    if out.strip():
        sys.stderr.write(out + "\n")


def _check_no_missing_kernels() -> None:
    """A kernel whose device or host half failed to be emitted shows up as an undefined
    symbol of this project's namespace; refuse such a library."""
    nm = shutil.which("nm")
    if not nm:
        return
    out = subprocess.run([nm, "-D", "--undefined-only", str(LIB_PATH)], stdout=subprocess.PIPE,
                         text=True).stdout
    missing = [l.split()[-1] for l in out.splitlines() if "int4linear" in l]
    if missing:
        raise RuntimeError("libint4linear.so has undefined project symbols: " + ", ".join(missing))


def build_library(verbose: bool = False, save_temps: bool = False) -> Path:
    """Compile every source and link the shared library.  Always recompiles."""
    hipcc = _hipcc()
    LIB_DIR.mkdir(exist_ok=True)
    OBJ_DIR.mkdir(exist_ok=True)
    jobs = []
    for src in HIP_SOURCES:
        obj = OBJ_DIR / (src + ".o")
        extra = _accepted_flags(hipcc, EXTRA_HIP_FLAGS[src]) if src in EXTRA_HIP_FLAGS else []
        cmd = [hipcc, *HIP_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
        if save_temps:
            cmd.insert(1, "-save-temps=obj")
        jobs.append((cmd, obj))
    for src in CXX_SOURCES:
        obj = OBJ_DIR / (src + ".o")
        jobs.append(([hipcc, "-O3", "-std=c++20", "-fPIC", "-c", str(CSRC / src), "-o", str(obj)], obj))
    if verbose:
        for cmd, _ in jobs:
            print(" ".join(cmd))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        list(pool.map(lambda j: _run(j[0]), jobs))
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH)]
    link += [str(obj) for _, obj in jobs]
    if verbose:
        print(" ".join(link))
    _run(link)
    _check_no_missing_kernels()
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose="-v" in sys.argv, save_temps="--save-temps" in sys.argv)
    print(path)
