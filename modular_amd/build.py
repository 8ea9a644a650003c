"""Builds libmaxfp8.so (hand-written gfx950 HIP kernels + the C ABI) with hipcc.

    python -m modular_amd.build

hipcc cross-compiles for gfx950 without a GPU.  The library is written in-tree
(modular_amd/lib/libmaxfp8.so) so it travels with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libmaxfp8.so")

SOURCES = ["api.hip", "quant.hip", "naive.hip", "gemm_tiled.hip", "gemm_w4.hip", "gemm_skinny.hip", "moe.hip"]

# packed-fp32 VALU ops are switched off for every kernel (they are not used by hand either)
COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]
# the naive kernels must round every product and sum like a scalar host loop
# the four-wave kernels keep their MFMA results in ordinary VGPRs (the promotions are VALU work) and their operand
# fragments in AGPRs: left to itself the compiler writes every MFMA result to AGPRs once a kernel uses any
PER_FILE = {"naive.hip": ["-ffp-contract=off"], "gemm_w4.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src: str, objdir: str, extra: list[str]) -> str:
    obj = os.path.join(objdir, src.replace(".hip", ".o"))
    cmd = [hipcc(), *COMMON, *PER_FILE.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
    return obj


def build_library(extra: list[str] | None = None, verbose: bool = True) -> str:
    """Compile every HIP source for gfx950 and link the shared library."""
    extra = list(extra or [])
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(lambda s: _compile(s, objdir, extra), SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB + ".tmp", *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    os.replace(LIB + ".tmp", LIB)
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB) // 1024} KiB)")
    return LIB


if __name__ == "__main__":
    build_library(sys.argv[1:])
