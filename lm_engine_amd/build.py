"""Builds lm_engine_amd/libgdn_hip.so from the HIP sources in lm_engine_amd/csrc with hipcc.

The library is a plain C-ABI shared object (see include/gdn_hip.h): it links only the HIP
runtime, so it is independent of the ROCm version PyTorch was built against.  hipcc
cross-compiles for gfx950 without a GPU present.

    python -m lm_engine_amd.build
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor


PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PACKAGE_DIR, "csrc")
INCLUDE_DIR = os.path.join(os.path.dirname(PACKAGE_DIR), "include")
LIBRARY_PATH = os.path.join(PACKAGE_DIR, "libgdn_hip.so")

SOURCES = ("gdn_api.hip", "gdn_recurrent.hip", "gdn_chunk.hip", "gdn_chunk32.hip", "gdn_chunk_fused.hip", "gdn_chunk_bwd.hip", "gdn_conv1d.hip", "gdn_conv1d_bwd.hip", "gdn_elementwise.hip")

HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the scan kernels are one fully unrolled schedule per chunk; the default size limit for "#pragma unroll"
    # would leave their register arrays dynamically indexed, i.e. in scratch memory
    "-mllvm", "-pragma-unroll-threshold=200000",
)  # fmt: skip


def _hipcc() -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found; the gated delta-rule library needs ROCm to build")
    return hipcc


CYCLE_BUDGET_LIBRARY_PATH = os.path.join(PACKAGE_DIR, "libgdn_hip_cycles.so")
CYCLE_BUDGET_SOURCES = ("gdn_api.hip", "gdn_chunk.hip", "gdn_chunk32.hip", "gdn_chunk_bwd.hip")  # the sources that read GDN_CYCLE_BUDGET


def build_library(verbose: bool = False, extra_flags: tuple[str, ...] = (), cycle_budget: bool = False) -> str:
    """Compiles every source and links the shared library; always rebuilds.

    ``cycle_budget``: the measurement build instead, ``libgdn_hip_cycles.so`` - the same library with the shader clock
    read between the groups of MFMAs of the half-slice scan's chunk loop and between the steps of the chunk-local backward
    kernel (``-DGDN_CYCLE_BUDGET``; only the sources that
    read the macro are compiled again, the rest is linked from the objects of the library proper, which must exist).
    ``bench.py --cycle-budget`` loads it; nothing else does."""
    hipcc = _hipcc()
    build_dir = os.path.join(CSRC_DIR, "build")
    os.makedirs(build_dir, exist_ok=True)
    sources, library_path, object_dir = SOURCES, LIBRARY_PATH, build_dir
    if cycle_budget:
        sources, library_path, object_dir = CYCLE_BUDGET_SOURCES, CYCLE_BUDGET_LIBRARY_PATH, os.path.join(build_dir, "cycles")
        os.makedirs(object_dir, exist_ok=True)
        extra_flags = (*extra_flags, "-DGDN_CYCLE_BUDGET")

    def compile_one(src: str) -> str:
        obj = os.path.join(object_dir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}", "-c",
               os.path.join(CSRC_DIR, src), "-o", obj]  # fmt: skip
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
        if verbose and proc.stderr.strip():
            print(proc.stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=len(sources)) as pool:
        objects = list(pool.map(compile_one, sources))
    if cycle_budget:
        objects += [os.path.join(build_dir, src.replace(".hip", ".o")) for src in SOURCES if src not in CYCLE_BUDGET_SOURCES]

    tmp = library_path + ".tmp"
    proc = subprocess.run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", *objects, "-o", tmp],
                          capture_output=True, text=True)  # fmt: skip
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, library_path)
    return library_path


if __name__ == "__main__":
    print(build_library(verbose=True, cycle_budget="--cycle-budget" in sys.argv[1:]))
