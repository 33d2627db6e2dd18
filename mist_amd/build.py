"""Compiles the HIP sources of this package into ``mist_amd/libmist_search.so`` for gfx950.

``hipcc`` cross-compiles without a GPU.  Flags that matter for correctness:
``-ffp-contract=off`` (no fused multiply-add: results must equal the numpy formulation operation
for operation) and no fast-math.
"""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, "libmist_search.so")
SOURCES = [os.path.join(PKG_DIR, "csrc", name) for name in ("mist_search.hip", "mist_dp.hip", "mist_mip.hip", "mist_inter.hip", "mist_plan.hip")]
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build_library(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    sources = [s for s in SOURCES if os.path.exists(s)]
    extra = os.environ.get("MIST_HIPCC_EXTRA", "").split()
    cmd = [hipcc, *HIPCC_FLAGS, *extra, "-I" + os.path.join(REPO_DIR, "include"), *sources, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
