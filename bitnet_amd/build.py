"""Builds libbitlinear_hip.so for gfx950 with hipcc, in-tree.

    python -m bitnet_amd.build

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain
is installed.  The counterpart of the reference's one-line nvcc recipe
(gpu/bitnet_kernels/compile.sh:1).
"""
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
SOURCES = [os.path.join(PKG_DIR, "csrc", "bitlinear_hip.hip"), os.path.join(PKG_DIR, "csrc", "decoder_ops.hip")]
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbitlinear_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-ffp-contract=off",
    # packed fp32 VALU forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP library cannot be built")


def build_library(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-I", os.path.join(REPO_ROOT, "include"), *SOURCES, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
