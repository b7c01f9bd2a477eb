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
# source -> extra flags of that translation unit
SOURCES = {
    os.path.join(PKG_DIR, "csrc", "bitlinear_hip.hip"): [],
    os.path.join(PKG_DIR, "csrc", "decoder_ops.hip"): [],
    # keep the attention kernel's accumulators in the vector register file (see the file's header)
    os.path.join(PKG_DIR, "csrc", "attn_prefill.hip"): ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}
OBJ_DIR = os.path.join(PKG_DIR, "lib", "obj")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbitlinear_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-ffp-contract=off",
    # packed fp32 VALU forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the leading kernel arguments arrive in registers at wave start instead of through scalar loads
    # (a memory round trip in front of every kernel's first useful instruction otherwise)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP library cannot be built")


def _finish(cmd, res, verbose):
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed: " + " ".join(cmd) + "\n" + res.stdout + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build_library(verbose: bool = True) -> str:
    """One object per source (compiled side by side), then one link."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = hipcc_path()
    jobs = []
    for src, extra in SOURCES.items():
        obj = os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(src))[0] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *extra, "-I", os.path.join(REPO_ROOT, "include"), "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        jobs.append((cmd, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
    objs = []
    for cmd, obj, proc in jobs:
        out, err = proc.communicate()
        _finish(cmd, subprocess.CompletedProcess(cmd, proc.returncode, out, err), verbose)
        objs.append(obj)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    _finish(cmd, subprocess.run(cmd, capture_output=True, text=True), verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
