"""Compiles the HIP sources under csrc/ into warpconvnet_amd/libwcn_hip.so for gfx950."""
import glob
import os
import shutil
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libwcn_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 instructions are kept out of every code object of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build_library(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    sources = sorted(glob.glob(os.path.join(_PKG, "csrc", "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources found under csrc/")
    cmd = [hipcc, *HIPCC_FLAGS, "-o", LIB_PATH, *sources]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
