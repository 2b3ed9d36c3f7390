"""Builds libkitty_hip.so (the C-ABI library holding every HIP kernel) in-tree with hipcc for gfx950.

    python -m kitty_amd.build
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libkitty_hip.so")
ARCH = "gfx950"


def sources():
    return sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [
        hipcc, f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
        # packed-fp32 VALU forms are kept out of the generated code on purpose
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wno-unused-command-line-argument",
        "-o", LIB,
    ] + sources()
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
