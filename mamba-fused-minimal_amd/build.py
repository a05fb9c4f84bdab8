"""Builds libssd_gfx950.so (the C-ABI library with the gfx950 HIP kernels) in-tree with hipcc.

Usage:  python build.py            (from anywhere)
hipcc cross-compiles for gfx950 without a GPU, so this runs on a CPU-only machine."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libssd_gfx950.so")
SOURCES = ["ssd_capi.hip", "ssd_mfma.hip", "ssd_quad.hip", "ssd_step_split.hip", "ssd_generic.hip", "ssd_state_passing.hip", "ssd_chunk_cumsum.hip", "ssd_chunk_scan_states.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build_library(verbose=False, extra_flags=()):
    cmd = [hipcc(), *FLAGS, *extra_flags, *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True, extra_flags=sys.argv[1:]))
