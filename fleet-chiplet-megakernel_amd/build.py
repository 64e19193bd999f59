"""Build libfleet_mk.so (HIP kernel + C-ABI host library) for gfx950 with hipcc.

Usage: python build.py            (from anywhere; output lands next to this file)
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libfleet_mk.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU forms are disabled for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build(verbose: bool = True, defines=(), out: str = None) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: the megakernel library cannot be built")
    lib = out or LIB
    cmd = [hipcc] + HIPCC_FLAGS + ["-D" + d for d in defines] + [os.path.join(CSRC, "fleet_mk.hip"), "-o", lib]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=CSRC, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return lib


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
