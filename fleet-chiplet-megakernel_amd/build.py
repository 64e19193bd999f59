"""Build libfleet_mk.so (HIP kernel + C-ABI host library) for gfx950 with hipcc.

Usage: python build.py            (from anywhere; output lands next to this file: the library, then the Cython binding
                                   mirage/_cython/core.*.so that links against it)
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


def build_cython(verbose: bool = True) -> str:
    """Compile the Cython binding (mirage/_cython/core.pyx -> core.<abi>.so) against include/fleet_mk.h and link it to the
    library next to this file.  Needs the library to be built first."""
    import sysconfig
    cy_dir = os.path.join(HERE, "mirage", "_cython")
    c_file = os.path.join(cy_dir, "core.c")
    out = os.path.join(cy_dir, "core" + sysconfig.get_config_var("EXT_SUFFIX"))
    steps = [
        [sys.executable, "-m", "cython", "-3", "--module-name", "mirage._cython.core", "core.pyx", "-o", c_file],
        [shutil.which("gcc") or "gcc", "-O2", "-fPIC", "-shared", "-Wno-unused-function", "-I" + sysconfig.get_paths()["include"],
         "-I" + os.path.join(os.path.dirname(HERE), "include"), c_file, "-o", out, "-L" + HERE, "-lfleet_mk", "-Wl,-rpath,$ORIGIN/../.."],
    ]
    for cmd in steps:
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, cwd=cy_dir, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("building the Cython binding failed:\n" + res.stdout)
    return out


if __name__ == "__main__":
    build()
    print("built", LIB)
    print("built", build_cython())
    sys.exit(0)
