"""Build recipe for the C-ABI library (hipcc, gfx950 only)."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libxfc_mi355x.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = [os.path.join(HERE, "csrc", "xfc_kernels.hip")]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-shared",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the global->LDS fetches list M0 as clobbered on purpose; hipcc notes that the register is reserved
    "-Wno-inline-asm",
]
# The kernels schedule their own waits around inline-asm fetches (csrc/pipe_core.hpp); they were validated
# on the GPU with this compiler.  Another version may schedule around the asm differently: rerun the GPU
# tests before trusting a build made with it.
VALIDATED_HIPCC = "7.2.26015"


def hipcc_version(hipcc: str) -> str:
    try:
        out = subprocess.run([hipcc, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True).stdout
    except OSError:
        return "unknown"
    for line in out.splitlines():
        if line.startswith("HIP version:"):
            return line.split(":", 1)[1].strip()
    return "unknown"


def build(verbose: bool = False) -> str:
    """Compile the library in-tree and return its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    ver = hipcc_version(hipcc)
    if not ver.startswith(VALIDATED_HIPCC):
        print(f"renee_amd.build: warning: hipcc {ver} is not the validated {VALIDATED_HIPCC}; "
              "run the GPU test suite before using this build", file=sys.stderr, flush=True)
    cmd = [hipcc, *HIPCC_FLAGS, *SOURCES, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
