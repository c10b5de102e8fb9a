"""Build recipe for libtriteia_hip.so (gfx950) -- run as `python -m triteia_amd.build`.

hipcc cross-compiles without a GPU, so this works in a CPU-only container.  The
library is built in-tree at triteia_amd/lib/libtriteia_hip.so.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "triteia_hip.hip")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libtriteia_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build(verbose: bool = True, extra_flags=()) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-o", LIB, SRC]
    if verbose:
        print("[triteia_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the gfx950-only feature flag and says so; drop that line
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    print(build(extra_flags=sys.argv[1:]))
