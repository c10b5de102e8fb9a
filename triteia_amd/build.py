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


# The wide kernels wait for their direct-to-LDS loads with hand-counted `s_waitcnt vmcnt(N)`: N counts
# the loads the compiler emits behind them in program order.  The counts were checked against the assembly
# output of this compiler; another one may order or split the loads differently, so the build refuses it
# unless TRITEIA_HIP_ANY_COMPILER=1 says that the counts have been checked again (`-S`, then the GPU parity tests).
VERIFIED_COMPILER = "roc-7.2.0"


def check_compiler(hipcc: str) -> str:
    out = subprocess.run([hipcc, "--version"], capture_output=True, text=True).stdout
    if VERIFIED_COMPILER not in out and os.environ.get("TRITEIA_HIP_ANY_COMPILER") != "1":
        raise RuntimeError(
            f"{hipcc} is not the compiler the hand-counted waits were verified with ({VERIFIED_COMPILER}):\n{out}"
            "set TRITEIA_HIP_ANY_COMPILER=1 after checking them again")
    return out


def build(verbose: bool = True, extra_flags=()) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    check_compiler(hipcc)
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


def ensure_built(verbose: bool = True) -> str:
    """The built library's path; compiles it first if (and only if) there is none in the tree.  For tests,
    smoke runs and benchmarks, which load what is built; `build()` itself compiles every time."""
    if not os.path.exists(LIB):
        build(verbose=verbose)
    return LIB


if __name__ == "__main__":
    print(build(extra_flags=sys.argv[1:]))
