"""In-tree build of the HIP library: ``python -m fbgemm_amd.build``.

One hipcc invocation, gfx950 only. hipcc cross-compiles without a GPU, so this
also runs on a CPU-only machine.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "lib", "libfbgemm_amd.so")

SOURCES = ["lookup_kernels.hip", "c_api.cpp"]

# -ffp-contract=off: the kernels spell out every fma; nothing else may be fused,
#   or the fp32 rounding sequence would differ from the reference's.
# -packed-fp32-ops off: keep the compiler from forming packed fp32 instructions.
FLAGS = [
    "-x", "hip", "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # error reporting uses a few atomics on one address; keep them as plain
    # atomics instead of a wave-wide reduction loop in front of each
    "-mllvm", "-amdgpu-atomic-optimizer-strategy=None",
]


def build_library(verbose=False):
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    cmd = ["hipcc", *FLAGS, "-o", OUT, *[os.path.join(CSRC, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only target feature; that warning is noise
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{out}")
    if verbose and out.strip():
        print(out)
    return OUT


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
