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

# the lookup kernels compile one instance per translation unit (the slowest files first)
SOURCES = ["lookup_lean_i64_exact.hip", "lookup_lean_i64_fast.hip", "lookup_lean_i32_exact.hip", "lookup_lean_i32_fast.hip",
           "lookup_lean_i64_exact_w4.hip", "lookup_lean_i64_fast_w4.hip", "lookup_lean_i32_exact_w4.hip", "lookup_lean_i32_fast_w4.hip",
           "lookup_lean_i64_exact_q8.hip", "lookup_lean_i64_fast_q8.hip", "lookup_lean_i32_exact_q8.hip", "lookup_lean_i32_fast_q8.hip",
           "lookup_i64.hip", "lookup_i32.hip", "lookup_i64_general.hip", "lookup_i32_general.hip",
           "lookup_kernels.hip", "index_ops_kernels.hip", "quantize_kernels.hip", "sequence_kernels.hip",
           "prune_kernels.hip", "remap_rank_kernels.hip", "split_bag_kernels.hip", "update_kernels.hip", "c_api.cpp"]
HEADERS = ["cache_policy.h", "launchers.h", "lookup_common.h", "lookup_device.h", "lookup_general.h", "lookup_lean.h", os.path.join("..", "..", "include", "fbgemm_amd.h"),
           os.path.join("..", "..", "include", "fbgemm_amd_bench.h")]

# -ffp-contract=off: the kernels spell out every fma; nothing else may be fused,
#   or the fp32 rounding sequence would differ from the reference's.
# -packed-fp32-ops off: keep the compiler from forming packed fp32 instructions.
FLAGS = [
    "-x", "hip", "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # error reporting uses a few atomics on one address; keep them as plain
    # atomics instead of a wave-wide reduction loop in front of each
    "-mllvm", "-amdgpu-atomic-optimizer-strategy=None",
]


def _hipcc(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only target feature; that warning is noise
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{out}")
    return out


def build_library(verbose=False, force=True):
    """Compile every source to an object (side by side) and link them.
    ``force=False`` keeps objects that are newer than their source and the
    shared headers (for edit-compile loops); the default compiles everything."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(HERE, "lib", "obj")
    os.makedirs(objdir, exist_ok=True)
    newest_header = max(os.path.getmtime(os.path.join(CSRC, h)) for h in HEADERS)
    jobs = []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        stale = force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(path), newest_header)
        if stale:
            jobs.append(["hipcc", *FLAGS, "-c", "-o", obj, path])
    if verbose:
        for j in jobs:
            print(" ".join(j), flush=True)
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 4)) as pool:
        outs = list(pool.map(_hipcc, jobs))
    objs = [os.path.join(objdir, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    outs.append(_hipcc(["hipcc", "--offload-arch=gfx950", "-fPIC", "-shared", "-o", OUT, *objs]))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    return OUT


BENCH_OUT = os.path.join(HERE, "lib", "libfbgemm_amd_bench.so")


def build_bench_library(verbose=False):
    """The benchmark-only library: yardstick kernels for profiles (include/fbgemm_amd_bench.h).
    Not linked into the product library and not loaded by it."""
    cmd = ["hipcc", "-x", "hip", "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-o", BENCH_OUT, os.path.join(CSRC, "bench_kernels.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = _hipcc(cmd)
    if verbose and out.strip():
        print(out)
    return BENCH_OUT


TORCH_OP_OUT = os.path.join(HERE, "lib", "libfbgemm_amd_torch.so")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"{cmd[0]} failed:\n{proc.stdout}")


def build_torch_op(verbose=False):
    """The torch operator library (schema registration + CUDA-key kernels).
    Host code only: g++ against the torch headers, linked to libfbgemm_amd.so."""
    import torch

    tdir = os.path.dirname(torch.__file__)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi()),
           f"-I{tdir}/include", f"-I{tdir}/include/torch/csrc/api/include", "-I/opt/rocm/include",
           "-o", TORCH_OP_OUT, os.path.join(CSRC, "torch_op.cpp"),
           f"-L{os.path.dirname(OUT)}", "-lfbgemm_amd", f"-L{tdir}/lib", "-ltorch_cpu", "-lc10", "-lc10_hip",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tdir}/lib"]
    _run(cmd, verbose)
    return TORCH_OP_OUT


if __name__ == "__main__":
    print(build_library(verbose=True, force="--incremental" not in sys.argv))
    print(build_bench_library(verbose=True))
    print(build_torch_op(verbose=True))
    sys.exit(0)
