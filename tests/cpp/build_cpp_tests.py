"""Builds the C++ test programs of tests/cpp: ``python tests/cpp/build_cpp_tests.py``.

test_factories: the C++ factory templates (include/fbgemm_amd_embedding.hpp) against the C oracle,
on the GPU. hipcc cross-compiles it without a GPU; the GPU tests run what is built here."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT_DIR = os.path.join(HERE, "_build")
TEST_FACTORIES = os.path.join(OUT_DIR, "test_factories")


def build_test_factories(verbose=False):
    libdir = os.path.join(ROOT, "fbgemm_amd", "lib")
    obuild = os.path.join(ROOT, "oracle", "_build")
    os.makedirs(OUT_DIR, exist_ok=True)
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "oracle"])
    cmd = ["hipcc", "-x", "hip", "-O2", "--offload-arch=gfx950", "-std=c++17", "-o", TEST_FACTORIES,
           os.path.join(HERE, "test_factories.cpp"), f"-L{libdir}", "-lfbgemm_amd",
           f"-L{obuild}", "-lembedding_oracle", f"-Wl,-rpath,{libdir}", f"-Wl,-rpath,{obuild}"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{proc.stdout}")
    return TEST_FACTORIES


if __name__ == "__main__":
    print(build_test_factories(verbose=True))
    sys.exit(0)
