"""The eviction rule of the library's two bounded caches (a plan's work lists per batch size, the
torch operator's plans per metadata set), on the host: the least recently used entry goes, never
one that a captured HIP graph may hold. The rule is a header shared by both caches; this test
builds tests/cpp/test_cache_policy.cpp against it with g++ and runs it. No GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_eviction_rule(tmp_path):
    exe = str(tmp_path / "test_cache_policy")
    src = os.path.join(ROOT, "tests", "cpp", "test_cache_policy.cpp")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-o", exe, src])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and "PASSED" in out.stdout, out.stdout + out.stderr
