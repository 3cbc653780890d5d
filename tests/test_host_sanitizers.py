"""The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer, on the CPU:
fbgemm_amd/csrc/c_api.cpp is built with g++ against a host-only stand-in for the HIP runtime
(tests/cpp/hip_stub: "device" memory is malloc'ed, launches do nothing) and driven through the
lifetimes of plans, cached work lists, per-stream and per-thread scratch
(tests/cpp/test_host_sanitized.cpp). A use after free, a double free, an overrun, a leak or
undefined arithmetic ends the program with a report. (The reference builds its tests with the
same sanitizers: CMakeLists.txt:97,199-200.) No GPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_code_under_asan_and_ubsan(tmp_path):
    exe = str(tmp_path / "test_host_sanitized")
    cpp = os.path.join(ROOT, "tests", "cpp")
    cmd = ["g++", "-std=c++17", "-g", "-O1", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-fno-omit-frame-pointer", "-static-libasan", "-pthread", f"-I{os.path.join(cpp, 'hip_stub')}",
           "-o", exe, os.path.join(cpp, "test_host_sanitized.cpp"), os.path.join(cpp, "hip_stub", "hip_stub.cpp"),
           os.path.join(ROOT, "fbgemm_amd", "csrc", "c_api.cpp")]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)
    out = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=600)
    assert out.returncode == 0 and "PASSED" in out.stdout, (out.stdout + out.stderr)[-6000:]
