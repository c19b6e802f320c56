"""The library's host plumbing without a GPU: homura_amd/csrc/runtime.hip and memory.hip are compiled as plain C++
against a scripted HIP runtime (tests/fake_hip) and driven through their failure paths by
tests/host_plumbing_check.cpp - every step of hmr_context_create failing in turn and what it leaves behind, the
exception fence, HIP's sticky last error, the caller's current device, the armed test failures, per-thread
messages (ref: csrc/tests/host_failures.cpp tests the reference's plumbing the same way). Built with the
address and undefined-behaviour sanitizers: a leak or a use after free in an unwinding path fails the run."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_failure_paths_of_the_runtime_and_memory_entry_points(tmp_path):
    exe = tmp_path / "host_plumbing_check"
    subprocess.check_call(
        ["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Werror", "-x", "c++", "-fsanitize=address,undefined",
         "-fno-sanitize-recover=undefined", '-DHMR_OFFLOAD_ARCHS="gfx950"', "-I", os.path.join(ROOT, "tests", "fake_hip"),
         "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "homura_amd", "csrc"),
         os.path.join(ROOT, "tests", "host_plumbing_check.cpp"), "-o", str(exe), "-lpthread"])
    # The harness preloads a library of its own, which the address sanitizer's start-up check would refuse.
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    done = subprocess.run([str(exe)], capture_output=True, text=True, env=env, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.strip().endswith("host plumbing ok")
