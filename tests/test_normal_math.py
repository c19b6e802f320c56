"""The f64 polynomials behind hmr_random_normal's 16- and 32-bit outputs (homura_amd/csrc/normal_math.hpp),
run on the host by tests/normal_math_check.cpp against long double functions: the logarithm, the square root and the
sine / cosine pair each stay within 2^-49 of their value over three million draws and the corners (u1 = 2^-53 and 1,
u2 on and next to the eighth turns), with the hardware's reciprocal estimates replaced by ones cut to 22 bits. The
GPU's samples are checked against the CPU backend's in tests/test_random.py
(ref: tests/rocm_random.rs:145-222, whose bound is 6 * 2^-53 * M plus one output ulp)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_polynomials_of_the_normal_pair_are_within_2_to_the_minus_49(tmp_path):
    exe = tmp_path / "normal_math_check"
    subprocess.check_call(
        ["g++", "-std=c++17", "-O2", "-Wall", "-Werror", "-I", os.path.join(ROOT, "tests", "fake_hip"),
         "-I", os.path.join(ROOT, "homura_amd", "csrc"), os.path.join(ROOT, "tests", "normal_math_check.cpp"),
         "-o", str(exe)])
    done = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.strip().endswith("normal math ok")
