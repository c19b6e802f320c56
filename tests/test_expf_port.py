"""homura_amd/csrc/expf_like_libm.hpp against the host C library's expf, on the CPU.

The GPU's exp for f32 values restates the algorithm of the host's expf so that exp, sigmoid, silu and log_sigmoid get
the CPU's bits. tests/expf_check.cpp compiles the same header for the host and compares it with expf bit for bit. Over
all 2^32 inputs the fused form (what the library builds) differs for none and the unfused form for two; that run
takes half a minute of eight cores, so the suite walks every 61st pattern (70 million inputs, every binade and both
tails) and the full walk is one command: `expf_check 1 1`."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_restated_expf_has_the_host_librarys_bits(tmp_path):
    exe = str(tmp_path / "expf_check")
    subprocess.run(["g++", "-std=c++17", "-O2", "-Wall", "-Werror", "-ffp-contract=off", "-I", os.path.join(ROOT, "tests", "fake_hip"),
                    "-I", os.path.join(ROOT, "homura_amd", "csrc"), os.path.join(ROOT, "tests", "expf_check.cpp"), "-o", exe,
                    "-lpthread"], check=True)
    fused = subprocess.run([exe, "61", "1"], check=True, capture_output=True, text=True).stdout
    assert fused.strip() == "0 differ", fused
    plain = subprocess.run([exe, "61", "0"], check=True, capture_output=True, text=True).stdout
    assert int(plain.split()[0]) <= 2, plain
