"""The restated f32 library functions (homura_amd/csrc/expf_like_libm.hpp, f32_like_libm.hpp) against the host C
library's, on the CPU.

The GPU's exp, expm1, tanh and log1p for f32 values restate the algorithms of the host's expf, expm1f, tanhf and
log1pf so that exp, sigmoid, silu, tanh, gelu_tanh and log_sigmoid get the CPU's bits. tests/libm_check.cpp compiles
the same headers for the host and compares each function with the library's, bit for bit. Over all 2^32 inputs none
of the four differs (expf in the fused form, which is what the library builds; its unfused form differs for two);
that walk takes half a minute of eight cores a function (`libm_check tanhf 1`), so the suite walks every 61st
pattern: 70 million inputs a function, every binade and both tails."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("libm") / "libm_check")
    subprocess.run(["g++", "-std=c++17", "-O2", "-Wall", "-Werror", "-ffp-contract=off", "-I", os.path.join(ROOT, "tests", "fake_hip"),
                    "-I", os.path.join(ROOT, "homura_amd", "csrc"), os.path.join(ROOT, "tests", "libm_check.cpp"), "-o", exe,
                    "-lpthread"], check=True)
    return exe


@pytest.mark.parametrize("function", ["expf", "expm1f", "tanhf", "log1pf"])
def test_the_restated_function_has_the_host_librarys_bits(checker, function):
    out = subprocess.run([checker, function, "61"], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "0 differ", out


def test_the_unfused_expf_differs_for_two_inputs_at_most(checker):
    out = subprocess.run([checker, "expf", "61", "0"], check=True, capture_output=True, text=True).stdout
    assert int(out.split()[0]) <= 2, out
