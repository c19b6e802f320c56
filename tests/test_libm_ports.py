"""The restated f32 library functions (homura_amd/csrc/expf_like_libm.hpp, f32_like_libm.hpp) against the host C
library's, on the CPU.

The GPU's exp, log, sin, cos, expm1, tanh and log1p for f32 values restate the algorithms of the host's expf, logf,
sinf, cosf, expm1f, tanhf and log1pf so that exp, log, sin, cos, sigmoid, silu, tanh, gelu_tanh and log_sigmoid get
the CPU's bits; pow restates powf. tests/libm_check.cpp compiles
the same headers for the host and compares each function with the library's, bit for bit. Over all 2^32 inputs none
of the seven differs (expf, sinf, cosf and logf in the fused form, which is what the library builds; unfused, expf
differs for 2 inputs, sinf for 12, cosf for 22);
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


@pytest.mark.parametrize("function", ["expf", "expm1f", "tanhf", "log1pf", "sinf", "cosf", "logf"])
def test_the_restated_function_has_the_host_librarys_bits(checker, function):
    out = subprocess.run([checker, function, "61"], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "0 differ", out


@pytest.mark.parametrize("function", ["tanh", "expm1"])
def test_the_restated_f64_functions_have_the_host_librarys_bits(checker, function):
    """f64: sampled, 24 million inputs here (arbitrary bits, (-25, 25), (-2, 2), every binade down to 2^-70);
    `libm_check tanh 1` draws 480 million and differs for none either."""
    out = subprocess.run([checker, function, "20"], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "0 differ", out


def test_the_restated_powf_has_the_host_librarys_bits(checker):
    """Two arguments, so no walk over all inputs: 26 exponents times every 251st base and 8 million random pairs here;
    `libm_check powf 7` (every 7th base, 286 million pairs, four minutes of eight cores) differs for none either."""
    out = subprocess.run([checker, "powf", "251"], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "0 differ", out


@pytest.mark.parametrize("function, most", [("expf", 2), ("sinf", 12), ("cosf", 22), ("logf", 0)])
def test_the_unfused_forms_differ_for_a_handful_of_inputs_at_most(checker, function, most):
    out = subprocess.run([checker, function, "61", "0"], check=True, capture_output=True, text=True).stdout
    assert int(out.split()[0]) <= most, out
