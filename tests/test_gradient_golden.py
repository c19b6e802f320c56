"""The gradients of the reductions and of softmax against PyTorch's (tests/golden/grads.safetensors, the data file of
ref: tests/autograd_golden.rs, written by the reference's tools/golden/gen_grads.py).

The host layer composes each gradient from the forward ops as the reference's backward nodes do (ref:
src/autograd/formulas/reduce.rs, softmax.rs), so these cases check the path end to end in the form training uses it:
broadcast gradients (expand, sum_to_size), mean / var / std scaling, the tie and NaN rules of max / min, softmax's
y * (g - sum(g * y)) with f32 intermediates for the halves. For an input with zeros the gradient of prod is g times
exclusive_cumprod(x) * exclusive_cumprod(x, reverse): the `special.prod*` cases compare exactly (ref:
tests/autograd_golden.rs:236-246) and fix that kernel's multiplication order, accumulation type and rounding point.
The gradient of max_dim / min_dim scatters g through the saved indices (scatter_add). On the CPU this pins the oracle's
exclusive_cumprod; on the GPU everything runs on the HIP kernels.
"""
import os

import numpy as np
import pytest

from tests import oracle
from tests.support import DT, GPU, array, h, load_golden, tensor, to_f64

h.register_cpu_backend(oracle.backend_address())
GOLDEN = load_golden(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "grads.safetensors"))
# rtol = atol, as the reference's test takes them (ref: tests/autograd_golden.rs:236-246, tests/common/mod.rs:103-113).
TOL = {DT.F16: 2.0 ** -10, DT.BF16: 2.0 ** -7, DT.F32: 1e-5, DT.F64: 1e-12}

# op -> the input gradient from x and g, through the forward op where the node saves its result
# (ref: tests/autograd_golden.rs:32-33, 107-135, 164-169).
OPS = {
    "sum": lambda x, g: h.grad_sum(g, x.shape, [], False),
    "sum_dim": lambda x, g: h.grad_sum(g, x.shape, [1], False),
    "sum_dims_keep": lambda x, g: h.grad_sum(g, x.shape, [0, 2], True),
    "sum_to_size": lambda x, g: h.grad_sum_to_size(g, x.shape),
    "mean": lambda x, g: h.grad_mean(g, x.shape, [], False),
    "mean_dim": lambda x, g: h.grad_mean(g, x.shape, [-1], False),
    "mean_dims_keep": lambda x, g: h.grad_mean(g, x.shape, [0, 1], True),
    "prod": lambda x, g: h.grad_prod(g, x, x.prod(), None, False),
    "prod_dim": lambda x, g: h.grad_prod(g, x, x.prod_dim(1, False), 1, False),
    "prod_dim_keep": lambda x, g: h.grad_prod(g, x, x.prod_dim(0, True), 0, True),
    "max": lambda x, g: h.grad_extremum(g, x, x.max()),
    "min": lambda x, g: h.grad_extremum(g, x, x.min()),
    "max_dim": lambda x, g: h.grad_extremum_dim(g, x.max_dim(1, False)[1], x.shape, 1, False),
    "min_dim_keep": lambda x, g: h.grad_extremum_dim(g, x.min_dim(0, True)[1], x.shape, 0, True),
    "var": lambda x, g: h.grad_var_std(g, x, None, [], 1, False),
    "var_c2": lambda x, g: h.grad_var_std(g, x, None, [], 2, False),
    "var_c4": lambda x, g: h.grad_var_std(g, x, None, [], 4, False),
    "var_dim": lambda x, g: h.grad_var_std(g, x, None, [1], 1, False),
    "var_dim_c3": lambda x, g: h.grad_var_std(g, x, None, [1], 3, False),
    "var_dim_c4": lambda x, g: h.grad_var_std(g, x, None, [1], 4, False),
    "var_dims_keep": lambda x, g: h.grad_var_std(g, x, None, [0, 1], 0, True),
    "std": lambda x, g: h.grad_var_std(g, x, x.std(1), [], 1, False),
    "std_c3": lambda x, g: h.grad_var_std(g, x, x.std(3), [], 3, False),
    "std_dim": lambda x, g: h.grad_var_std(g, x, x.std_dim([0], 2, False), [0], 2, False),
    "std_dim_c4": lambda x, g: h.grad_var_std(g, x, x.std_dim([1], 4, False), [1], 4, False),
    "softmax_dim1": lambda x, g: h.grad_softmax(g, x.softmax(1), 1, False),
    "softmax_last": lambda x, g: h.grad_softmax(g, x.softmax(-1), -1, False),
    "log_softmax_dim0": lambda x, g: h.grad_softmax(g, x.log_softmax(0), 0, True),
    "log_softmax_last": lambda x, g: h.grad_softmax(g, x.log_softmax(-1), -1, True),
}
ALIASES = {"prod_zero": "prod", "prod_two_zeros": "prod", "prod_overflow": "prod", "prod_order_bf16": "prod",
           "prod_dim_zeros": "prod_dim", "prod_dim_overflow": "prod_dim", "prod_dim_order_f64": "prod_dim",
           "prod_dim_order_f32": "prod_dim", "prod_dim_order_f16": "prod_dim", "prod_dim_order_bf16": "prod_dim",
           "max_ties": "max", "softmax_masked": "softmax_last", "softmax_opmath_f16": "softmax_last",
           "log_softmax_masked": "log_softmax_last", "log_softmax_opmath_bf16": "log_softmax_last"}
FAMILIES = ("sum", "mean", "prod", "max", "min", "var", "std", "softmax", "log_softmax")


def on_the_path(case):
    op = case.partition(".")[2]
    return any(op == f or op.startswith(f + "_") for f in FAMILIES)


CASES = sorted(c for c in GOLDEN if on_the_path(c))


def check(case, device):
    tensors = GOLDEN[case]
    category, _, op = case.partition(".")
    assert set(tensors) == {"x", "g", "grad_x"}, case
    (xa, xd), (ga, gd), (ea, ed) = tensors["x"], tensors["g"], tensors["grad_x"]
    x, g = tensor(xa, xd, list(xa.shape), device), tensor(ga, gd, list(ga.shape), device)
    grad = OPS[ALIASES.get(op, op)](x, g)
    assert grad.dtype == ed and list(grad.shape) == list(ea.shape) and grad.device == device, case
    got, want = to_f64(array(grad.contiguous()), ed).reshape(-1), to_f64(ea, ed).reshape(-1)
    tol = 0.0 if category == "special" else TOL[ed]
    for i, (a, e) in enumerate(zip(got, want)):
        if np.isnan(a) or np.isnan(e):
            ok = np.isnan(a) and np.isnan(e)
        elif tol == 0.0:
            ok = a == e and np.signbit(a) == np.signbit(e)
        elif np.isinf(a) or np.isinf(e):
            ok = a == e
        else:
            ok = abs(a - e) <= tol + tol * abs(e)
        assert ok, f"{case} on {device}: element {i}: got {a!r}, PyTorch's is {e!r}"


def test_every_reduction_and_softmax_gradient_of_the_fixture_is_handled():
    assert len(CASES) == 71
    # The cases that reach the cumulative products: every dtype's accumulation order, overflowing partial products,
    # one zero and two.
    with_zeros = {c for c in CASES if "prod" in c and (GOLDEN[c]["x"][0] == 0).any()}
    assert {"special.prod_dim_order_f16", "special.prod_dim_order_bf16", "special.prod_dim_order_f32",
            "special.prod_dim_order_f64", "special.prod_order_bf16", "special.prod_dim_overflow", "special.prod_overflow",
            "special.prod_two_zeros", "grad.prod_zero", "grad.prod_dim_zeros"} <= with_zeros, with_zeros


@pytest.mark.parametrize("case", CASES)
def test_gradients_on_cpu_oracle(case):
    check(case, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_gradients_on_gpu(case):
    check(case, GPU)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [DT.BF16, DT.F32, DT.F64])
def test_gradients_of_larger_tensors_match_the_cpu(dtype):
    """The same compositions at sizes where the reductions take their split plans (ref: tests/rocm_autograd_reduce.rs):
    the GPU against the oracle within the fixture's tolerance for the dtype, every element."""
    from tests.support import from_f64, normal
    rows, cols = 96, 3000
    x = tensor(from_f64(normal(21, rows * cols), dtype), dtype).reshape([rows, cols])
    x = x.masked_fill(x.abs().less(0.02), 0.0)  # some exact zeros, for prod
    g_full = tensor(from_f64(normal(22, rows * cols), dtype), dtype).reshape([rows, cols])
    g_rows = tensor(from_f64(normal(23, rows), dtype), dtype)
    small = x.narrow(1, 0, 12).mul(1.5)
    pairs = {
        "softmax": lambda d: h.grad_softmax(g_full.to(d), x.to(d).softmax(-1), -1, False),
        "log_softmax dim 0": lambda d: h.grad_softmax(g_full.to(d), x.to(d).log_softmax(0), 0, True),
        "mean_dim": lambda d: h.grad_mean(g_rows.to(d), x.shape, [1], False),
        "var_dim": lambda d: h.grad_var_std(g_rows.to(d), x.to(d), None, [1], 1, False),
        "std_dim": lambda d: h.grad_var_std(g_rows.to(d), x.to(d), x.to(d).std_dim([1], 1, False), [1], 1, False),
        "max": lambda d: h.grad_extremum(g_rows.to(d).narrow(0, 0, 1).reshape([]), x.to(d), x.to(d).max()),
        "prod_dim with zeros": lambda d: h.grad_prod(g_rows.to(d), small.to(d), small.to(d).prod_dim(1, False), 1, False),
        "sum_to_size": lambda d: h.grad_sum_to_size(g_rows.to(d).reshape([rows, 1]), x.shape),
    }
    for name, f in pairs.items():
        close_to_the_cpu(f(GPU), f("cpu"), dtype, name)


def close_to_the_cpu(gpu, cpu, dtype, name):
    """Every element within the fixture's tolerance for the dtype (relative to the element, for the compositions
    that subtract also to the largest element), NaNs in the same places."""
    tol = TOL[dtype]
    assert gpu.device == GPU and gpu.dtype == dtype and gpu.shape == cpu.shape, name
    a, e = to_f64(array(gpu.contiguous()), dtype).reshape(-1), to_f64(array(cpu.contiguous()), dtype).reshape(-1)
    nan = np.isnan(a) | np.isnan(e)
    assert (np.isnan(a) == np.isnan(e)).all(), name
    if a.size == 0:
        return
    with np.errstate(all="ignore"):
        scale = np.abs(e) + (np.nanmax(np.abs(e)) if name.startswith(("softmax", "log_softmax", "var", "std")) else 0.0)
        bad = ~nan & ~(np.abs(a - e) <= tol * scale + 1e-300) & ~(a == e)
    assert not bad.any(), f"{name} {dtype}: element {np.nonzero(bad)[0][0]}: gpu {a[bad][0]!r}, cpu {e[bad][0]!r}"


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(6))
def test_gradients_over_random_shapes_and_dimensions_match_the_cpu(seed):
    """The same compositions with shapes, dimensions, keepdim and corrections drawn from a seeded generator."""
    from tests.support import from_f64, normal
    rng = np.random.default_rng(0x5EED7000 + seed)
    for case in range(25):
        dtype = [DT.BF16, DT.F32, DT.F64, DT.F16][int(rng.integers(0, 4))]
        shape = [int(rng.choice([1, 2, 3, 7, 16, 65, 300])) for _ in range(int(rng.integers(1, 4)))]
        n, nd = int(np.prod(shape)), len(shape)
        x = tensor(from_f64(normal(50 * seed + case, n), dtype), dtype).reshape(shape)
        dims = sorted(int(d) for d in rng.choice(nd, int(rng.integers(1, nd + 1)), replace=False))
        keep = bool(rng.integers(0, 2))
        d = int(rng.integers(0, nd))
        correction = int(rng.integers(0, 3))
        reduced = x.sum_dim(dims, keep)
        g_red = tensor(from_f64(normal(51 * seed + case, reduced.num_elements()), dtype), dtype).reshape(reduced.shape)
        g_full = tensor(from_f64(normal(52 * seed + case, n), dtype), dtype).reshape(shape)
        one = x.max_dim(d, keep)[0]
        g_one = tensor(from_f64(normal(53 * seed + case, one.num_elements()), dtype), dtype).reshape(one.shape)
        what = f"seed {seed} case {case}: {dtype} {shape} dims {dims} keep {keep} along {d} correction {correction}"
        pairs = {
            "sum": lambda v: h.grad_sum(g_red.to(v), shape, dims, keep),
            "mean": lambda v: h.grad_mean(g_red.to(v), shape, dims, keep),
            "var": lambda v: h.grad_var_std(g_red.to(v), x.to(v), None, dims, correction, keep),
            "std": lambda v: h.grad_var_std(g_red.to(v), x.to(v), x.to(v).std_dim(dims, correction, keep), dims, correction, keep),
            "softmax": lambda v: h.grad_softmax(g_full.to(v), x.to(v).softmax(d), d, False),
            "log_softmax": lambda v: h.grad_softmax(g_full.to(v), x.to(v).log_softmax(d), d, True),
            "max_dim": lambda v: h.grad_extremum_dim(g_one.to(v), x.to(v).max_dim(d, keep)[1], shape, d, keep),
            "prod_dim": lambda v: h.grad_prod(g_one.to(v), x.to(v), x.to(v).prod_dim(d, keep), d, keep),
        }
        for name, f in pairs.items():
            try:
                cpu = f("cpu")
            except Exception as refusal:
                with pytest.raises(type(refusal)) as got:
                    f(GPU)
                assert str(got.value) == str(refusal), f"{what}: {name}"
                continue
            close_to_the_cpu(f(GPU), cpu, dtype, f"{name} ({what})")
