"""exclusive_cumprod against PyTorch's gradients of prod (tests/golden/grads.safetensors, the data file of ref:
tests/autograd_golden.rs, written by the reference's tools/golden/gen_grads.py).

For an input with zeros the gradient of prod is g times the product of all the other elements of the slice, which the
reference computes without dividing as exclusive_cumprod(x) * exclusive_cumprod(x, reverse) (ref:
src/autograd/formulas/reduce.rs:258-329). The `special.*` cases are compared exactly (ref: tests/autograd_golden.rs:
239-241): they fix the order of the multiplications, the accumulation type of each dtype and where the result is
rounded. On the CPU this pins the oracle's exclusive_cumprod; on the GPU it checks hmr_exclusive_cumprod.
"""
import os

import numpy as np
import pytest

from tests import oracle
from tests.support import DT, GPU, array, h, load_golden, tensor, to_f64

h.register_cpu_backend(oracle.backend_address())
GOLDEN = load_golden(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "grads.safetensors"))
CASES = sorted(c for c in GOLDEN if c.partition(".")[2].startswith("prod"))
# rtol = atol, as the reference's test takes them (ref: tests/autograd_golden.rs:236-246, tests/common/mod.rs:103-113).
TOL = {DT.F16: 2.0 ** -10, DT.BF16: 2.0 ** -7, DT.F32: 1e-5, DT.F64: 1e-12}


def prod_gradient(x, g, dim, keepdim):
    """The input gradient of x.prod() (dim None) or x.prod_dim(dim, keepdim) for the output gradient g, as
    ProdBackward::apply computes it outside grad mode (ref: src/autograd/formulas/reduce.rs:281-316)."""
    if len(x.shape) == 0:
        return g
    result = x.prod() if dim is None else x.prod_dim(dim, keepdim)
    if dim is not None and not keepdim:
        kept = list(x.shape)
        kept[dim] = 1
        g, result = g.reshape(kept), result.reshape(kept)
    zeros = int(array(x.equal(0.0).sum()))
    if zeros == 0:
        return g.mul(result.div(x))
    if dim is None and zeros > 1:
        return h.full(list(x.shape), 0.0, x.dtype, x.device)
    flat, d = (x.reshape([-1]), 0) if dim is None else (x, dim)
    if flat.shape[d] == 1:
        return g.reshape(list(x.shape))
    others = h.exclusive_cumprod(flat, d, False).mul(h.exclusive_cumprod(flat, d, True))
    return g.mul(others).reshape(list(x.shape))


def check(case, device):
    tensors = GOLDEN[case]
    category, _, op = case.partition(".")
    (xa, xd), (ga, gd), (ea, ed) = tensors["x"], tensors["g"], tensors["grad_x"]
    assert set(tensors) == {"x", "g", "grad_x"}
    x, g = tensor(xa, xd, list(xa.shape), device), tensor(ga, gd, list(ga.shape), device)
    dim, keepdim = (None, False) if not op.startswith("prod_dim") else ((0, True) if op == "prod_dim_keep" else (1, False))
    grad = prod_gradient(x, g, dim, keepdim)
    assert grad.dtype == ed and list(grad.shape) == list(ea.shape) and grad.device == device, case
    got, want = to_f64(array(grad), ed).reshape(-1), to_f64(ea, ed).reshape(-1)
    tol = 0.0 if category == "special" else TOL[ed]
    for i, (a, e) in enumerate(zip(got, want)):
        if np.isnan(a) or np.isnan(e):
            ok = np.isnan(a) and np.isnan(e)
        elif np.isinf(a) or np.isinf(e) or tol == 0.0:
            ok = a == e and np.signbit(a) == np.signbit(e) if tol == 0.0 else a == e
        else:
            ok = abs(a - e) <= tol + tol * abs(e)
        assert ok, f"{case} on {device}: element {i}: got {a!r}, PyTorch's is {e!r}"
    return int(array(x.equal(0.0).sum()))


def test_the_fixture_has_cases_that_reach_the_cumulative_products():
    assert len(CASES) == 16
    with_zeros = [c for c in CASES if (GOLDEN[c]["x"][0] == 0).any()]
    # Every dtype's accumulation order, overflowing partial products, one zero and two.
    assert {"special.prod_dim_order_f16", "special.prod_dim_order_bf16", "special.prod_dim_order_f32",
            "special.prod_dim_order_f64", "special.prod_order_bf16", "special.prod_dim_overflow", "special.prod_overflow",
            "special.prod_two_zeros", "grad.prod_zero", "grad.prod_dim_zeros"} <= set(with_zeros), with_zeros


@pytest.mark.parametrize("case", CASES)
def test_prod_gradients_on_cpu_oracle(case):
    check(case, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_prod_gradients_on_gpu(case):
    check(case, GPU)
