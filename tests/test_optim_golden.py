"""The optimizers' fused steps against the reference's own optimizer fixtures: several steps of SGD,
Adam and AdamW in F16 / BF16 / F32 / F64, bit for bit with PyTorch's vectorised CPU kernels
(tests/golden/m2_optim.safetensors and m2_optim_edges.safetensors, the data files of ref:
tests/optim.rs:158-262, written by the reference's tools/golden/gen_m2_optim.py).

A step is ScaledAdd / Lerp / Addcmul / Addcdiv with one rounding each (ref: src/backend/cpu/mod.rs:509-569)
around a few plain elementwise ops, so these fixtures fix where every FMA sits and how each coefficient is
rounded. On the CPU they pin the oracle's `fused`; on the GPU they check hmr_fused through the host layer.
"""
import os

import numpy as np
import pytest

from tests import oracle
from tests.support import DT, GPU, array, assert_bitwise, bits, from_f64, h, load_golden, normal, tensor

h.register_cpu_backend(oracle.backend_address())

HERE = os.path.dirname(os.path.abspath(__file__))
MULTI = load_golden(os.path.join(HERE, "golden", "m2_optim.safetensors"))
EDGES = load_golden(os.path.join(HERE, "golden", "m2_optim_edges.safetensors"))
STEPS = 5


def same_bits(actual, expected, what):
    """ref: tests/optim.rs:44-56: dtype, shape and bits, where a NaN only has to meet a NaN."""
    arr, dtype = expected
    assert actual.dtype == dtype, f"{what}: dtype {actual.dtype}"
    assert list(actual.shape) == list(arr.shape), f"{what}: shape {actual.shape}"
    got = array(actual)
    view = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[got.dtype.itemsize]
    g, e = got.reshape(-1).view(view), arr.reshape(-1).view(view)
    if dtype in (DT.F32, DT.F64):
        both_nan = np.isnan(got.reshape(-1)) & np.isnan(arr.reshape(-1))
    else:
        top = 0x7C00 if dtype == DT.F16 else 0x7F80
        both_nan = ((g & 0x7FFF) > top) & ((e & 0x7FFF) > top)
    bad = np.nonzero((g != e) & ~both_nan)[0]
    assert bad.size == 0, f"{what}: element {bad[0]} is {int(g[bad[0]]):#x}, PyTorch's is {int(e[bad[0]]):#x}"


class Group:
    """One parameter group of a case's optimizer (ref: tests/optim.rs:95-157)."""

    def __init__(self, kind, case, lr_scale):
        opt = lambda name: float(case["opt." + name][0])
        self.kind = kind
        self.lr = lr_scale * opt("lr")
        if kind == "sgd":
            self.o = dict(momentum=opt("momentum"), dampening=opt("dampening"), weight_decay=opt("weight_decay"),
                          nesterov=opt("nesterov") != 0.0, maximize=opt("maximize") != 0.0)
        else:
            self.o = dict(beta1=opt("beta1"), beta2=opt("beta2"), eps=opt("eps"), weight_decay=opt("weight_decay"),
                          amsgrad=opt("amsgrad") != 0.0, maximize=opt("maximize") != 0.0,
                          decoupled_weight_decay=kind == "adamw")

    def step(self, p, grad, state):
        if self.kind == "sgd":
            return h.sgd_step(p, grad, state, lr=self.lr, **self.o)
        return h.adam_step(p, grad, state, lr=self.lr, **self.o)

    def state_tensors(self, state):
        """{PyTorch's name: tensor or number} of a parameter's state."""
        if state is None:
            return {}
        if self.kind == "sgd":
            return {"momentum_buffer": state}
        out = {"step": state[0], "exp_avg": state[1], "exp_avg_sq": state[2]}
        if state[3] is not None:
            out["max_exp_avg_sq"] = state[3]
        return out


def check_after(case, name, t, n, p, group, state, used):
    key = f"after{t}.{n}"
    same_bits(p, case[key], f"{name}/{key}")
    used.add(key)
    tensors = group.state_tensors(state)
    stored = {k for k in case if k.startswith(key + ".")}
    assert {f"{key}.{s}" for s in tensors} == stored, f"{name}: state of {n} after step {t}"
    for s, value in tensors.items():
        arr, dtype = case[f"{key}.{s}"]
        if s == "step":
            assert dtype == DT.F32 and float(arr) == value, f"{name}/{key}.step"
        else:
            same_bits(value, (arr, dtype), f"{name}/{key}.{s}")
        used.add(f"{key}.{s}")


def run_multi(name, device):
    """ref: tests/optim.rs:159-211: parameters a and c in the first group, b in a second with twice the learning
    rate; the first group's rate is halved before the third step; a parameter without a gradient is skipped."""
    case = MULTI[name]
    kind = name.split(".")[0].split("_")[0]
    groups = {"a": Group(kind, case, 1.0), "c": Group(kind, case, 1.0), "b": Group(kind, case, 2.0)}
    used = {k for k in case if k.startswith("opt.")}
    params, states = {}, {}
    for n in "abc":
        arr, dtype = case[f"init.{n}"]
        params[n], states[n] = tensor(arr, dtype, list(arr.shape), device), None
        used.add(f"init.{n}")
    for t in range(STEPS):
        if t == 2:
            groups["a"].lr *= 0.5
            groups["c"].lr *= 0.5
        for n in "abc":
            key = f"grad{t}.{n}"
            if key in case:
                arr, dtype = case[key]
                used.add(key)
                params[n], states[n] = groups[n].step(params[n], tensor(arr, dtype, list(arr.shape), device), states[n])
        for n in "abc":
            check_after(case, name, t, n, params[n], groups[n], states[n], used)
    assert used == set(case), f"{name}: unused {set(case) - used}"


def run_edges(name, device):
    """ref: tests/optim.rs:217-254"""
    case = EDGES[name]
    kind = name.split(".")[0].split("_")[0]
    group = Group(kind, case, 1.0)
    used = {k for k in case if k.startswith("opt.")} | {"init.p"}
    arr, dtype = case["init.p"]
    p, state = tensor(arr, dtype, list(arr.shape), device), None
    t = 0
    while f"grad{t}.p" in case:
        arr, dtype = case[f"grad{t}.p"]
        used.add(f"grad{t}.p")
        p, state = group.step(p, tensor(arr, dtype, list(arr.shape), device), state)
        check_after(case, name, t, "p", p, group, state, used)
        t += 1
    assert t > 0 and used == set(case), f"{name}: unused {set(case) - used}"


def test_the_fixtures_are_the_references():
    assert len(MULTI) == 4 * 10 and len(EDGES) == 18


@pytest.mark.parametrize("name", sorted(MULTI))
def test_multi_step_golden_on_cpu_oracle(name):
    run_multi(name, "cpu")


@pytest.mark.parametrize("name", sorted(EDGES))
def test_edge_values_golden_on_cpu_oracle(name):
    run_edges(name, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(MULTI))
def test_multi_step_golden_on_gpu(name):
    run_multi(name, GPU)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(EDGES))
def test_edge_values_golden_on_gpu(name):
    run_edges(name, GPU)


def one_step(kind, dtype, p, g, lr, eps, device):
    """ref: tests/optim.rs:256-268: one step from a single value."""
    param = h.full([32], p, dtype, device)
    grad = h.full([32], g, dtype, device)
    if kind == "sgd":
        out, _ = h.sgd_step(param, grad, None, lr=lr)
    else:
        out, _ = h.adam_step(param, grad, None, lr=lr, eps=eps, weight_decay=0.0 if kind == "adam" else 1e-2,
                             decoupled_weight_decay=kind == "adamw")
    return array(out.to(DT.F64))


def spelled_out(device):
    """ref: tests/optim.rs:269-290: products that overflow or vanish on their own, but not inside one rounding."""
    for kind in ("adam", "adamw"):
        p = one_step(kind, DT.F16, 0.0, 1e-5, 1e-3, 1e-4, device)
        assert (p == -0.00010132789611816406).all(), (kind, p)
    p = one_step("sgd", DT.F16, 60000.0, 2.0, 60000.0, 0.0, device)
    assert (p == -60000.0).all(), p
    for dtype in (DT.BF16, DT.F32):
        p = one_step("sgd", dtype, 3e38, 2.0, 3e38, 0.0, device)
        assert (np.isfinite(p) & (p < -2.9e38)).all(), (dtype, p)
    p = one_step("sgd", DT.F64, 1e308, 2.0, 1e308, 0.0, device)
    assert (p == -1e308).all(), p


def test_spelled_out_steps_on_cpu_oracle():
    spelled_out("cpu")


@pytest.mark.gpu
def test_spelled_out_steps_on_gpu():
    spelled_out(GPU)


def rejected(device):
    """ref: src/optim/mod.rs:681-695 and tests/optim.rs:297-330: a finite coefficient beyond its type is an error
    before anything is computed; infinities pass."""
    t = h.full([2], 1.0, DT.F16, device)
    with pytest.raises(Exception, match="value cannot be converted to type f16 without overflow"):
        h.scaled_add(t, t, 1e5)
    with pytest.raises(Exception, match="value cannot be converted to type f32 without overflow"):
        h.addcdiv_step(t, t, t, 1e39)
    inf16 = 0x7C00
    assert (bits(h.addcdiv_step(t, t, t, 1e5)) == inf16).all()  # in F32, the computation type of F16
    assert (bits(h.scaled_add(t, t, float("inf"))) == inf16).all()
    for dtype, big in ((DT.F16, 1e5), (DT.BF16, 1e40), (DT.F32, 1e40)):
        p = h.full([32], 1.0, dtype, device)
        for lr, wd in ((big, 0.0), (0.1, big)):
            with pytest.raises(Exception, match="without overflow"):
                h.sgd_step(p, p, None, lr=lr, weight_decay=wd, momentum=0.9)
    with pytest.raises(Exception, match="Nesterov momentum requires a momentum and zero dampening"):
        h.sgd_step(t, t, None, lr=0.1, nesterov=True)


def test_coefficients_that_overflow_are_rejected_on_cpu_oracle():
    rejected("cpu")


@pytest.mark.gpu
def test_coefficients_that_overflow_are_rejected_on_gpu():
    rejected(GPU)


def random_runs(seed, device_pair):
    """Three steps of SGD and of Adam / AdamW with options drawn from a seeded generator, on both devices: the
    parameter and the state after every step."""
    cpu, gpu = device_pair
    rng = np.random.default_rng(0x5EED6000 + seed)
    for case in range(12):
        dtype = [DT.F32, DT.BF16, DT.F16, DT.F64][int(rng.integers(0, 4))]
        shape = [int(rng.choice([1, 3, 17, 64, 1000, 4099]))] if rng.integers(0, 2) else [int(rng.choice([2, 5, 33])), int(rng.choice([7, 128, 513]))]
        n = int(np.prod(shape))
        p0 = from_f64(normal(100 * seed + case, n), dtype)
        grads = [from_f64(normal(100 * seed + case + 1 + s, n, 0.0, 0.3), dtype) for s in range(3)]
        lr = float(rng.choice([1e-3, 0.05, 0.5]))
        wd = float(rng.choice([0.0, 1e-2, 0.1]))
        maximize = bool(rng.integers(0, 2))
        if rng.integers(0, 2):
            momentum = float(rng.choice([0.0, 0.9, 0.5]))
            dampening = float(rng.choice([0.0, 0.1])) if momentum else 0.0
            nesterov = bool(momentum and dampening == 0.0 and rng.integers(0, 2))
            what = f"seed {seed} case {case}: sgd {dtype} {shape} lr {lr} wd {wd} momentum {momentum} dampening {dampening} nesterov {nesterov} maximize {maximize}"
            states = {d: None for d in (cpu, gpu)}
            params = {d: tensor(p0, dtype, shape, d) for d in (cpu, gpu)}
            for s in range(3):
                for d in (cpu, gpu):
                    params[d], states[d] = h.sgd_step(params[d], tensor(grads[s], dtype, shape, d), states[d], lr=lr, momentum=momentum,
                                                      dampening=dampening, weight_decay=wd, nesterov=nesterov, maximize=maximize)
                assert_bitwise(params[gpu], params[cpu], f"{what}: parameter after step {s}")
                if states[cpu] is not None:
                    assert_bitwise(states[gpu], states[cpu], f"{what}: momentum buffer after step {s}")
        else:
            decoupled, amsgrad = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
            beta1, beta2 = float(rng.choice([0.9, 0.5])), float(rng.choice([0.999, 0.9]))
            eps = float(rng.choice([1e-8, 1e-4]))
            what = f"seed {seed} case {case}: adam {dtype} {shape} lr {lr} wd {wd} betas {beta1}, {beta2} eps {eps} amsgrad {amsgrad} decoupled {decoupled} maximize {maximize}"
            states = {d: None for d in (cpu, gpu)}
            params = {d: tensor(p0, dtype, shape, d) for d in (cpu, gpu)}
            for s in range(3):
                for d in (cpu, gpu):
                    params[d], states[d] = h.adam_step(params[d], tensor(grads[s], dtype, shape, d), states[d], lr=lr, beta1=beta1, beta2=beta2,
                                                       eps=eps, weight_decay=wd, amsgrad=amsgrad, maximize=maximize,
                                                       decoupled_weight_decay=decoupled)
                assert_bitwise(params[gpu], params[cpu], f"{what}: parameter after step {s}")
                assert states[gpu][0] == states[cpu][0]
                for k in (1, 2, 3):
                    if states[cpu][k] is not None:
                        assert_bitwise(states[gpu][k], states[cpu][k], f"{what}: state {k} after step {s}")


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(6))
def test_random_optimizer_runs_match_the_cpu(seed):
    random_runs(seed, ("cpu", GPU))
