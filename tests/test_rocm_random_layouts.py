"""Randomly composed views through every kernel family on the GPU against the CPU oracle, bit for bit.

The layout tables of the other tests are fixed lists; the kernels, though, pick their variant from sizes, strides,
alignment and offsets (flat rows, rows with outer dimensions, tiles of two dimensions in both forms, lines, the general
kernel), and the edges between the variants are where a wrong choice would hide. Every case here is drawn from a seeded
generator, so a failure names the seed and the case and repeats: a base tensor with a random shape, a random chain of
view operations (permute, transpose, narrow, stepped slices, select, unsqueeze + expand, unfold), the same chain on the
CPU and on the GPU, and an operation whose result must have the CPU's bits (copy and conversion, unary and binary
arithmetic with a partner that is contiguous, broadcast, viewed the same way or of another dtype, scalar operands,
comparison, where, integer sums and extremes with their positions along every dimension, writes through the view)
or stay within its class (transcendental functions, float sums, means and variances, softmax). Further tests walk
the same chains through the families next to the path, through tensors of hundreds of megabytes, and with NaNs,
infinities, signed zeros and ties sprinkled into the data. What these tests found when they were written: a
log_softmax of 16-bit rows 21 ulp off where one element dominates, a NaN variance of a column clamped to 0, an
infinite mean merged into an infinite variance where the CPU has NaN, f64 column variances outside their class,
sigmoid and silu two to four ulps from the CPU for 1 input in 18 000, pow of a signaling NaN."""
import numpy as np
import pytest

from tests import oracle
from tests.support import DT, FLOATS, GPU, NP, array, assert_bitwise, check_within, from_f64, h, tensor, to_f64, values

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())

# Sizes that sit on, below and above the tile edges of the kernels (8, 16, 64, 128, 256) and a few odd ones.
SIZES = [1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 130, 200, 256, 257, 384]


# For a few cases of several million elements: more than one workgroup per row, tile, line and slice.
LARGE_SIZES = [2, 3, 8, 64, 128, 256, 257, 384, 512, 1000, 1024, 2048]


# Empty and one-element dimensions, for the seeds from 400 on: kernels that have nothing to do, reductions over nothing.
TINY_SIZES = [0, 0, 1, 1, 2, 3, 4, 5, 8, 17]


# Five to eight dimensions of a few elements each, for the seeds from 600 on: more dimensions than the row kernels
# walk, so the general kernels and the plans for many kept and reduced dimensions.
DEEP_SIZES = [1, 2, 2, 3, 3, 4, 5, 7]


def sizes_of(seed):
    if 600 <= seed < 700:
        return DEEP_SIZES
    return TINY_SIZES if 400 <= seed < 500 else (LARGE_SIZES if seed >= 100 else SIZES)


def random_shape(rng, limit, sizes=SIZES):
    ndim = int(rng.integers(5, 9)) if sizes is DEEP_SIZES else int(rng.integers(1, 5))
    while True:
        shape = [int(rng.choice(sizes)) for _ in range(ndim)]
        if int(np.prod(shape)) <= limit:
            return shape


def random_chain(rng, shape):
    """A list of (method, arguments) applicable in order to a tensor of `shape`, and the shape it ends with."""
    chain, shape = [], list(shape)
    for _ in range(int(rng.integers(0, 4))):
        nd = len(shape)
        kind = rng.choice(["permute", "transpose", "narrow", "slice", "select", "expand", "unfold"])
        if kind == "permute" and nd >= 2:
            perm = [int(p) for p in rng.permutation(nd)]
            chain.append(("permute", (perm,)))
            shape = [shape[p] for p in perm]
        elif kind == "transpose" and nd >= 2:
            a, b = (int(x) for x in rng.choice(nd, 2, replace=False))
            chain.append(("transpose", (a, b)))
            shape[a], shape[b] = shape[b], shape[a]
        elif kind == "narrow" and nd >= 1:
            d = int(rng.integers(0, nd))
            if shape[d] >= 2:
                start = int(rng.integers(0, shape[d] - 1))
                length = int(rng.integers(1, shape[d] - start + 1))
                chain.append(("narrow", (d, start, length)))
                shape[d] = length
        elif kind == "slice" and nd >= 1:
            d = int(rng.integers(0, nd))
            if shape[d] >= 3:
                start, step = int(rng.integers(0, 2)), int(rng.integers(2, 4))
                chain.append(("slice", (d, start, None, step)))
                shape[d] = len(range(start, shape[d], step))
        elif kind == "select" and nd >= 2:
            d = int(rng.integers(0, nd))
            if shape[d] > 0:
                chain.append(("select", (d, int(rng.integers(0, shape[d])))))
                del shape[d]
        elif kind == "expand" and nd <= 3:
            d = int(rng.integers(0, nd + 1))
            times = int(rng.choice([2, 3, 8, 64]))
            chain.append(("unsqueeze", (d,)))
            shape.insert(d, times)
            chain.append(("expand", (list(shape),)))
        elif kind == "unfold" and nd >= 1 and nd <= 3:
            d = int(rng.integers(0, nd))
            if shape[d] >= 4:
                size, step = int(rng.integers(2, 5)), int(rng.integers(1, 4))
                chain.append(("unfold", (d, size, step)))
                shape[d] = (shape[d] - size) // step + 1
                shape.append(size)
    return chain, shape


def apply(t, chain):
    for method, args in chain:
        t = getattr(t, method)(*args)
    return t


def pair(dtype, shape, seed):
    t = tensor(values(dtype, int(np.prod(shape)), seed), dtype, shape)
    return t, t.to(GPU)


def same_outcome(on_gpu, on_cpu, what, judge=None):
    """on_gpu() against on_cpu(): the same result (bit for bit, or as `judge` says) or the same refusal."""
    try:
        want = on_cpu()
    except Exception as refusal:
        with pytest.raises(type(refusal)) as got:
            on_gpu()
        assert str(got.value) == str(refusal), what
        return
    got = on_gpu()
    if isinstance(want, tuple):
        for i, (g, c) in enumerate(zip(got, want)):
            (judge or assert_bitwise)(g, c, f"{what} [{i}]")
    else:
        (judge or assert_bitwise)(got, want, what)


def overlapping(t):
    """Whether two indices of the view may be one element (expanded or unfolded): such a view cannot be written."""
    reach = 0
    for stride, size in sorted((s, n) for s, n in zip(t.strides, t.shape) if n > 1):
        if stride <= reach:
            return True
        reach += (size - 1) * stride
    return False


@pytest.mark.parametrize("seed", list(range(32)) + [100, 101, 102, 103, 400, 401, 402, 600, 601, 602])
def test_random_views_through_every_kernel_family(seed):
    rng = np.random.default_rng(0x5EED0000 + seed)
    dtypes = [DT.F32, DT.BF16, DT.I64, DT.U8, DT.F16, DT.I32, DT.F64, DT.Bool]
    large = seed >= 100
    for case in range(20 if large else 150):
        dtype = dtypes[int(rng.integers(0, len(dtypes)))]
        base_shape = random_shape(rng, 3000000 if large else 120000, sizes_of(seed))
        chain, shape = random_chain(rng, base_shape)
        what = f"seed {seed} case {case}: {dtype} {base_shape} {chain}"
        (c, g) = pair(dtype, base_shape, 1000 * seed + case)
        vc, vg = apply(c, chain), apply(g, chain)
        assert vg.shape == vc.shape and vg.strides == vc.strides and vg.offset == vc.offset, what
        assert_bitwise(vg.contiguous(), vc.contiguous(), f"{what}: copy")
        other = dtypes[int(rng.integers(0, len(dtypes)))]
        assert_bitwise(vg.to(other), vc.to(other), f"{what}: to {other}")
        # A partner: contiguous of the view's shape, viewed the same way, or broadcast along some dimensions.
        choice = int(rng.integers(0, 3))
        if choice == 0 or not shape:
            pc, pg = pair(dtype, shape, 77 + case)
        elif choice == 1:
            bc, bg = pair(dtype, base_shape, 78 + case)
            pc, pg = apply(bc, chain), apply(bg, chain)
        else:
            small = [n if rng.integers(0, 2) else 1 for n in shape]
            pc, pg = pair(dtype, small, 79 + case)
        if dtype == DT.Bool:
            assert_bitwise(vg.logical_and(pg), vc.logical_and(pc), f"{what}: and")
            assert_bitwise(vg.logical_not(), vc.logical_not(), f"{what}: not")
        else:
            assert_bitwise(vg.add(pg), vc.add(pc), f"{what}: + partner {choice}")
            assert_bitwise(pg.sub(vg), pc.sub(vc), f"{what}: partner {choice} -")
            assert_bitwise(vg.mul(3), vc.mul(3), f"{what}: * 3")
            assert_bitwise(vg.abs(), vc.abs(), f"{what}: abs")
            assert_bitwise(vg.greater(pg), vc.greater(pc), f"{what}: >")
            mask_c = vc.greater(pc)
            assert_bitwise(h.where_(mask_c.to(GPU), vg, pg), h.where_(mask_c, vc, pc), f"{what}: where")
        # One more binary op, one exact unary op and (floats) one transcendental, drawn from the whole lists.
        from tests.test_rocm_elementwise import COMPARE, IEEE_UNARY, ONE_ULP, ops_for

        name = str(rng.choice(ops_for(dtype) + COMPARE + ["logical_and", "logical_or"]))
        assert_bitwise(getattr(vg, name)(pg), getattr(vc, name)(pc), f"{what}: {name} with partner {choice}")
        name = str(rng.choice([u for u in IEEE_UNARY if not (dtype == DT.Bool and u in ("neg", "abs", "relu"))]))
        assert_bitwise(getattr(vg, name)(), getattr(vc, name)(), f"{what}: {name}")
        if dtype in (DT.F32, DT.BF16, DT.F16):
            # The ops built on the restated library functions have the CPU's bits.
            exact = ["exp", "log", "sin", "cos", "erf", "sigmoid", "silu", "gelu", "tanh", "gelu_tanh", "log_sigmoid"]
            name = str(rng.choice(sorted(set(ONE_ULP) | set(exact))))
            if name in exact:
                assert_bitwise(getattr(vg, name)(), getattr(vc, name)(), f"{what}: {name}")
            else:
                check_within(getattr(vg, name)(), getattr(vc, name)(), extra=0.0, max_ulp=1, what=f"{what}: {name}")
        # A partner of another dtype: the result type and the converted operands must be the CPU's.
        if shape:
            qc, qg = pair(other, shape, 90 + case)
            name = str(rng.choice(["add", "mul", "sub", "maximum", "greater", "equal", "div"]))   # div of integers is true division
            try:
                want = getattr(vc, name)(qc)
            except Exception as refusal:            # e.g. bool - bool: the GPU must refuse in the same words
                with pytest.raises(type(refusal)) as got:
                    getattr(vg, name)(qg)
                assert str(got.value) == str(refusal), f"{what}: {name} with a {other} partner"
            else:
                assert_bitwise(getattr(vg, name)(qg), want, f"{what}: {name} with a {other} partner")
        # A scalar operand: the scalar's kind and the tensor's dtype decide the result type (ref: src/ops/binary.rs).
        scalar = [3, -2, 2.5, 0.1, 1e20, -0.0, 255, 65536, True, float("inf")][int(rng.integers(0, 10))]
        name = str(rng.choice(["add", "mul", "sub", "div", "maximum", "greater", "equal", "pow"]))
        try:
            want = getattr(vc, name)(scalar)
        except Exception as refusal:
            with pytest.raises(type(refusal)) as got:
                getattr(vg, name)(scalar)
            assert str(got.value) == str(refusal), f"{what}: {name} {scalar!r}"
        else:
            if name == "pow" and want.dtype == DT.F64:     # the one pow that is not the host library's restated
                check_within(getattr(vg, name)(scalar), want, extra=0.0, max_ulp=1, what=f"{what}: pow {scalar!r}")
            else:
                assert_bitwise(getattr(vg, name)(scalar), want, f"{what}: {name} {scalar!r}")
        if dtype in (DT.I64, DT.I32, DT.U8) and shape:
            d = int(rng.integers(0, len(shape)))
            assert_bitwise(vg.sum_dim([d], False), vc.sum_dim([d], False), f"{what}: sum along {d}")
            if shape[d] > 0:
                (gv, gi), (cv, ci) = vg.max_dim(d, False), vc.max_dim(d, False)
                assert_bitwise(gv, cv, f"{what}: max along {d}")
                assert_bitwise(gi, ci, f"{what}: positions of the max along {d}")
        if dtype in (DT.F32, DT.BF16) and shape and shape[-1] > 0:
            (gv, gi), (cv, ci) = vg.min_dim(-1, True), vc.min_dim(-1, True)
            assert_bitwise(gv, cv, f"{what}: min along the last dimension")
            assert_bitwise(gi, ci, f"{what}: positions of the min")
        # Writing through the view (when its elements are distinct): the whole base must agree afterwards.
        if not overlapping(vc) and dtype != DT.Bool:
            sc, sg = pair(dtype, shape, 80 + case)
            vc.copy_(sc)
            vg.copy_(sg)
            assert_bitwise(g, c, f"{what}: written through the view")
            vc.add_(pc)
            vg.add_(pg)
            assert_bitwise(g, c, f"{what}: updated through the view")


def f64_of(t):
    """The elements of t, in order, as float64."""
    return to_f64(array(t).reshape(-1), t.dtype)


def sprinkle(rng, t, dtype, shape):
    """A few NaNs, infinities of both signs and zeros at random places of t: some lines get one, most stay clean."""
    flat = f64_of(t).copy()
    count = max(1, flat.size // 200)
    where = rng.integers(0, flat.size, count)
    flat[where] = rng.choice([np.nan, np.inf, -np.inf, 0.0, -0.0], count)
    return tensor(from_f64(flat, dtype), dtype, shape)


@pytest.mark.parametrize("seed", list(range(12)) + [200, 201, 400, 401, 402, 600, 601, 602])
def test_random_views_through_float_reductions_and_softmax(seed):
    """The reduction and softmax plans pick their kernels from the merged kept and reduced dimensions of the view
    (rows, columns, slices cut across workgroups, the general walk): the same random chains of views as above, float
    data, and the classes of tests/test_rocm_reduce.py as the bar (sums and means within 2 n eps of the sum of
    magnitudes, variances within 4 n eps v, softmax within its row's class; extremes and their positions bit for bit)."""
    from tests.test_rocm_reduce import EPS, check_softmax, check_sum, f64, finite, folded

    rng = np.random.default_rng(0x5EED1000 + seed)
    large = seed >= 200
    for case in range(12 if large else 60):
        dtype = FLOATS[int(rng.integers(0, len(FLOATS)))]
        base_shape = random_shape(rng, 3000000 if large else 60000, sizes_of(seed))
        chain, shape = random_chain(rng, base_shape)
        if not shape:
            continue
        what = f"seed {seed} case {case}: {dtype} {base_shape} {chain}"
        n = int(np.prod(base_shape))
        c = finite(dtype, n, 12 if dtype == DT.F16 else 30, 5000 * seed + case).reshape(base_shape)
        sprinkled = case % 3 == 2 and n > 0
        if sprinkled:
            c = sprinkle(rng, c, dtype, base_shape)
        g = c.to(GPU)
        vc, vg = apply(c, chain), apply(g, chain)
        nd = len(shape)
        dims = sorted(int(d) for d in rng.choice(nd, int(rng.integers(1, nd + 1)), replace=False))
        keep = bool(rng.integers(0, 2))
        if 0 in shape:
            # Nothing to fold: sums of nothing are 0, means and variances NaN, extremes refuse, softmax is empty or
            # all NaN; whatever the CPU does, in its words.
            d, correction = int(rng.integers(0, nd)), int(rng.integers(0, 2))
            exact = lambda got, want, label: check_within(got, want, extra=0.0, max_ulp=0, what=label)
            for label, f in (("sum", lambda t: t.sum_dim(dims, keep)), ("mean", lambda t: t.mean_dim(dims, keep)),
                             ("var", lambda t: t.var_dim(dims, correction, keep)), ("std", lambda t: t.std_dim(dims, correction, keep)),
                             ("max_dim", lambda t: t.max_dim(d, keep)), ("argmin_dim", lambda t: t.argmin_dim(d, keep)),
                             ("softmax", lambda t: t.softmax(d)), ("log_softmax", lambda t: t.log_softmax(d)),
                             ("sum of all", lambda t: t.sum()), ("max of all", lambda t: t.max())):
                same_outcome(lambda: f(vg), lambda: f(vc), f"{what}: {label} over {dims} / along {d} of an empty view", exact)
            continue
        wide = vc.to(DT.F64)
        want = vc.sum_dim(dims, keep)
        count = folded(vc, want)
        abs_sum = wide.abs().sum_dim(dims, keep)
        check_sum(vg.sum_dim(dims, keep), want, abs_sum, count, False, f"{what}: sum over {dims}")
        check_sum(vg.mean_dim(dims, keep), vc.mean_dim(dims, keep), abs_sum, count, True, f"{what}: mean over {dims}")
        correction = int(rng.integers(0, 2))
        v = f64(wide.var_dim(dims, correction, keep))
        # The class of the reduce tests, 4 n eps v, plus what the rounding of the mean alone can move a variance by,
        # (n eps)^2 times the mean square: nothing next to the class unless the reduced elements are all but equal
        # (an expanded dimension reduced: v is 0 exactly and the CPU's own result is that rounding).
        mean_square = f64(wide.mul(wide).mean_dim(dims, keep))
        with np.errstate(all="ignore"):
            delta = np.nan_to_num(4.0 * count * EPS * v + 4.0 * (count * EPS) ** 2 * mean_square, nan=0.0, posinf=0.0)
        check_within(vg.var_dim(dims, correction, keep), vc.var_dim(dims, correction, keep), extra=delta,
                     what=f"{what}: var over {dims} correction {correction}")
        d = int(rng.integers(0, nd))
        same_outcome(lambda: vg.max_dim(d, keep), lambda: vc.max_dim(d, keep), f"{what}: max along {d} and its positions")
        if case % 3 == 1:
            # Ties, signed zeros and NaNs from a five-letter alphabet: the CPU keeps the first of equal values and the
            # first NaN, and the GPU's value and position must be that one (ref: src/backend/cpu/reduce.rs:75-86).
            letters = rng.choice([-1.0, 0.0, -0.0, 1.0, np.nan], n, p=[0.3, 0.2, 0.2, 0.28, 0.02])
            tc = tensor(from_f64(letters, dtype), dtype, base_shape)
            tvc, tvg = apply(tc, chain), apply(tc.to(GPU), chain)
            for best in ("max_dim", "min_dim"):
                same_outcome(lambda: getattr(tvg, best)(d, keep), lambda: getattr(tvc, best)(d, keep),
                             f"{what}: {best} of tied values along {d} and its positions")
            same_outcome(lambda: tvg.argmax(), lambda: tvc.argmax(), f"{what}: argmax of tied values")
            same_outcome(lambda: tvg.min(), lambda: tvc.min(), f"{what}: min of tied values")
        # Softmax on data of a few binades, as the reduce tests use (larger spreads make every row one-hot).
        sc = finite(dtype, n, 3, 7000 * seed + case).reshape(base_shape)
        if sprinkled:
            sc = sprinkle(rng, sc, dtype, base_shape)
        sg = sc.to(GPU)
        svc, svg = apply(sc, chain), apply(sg, chain)
        log = bool(rng.integers(0, 2))
        want = svc.log_softmax(d) if log else svc.softmax(d)
        got = svg.log_softmax(d) if log else svg.softmax(d)
        check_softmax(got, want, svc.to(DT.F64), d, log, f"{what}: {'log_' if log else ''}softmax along {d}")


def positions(rng, count, below, dtype, shape):
    picks = rng.integers(0, below, count).astype(np.int64 if dtype == DT.I64 else np.int32)
    return tensor(picks, dtype, shape)


@pytest.mark.parametrize("seed", list(range(16)) + [300, 301, 400, 401, 402, 600, 601, 602])
def test_random_views_through_the_families_next_to_the_path(seed):
    """flip, triu / tril, the fused optimizer steps, addr, exclusive_cumprod, masked_fill and the index family
    (index_select, gather, scatter_add, index_add) take their operands as views too, and each picks its kernel from
    the layout it finds (tiles of rows, lines staged in LDS, the element-wise walk): the same random chains of views,
    and the CPU's bits."""
    rng = np.random.default_rng(0x5EED2000 + seed)
    every = [DT.F32, DT.BF16, DT.I64, DT.U8, DT.F16, DT.I32, DT.F64, DT.Bool, DT.I8, DT.I16]
    large = seed >= 300
    for case in range(10 if large else 80):
        dtype = every[int(rng.integers(0, len(every)))]
        base_shape = random_shape(rng, 2000000 if large else 50000, sizes_of(seed))
        chain, shape = random_chain(rng, base_shape)
        if not shape:
            continue
        what = f"seed {seed} case {case}: {dtype} {base_shape} {chain}"
        (c, g) = pair(dtype, base_shape, 3000 * seed + case)
        vc, vg = apply(c, chain), apply(g, chain)
        nd = len(shape)
        d = int(rng.integers(0, nd))
        dims = sorted(int(x) for x in rng.choice(nd, int(rng.integers(1, nd + 1)), replace=False))
        assert_bitwise(vg.flip(dims), vc.flip(dims), f"{what}: flip {dims}")
        if nd >= 2:
            k = int(rng.integers(-3, 4))
            assert_bitwise(vg.triu(k), vc.triu(k), f"{what}: triu {k}")
            assert_bitwise(vg.tril(k), vc.tril(k), f"{what}: tril {k}")
        pc, pg = pair(dtype, shape, 81 + case)
        mask_c = pc.greater(vc) if dtype != DT.Bool else pc
        fill = True if dtype == DT.Bool else 3
        assert_bitwise(vg.masked_fill(mask_c.to(GPU), fill), vc.masked_fill(mask_c, fill), f"{what}: masked_fill")
        # clamp with scalar bounds, full and fill_ with scalars of every kind: the same result or the same refusal.
        def same(f_gpu, f_cpu, label):
            try:
                want = f_cpu()
            except Exception as refusal:
                with pytest.raises(type(refusal)) as got:
                    f_gpu()
                assert str(got.value) == str(refusal), f"{what}: {label}"
            else:
                assert_bitwise(f_gpu(), want, f"{what}: {label}")

        if dtype != DT.Bool:
            lo, hi = (float(x) for x in rng.choice([-100.0, -1.0, 0.0, 0.5, 3.0, 100.0], 2))
            if dtype not in FLOATS:
                lo, hi = int(lo), int(hi)
            same(lambda: vg.clamp(lo, hi), lambda: vc.clamp(lo, hi), f"clamp({lo}, {hi})")
            same(lambda: vg.clamp_min(lo), lambda: vc.clamp_min(lo), f"clamp_min({lo})")
            same(lambda: vg.clamp_max(hi), lambda: vc.clamp_max(hi), f"clamp_max({hi})")
        scalar = [0, 1, -1, 3, 255, 256, -129, 70000, 2.5, -0.0, 1e20, 1e-50, float("inf"), float("nan"), True][int(rng.integers(0, 15))]
        same(lambda: h.full(list(shape), scalar, dtype, GPU), lambda: h.full(list(shape), scalar, dtype, "cpu"), f"full {scalar!r}")
        if not overlapping(vc):
            fc, fg = pair(dtype, base_shape, 3000 * seed + case)
            same(lambda: (apply(fg, chain).fill_(scalar), fg)[1], lambda: (apply(fc, chain).fill_(scalar), fc)[1], f"fill_ {scalar!r} through the view")
        # The index family along d.
        if shape[d] == 0:
            continue     # no position to draw
        itype = DT.I64 if rng.integers(0, 2) else DT.I32
        count = int(rng.integers(1, 2 * shape[d] + 2))
        idx = positions(rng, count, shape[d], itype, [count])
        assert_bitwise(vg.index_select(d, idx.to(GPU)), vc.index_select(d, idx), f"{what}: index_select along {d}")
        sshape = list(shape)
        sshape[d] = count
        sc, sg = pair(dtype, sshape, 82 + case)
        assert_bitwise(vg.index_add(d, idx.to(GPU), sg), vc.index_add(d, idx, sc), f"{what}: index_add along {d}")
        ishape = [max(min(1, n), n - int(rng.integers(0, 2))) for n in shape]
        ishape[d] = count
        picks = positions(rng, int(np.prod(ishape)), shape[d], itype, ishape)
        assert_bitwise(vg.gather(d, picks.to(GPU)), vc.gather(d, picks), f"{what}: gather along {d}")
        assert_bitwise(vg.scatter_add(d, picks.to(GPU), sg), vc.scatter_add(d, picks, sc), f"{what}: scatter_add along {d}")
        if dtype in FLOATS:
            qc, qg = pair(dtype, shape, 83 + case)
            v = float(rng.choice([0.3, -0.7, 1.0 / 3.0, 2.0]))
            assert_bitwise(h.scaled_add(vg, pg, v), h.scaled_add(vc, pc, v), f"{what}: scaled_add {v}")
            assert_bitwise(h.lerp_step(vg, pg, v), h.lerp_step(vc, pc, v), f"{what}: lerp step {v}")
            assert_bitwise(h.addcmul_step(vg, pg, qg, v), h.addcmul_step(vc, pc, qc, v), f"{what}: addcmul step {v}")
            assert_bitwise(h.addcdiv_step(pg, qg, vg, v), h.addcdiv_step(pc, qc, vc, v), f"{what}: addcdiv step {v}")
            reverse = bool(rng.integers(0, 2))
            assert_bitwise(h.exclusive_cumprod(vg, d, reverse), h.exclusive_cumprod(vc, d, reverse),
                           f"{what}: exclusive_cumprod along {d} reverse {reverse}")
        if nd == 2 and dtype != DT.Bool:
            (ac, ag), (bc, bg) = pair(dtype, [shape[0]], 84 + case), pair(dtype, [shape[1]], 85 + case)
            beta, alpha = (0.5, -1.5) if dtype in FLOATS else (2, -3)
            assert_bitwise(vg.addr(ag, bg, beta, alpha), vc.addr(ac, bc, beta, alpha), f"{what}: addr")


@pytest.mark.parametrize("seed", range(6))
def test_random_views_of_large_tensors_agree_with_the_cpu_on_windows(seed):
    """Hundreds of megabytes: the sizes at which the kernels change their cache hints and their store forms. The
    operands are sampled on the GPU, the operation runs on the whole view, and windows of the result (a few rows of
    its first dimension) are compared with the CPU's result on the same windows of the operands: an element-wise
    operation on a window is the window of the operation."""
    rng = np.random.default_rng(0x5EED5000 + seed)
    bases = {DT.I64: [[8, 2048, 4096], [4, 4096, 32, 128]], DT.F32: [[12, 2048, 4096], [96, 1024, 1024]],
             DT.BF16: [[8192, 32000], [16, 2048, 32, 128], [8, 2048, 4096]], DT.U8: [[16384, 32768], [8, 4096, 128, 128]]}
    dtype = list(bases)[seed % 4]
    base_shape = bases[dtype][int(rng.integers(0, len(bases[dtype])))]
    while True:
        chain, shape = random_chain(rng, base_shape)
        if all(m not in ("expand", "unfold", "select") for m, _ in chain) and int(np.prod(shape)) >= int(np.prod(base_shape)) // 4:
            break
    what = f"seed {seed}: {dtype} {base_shape} {chain}"
    h.manual_seed(1234 + seed)
    if dtype in (DT.F32, DT.BF16):
        a, b = h.uniform(base_shape, -4.0, 4.0, dtype, GPU), h.uniform(base_shape, -4.0, 4.0, dtype, GPU)
    else:
        a, b = h.randint(0, 200, base_shape, dtype, GPU), h.randint(0, 200, base_shape, dtype, GPU)
    va, vb = apply(a, chain), apply(b, chain)
    ops = [("add", lambda x, y: x.add(y)), ("greater", lambda x, y: x.greater(y)), ("copy", lambda x, y: x.contiguous()),
           ("mul by 3", lambda x, y: x.mul(3)), ("where", lambda x, y: h.where_(x.greater(y), x, y))]
    if dtype == DT.BF16:
        ops += [("silu", lambda x, y: x.silu()), ("add an f32 partner", lambda x, y: x.add(y.to(DT.F32)))]
    if dtype == DT.I64:
        ops += [("bitwise_and", lambda x, y: x.bitwise_and(y))]
    rows = shape[0]
    for name, f in ops:
        whole = f(va, vb)
        for _ in range(3):
            k = max(1, min(rows, (1 << 21) // max(1, int(np.prod(shape[1:])))))
            start = int(rng.integers(0, rows - k + 1))
            wa, wb = va.narrow(0, start, k).contiguous().to("cpu"), vb.narrow(0, start, k).contiguous().to("cpu")
            assert_bitwise(whole.narrow(0, start, k).contiguous(), f(wa, wb), f"{what}: {name}, rows {start}..{start + k}")
        del whole
    if dtype in (DT.I64, DT.U8) and len(shape) >= 2:
        whole = va.sum_dim([len(shape) - 1], False)
        k = max(1, min(rows, (1 << 21) // max(1, int(np.prod(shape[1:])))))
        start = int(rng.integers(0, rows - k + 1))
        wa = va.narrow(0, start, k).contiguous().to("cpu")
        assert_bitwise(whole.narrow(0, start, k).contiguous(), wa.sum_dim([len(shape) - 1], False), f"{what}: sum along the last dimension")
    if dtype in (DT.F32, DT.BF16) and len(shape) >= 2:
        from tests.test_rocm_reduce import check_softmax, check_sum, folded
        last = len(shape) - 1
        k = max(1, min(rows, (1 << 21) // max(1, int(np.prod(shape[1:])))))
        start = int(rng.integers(0, rows - k + 1))
        wa = va.narrow(0, start, k).contiguous().to("cpu")
        wide = wa.to(DT.F64)
        for log in (False, True):
            whole = va.log_softmax(last) if log else va.softmax(last)
            want = wa.log_softmax(last) if log else wa.softmax(last)
            check_softmax(whole.narrow(0, start, k).contiguous(), want, wide, last, log, f"{what}: softmax along the last dimension, log {log}")
            del whole
        whole = va.sum_dim([last], False)
        want = wa.sum_dim([last], False)
        check_sum(whole.narrow(0, start, k).contiguous(), want, wide.abs().sum_dim([last], False), folded(wa, want), False,
                  f"{what}: sum along the last dimension")
        whole = va.var_dim([last], 1, False)
        v64 = np.nan_to_num(f64_of(wide.var_dim([last], 1, False)))
        from tests.test_rocm_reduce import EPS
        check_within(whole.narrow(0, start, k).contiguous(), wa.var_dim([last], 1, False), extra=4.0 * shape[last] * EPS * v64,
                     what=f"{what}: var along the last dimension")
    del a, b, va, vb
    h.empty_cache()
