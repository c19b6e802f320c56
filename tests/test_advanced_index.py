"""Advanced indexing (index tensors and bool masks, reading and index_put) through the host front end.

On the CPU the oracle is plugged in as the CPU backend and pinned three ways: PyTorch's outputs for the
`index.tensor*` cases of the reference's fixture (tests/golden/ops.safetensors), the known answers of the
reference's own unit tests (ref: src/ops/advanced_index.rs:442-518, tests/rocm_index.rs:395-404), and numpy,
whose advanced indexing follows the same rules (masks become their nonzero coordinates, the indices broadcast,
the indexed dimensions move to the front when they are not adjacent, the last of repeated positions wins an
assignment, np.add.at adds in order). On the GPU the same calls are compared with the CPU's results
(ref: tests/rocm_index.rs:280-450).
"""
import numpy as np
import pytest

from tests import oracle
from tests.support import DT, DTYPES, GPU, NP, array, assert_bitwise, assert_same, h, load_golden, tensor, values, words

h.register_cpu_backend(oracle.backend_address())
GOLDEN = load_golden()


def ints(v, dtype=DT.I64):
    a = np.asarray(v, dtype=np.int64)
    return tensor(a.astype(NP[dtype]), dtype, list(a.shape))


def bools(a):
    a = np.asarray(a, dtype=bool)
    return tensor(a.astype(np.uint8), DT.Bool, list(a.shape))


def mask(shape, seed):
    """ref: tests/rocm_index.rs:284-290: two of three elements are true."""
    return (words(seed, int(np.prod(shape))) % np.uint64(3) != 0).reshape(shape)


def same(a, b):
    """Same shape and bytes (NaNs included)."""
    return list(a.shape) == list(b.shape) and np.ascontiguousarray(a).tobytes() == np.ascontiguousarray(b).tobytes()


def golden(case, device):
    t = {name: tensor(arr, dtype, list(arr.shape), device) for name, (arr, dtype) in GOLDEN[case].items()}
    return t, GOLDEN[case]["out"]


@pytest.mark.parametrize("device", ["cpu", pytest.param(GPU, marks=pytest.mark.gpu)])
def test_the_reference_golden_cases(device):
    """ref: tests/golden_ops.rs:256-258"""
    t, (want, dtype) = golden("index.tensor", device)
    got = t["x"].index_tensors([t["idx"]])
    assert got.shape == list(want.shape) and np.array_equal(array(got), want)
    t, (want, dtype) = golden("index.tensor_2d", device)
    got = t["x"].index_tensors([None, t["idx"]])
    assert got.shape == list(want.shape) and np.array_equal(array(got), want)
    t, (want, dtype) = golden("index.tensor_after_select", device)
    got = t["x"].select(0, 1).index_tensors([None, t["idx"]])
    assert got.shape == list(want.shape) and np.array_equal(array(got), want)


def test_known_answers_of_the_reference():
    # ref: src/ops/advanced_index.rs:504-512
    x = tensor(np.arange(12, dtype=np.int64), DT.I64, [3, 4])
    y = x.index_tensors([ints([[-1], [0]]), ints([3, -4, 1])])
    assert y.shape == [2, 3] and array(y).reshape(-1).tolist() == [11, 8, 9, 3, 0, 1]
    # ref: src/ops/advanced_index.rs:452-476: indexed dimensions 0 and 2 move to the front; the result sees the
    # work copy in the original order.
    x = tensor(np.zeros(24, dtype=np.float32), DT.F32, [2, 3, 4])
    v = tensor(np.arange(6, dtype=np.float32), DT.F32, [2, 3])
    for accumulate in (False, True):
        y = x.index_put_tensors([ints([0, 1]), None, ints([1, 2])], v, accumulate)
        assert y.shape == [2, 3, 4] and y.strides == [12, 1, 3] and not y.is_contiguous()
        want = np.zeros((2, 3, 4), dtype=np.float32)
        for n, (i, j) in enumerate([(0, 1), (1, 2)]):
            for k in range(3):
                want[i, k, j] = n * 3 + k
        assert np.array_equal(array(y), want)
    # ref: src/ops/advanced_index.rs:478-501: a transposed slice with an offset.
    base = tensor(np.arange(30, dtype=np.float32), DT.F32, [5, 6])
    x = base.narrow(0, 1, 3).transpose(0, 1)
    picked = x.index_tensors([None, ints([2, 0])])
    xs = np.arange(30, dtype=np.float32).reshape(5, 6)[1:4].T
    assert picked.shape == [6, 2] and np.array_equal(array(picked), xs[:, [2, 0]])
    y = x.index_put_tensors([None, ints([2, 0])], tensor(np.full(12, -1, dtype=np.float32), DT.F32, [6, 2]), False)
    want = xs.copy()
    want[:, [2, 0]] = -1
    assert np.array_equal(array(y), want) and np.array_equal(array(base).reshape(-1), np.arange(30, dtype=np.float32))
    # ref: tests/rocm_index.rs:395-404: the last of repeated positions wins.
    x = tensor(np.arange(10, dtype=np.float32), DT.F32, [10])
    y = x.index_put_tensors([ints([3, 3, 7])], tensor(np.array([1, 2, 3], dtype=np.float32), DT.F32, [3]), False)
    assert array(y).tolist() == [0.0, 1.0, 2.0, 2.0, 4.0, 5.0, 6.0, 3.0, 8.0, 9.0]


def cases():
    """Index expressions over a [5, 6, 7] target as (name, views before indexing, indices, the numpy key)
    (ref: tests/rocm_index.rs:280-317)."""
    m56, m67 = mask([5, 6], 1), mask([6, 7], 2)
    transposed = np.array([0, 1, 2, 3, 4, 0]).reshape(2, 3).T
    return [
        ("one index with repeats and negatives", None, [np.array([4, -1, 0, -5, 2, 4])], lambda i: (i[0],)),
        ("two broadcast indices", None, [np.array([[1], [-2]]), np.array([0, 5, -6])], lambda i: (i[0], i[1])),
        ("non-adjacent", None, [np.array([3, 1]), None, np.array([6, -7])], lambda i: (i[0], slice(None), i[2])),
        ("after a slice", (0, 1, 3), [None, np.array([5, 0, 5])], lambda i: (slice(None), i[1])),
        ("mask over two dimensions", None, [m56], lambda i: (i[0],)),
        ("mask then index", None, [None, m67], lambda i: (slice(None), i[1])),
        ("transposed index", None, [transposed], lambda i: (i[0],)),
        ("mask and index, not adjacent", None, [mask([5], 3), None, np.array([[2], [0]])], lambda i: (i[0], slice(None), i[2])),
        ("empty index", None, [np.zeros([0], dtype=np.int64)], lambda i: (i[0],)),
    ]


def as_index(a, device, dtype=DT.I64):
    if a is None:
        return None
    if a.dtype == bool:
        return bools(a).to(device)
    if a is not None and a.ndim == 2 and a.shape == (3, 2) and not a.flags["C_CONTIGUOUS"]:
        return ints(np.ascontiguousarray(a.T), dtype).transpose(0, 1).to(device)
    return ints(a, dtype).to(device)


def test_reading_follows_numpy():
    for s, dtype in enumerate([DT.F32, DT.I64, DT.BF16, DT.Bool]):
        x = values(dtype, 5 * 6 * 7, 500 + s).reshape(5, 6, 7)
        t = tensor(x, dtype, [5, 6, 7])
        for name, cut, indices, key in cases():
            xs, ts = (x, t) if cut is None else (x[cut[1]:cut[1] + cut[2]], t.narrow(*cut))
            want = xs[key(indices)]
            for index_dtype in (DT.I64, DT.I32):
                got = ts.index_tensors([as_index(i, "cpu", index_dtype) for i in indices])
                assert got.shape == list(want.shape), name
                assert same(array(got), want), (name, dtype)


def test_writing_follows_numpy():
    for s, dtype in enumerate([DT.F32, DT.I32, DT.F64, DT.I64]):
        x = values(dtype, 5 * 6 * 7, 600 + s).reshape(5, 6, 7)
        t = tensor(x, dtype, [5, 6, 7])
        for name, cut, indices, key in cases():
            if cut is not None:
                continue
            k = key(indices)
            shape = x[k].shape
            # Small integers: sums are exact in every dtype, so numpy's running sums in the dtype agree.
            v = (words(700 + s, int(np.prod(shape))) % np.uint64(5)).astype(np.float64).astype(x.dtype).reshape(shape)
            idx = [as_index(i, "cpu") for i in indices]
            put = t.index_put_tensors(idx, tensor(v, dtype, list(shape)), False)
            want = x.copy()
            want[k] = v
            assert put.shape == [5, 6, 7] and same(array(put), want), (name, dtype)
            small = (words(800 + s, x.size) % np.uint64(7)).astype(np.float64).astype(x.dtype).reshape(x.shape)
            ts = tensor(small, dtype, [5, 6, 7])
            added = ts.index_put_tensors(idx, tensor(v, dtype, list(shape)), True)
            want = small.copy()
            np.add.at(want, k, v)
            assert np.array_equal(array(added), want), (name, dtype)
            if v.size:
                one = ts.index_put_tensors(idx, tensor(v.reshape(-1)[:1], dtype, []), False)
                want = small.copy()
                want[k] = v.reshape(-1)[0]
                assert np.array_equal(array(one), want), (name, dtype)


def test_mask_coordinates_are_numpys_nonzero():
    for shape, seed in [([7], 1), ([5, 6], 2), ([3, 4, 5], 3), ([2, 1, 3, 2], 4), ([0, 3], 5), ([70, 90], 6)]:
        m = mask(shape, seed)
        coords = bools(m).mask_coordinates()
        want = np.nonzero(m)
        assert len(coords) == len(shape)
        for got, w in zip(coords, want):
            assert got.dtype == DT.I64 and array(got).tolist() == w.tolist()
    # Through a layout: the coordinates are those of the view.
    m = mask([6, 5], 7)
    coords = bools(m).transpose(0, 1).mask_coordinates()
    for got, w in zip(coords, np.nonzero(m.T)):
        assert array(got).tolist() == w.tolist()


def test_errors_are_the_references():
    x = tensor(np.arange(24, dtype=np.float32), DT.F32, [2, 3, 4])

    def message(f):
        with pytest.raises(h.HomuraError) as e:
            f()
        return str(e.value)

    assert message(lambda: x.index_tensors([ints([0, 2])])) == "index 2 is out of bounds for dimension 0 with size 2"
    assert message(lambda: x.index_tensors([ints([0]), ints([1, -4])])) == "index -4 is out of bounds for dimension 1 with size 3"
    # The indices are checked in order, each in row-major order.
    assert message(lambda: x.index_tensors([ints([0, 5, 7]), ints([9, 1, 1])])) == "index 5 is out of bounds for dimension 0 with size 2"
    # Non-adjacent indices are numbered in the working order (the indexed dimensions first).
    assert message(lambda: x.index_tensors([ints([0]), None, ints([4])])) == "index 4 is out of bounds for dimension 1 with size 4"
    assert "must be i64, i32 or bool tensors, got u8; use a bool tensor for a mask" in message(
        lambda: x.index_tensors([tensor(np.zeros(2, dtype=np.uint8), DT.U8, [2])]))
    assert message(lambda: x.index_tensors([ints([0]), ints([0]), ints([0]), ints([0])])) == "too many indices for tensor of dimension 3 (got 4)"
    assert message(lambda: x.index_tensors([bools(np.ones((2, 2), dtype=bool))])) == (
        "The shape of the mask [2, 2] at index 1 does not match the shape of the indexed tensor [2, 3, 4] at index 1")
    assert message(lambda: x.index_tensors([ints([0, 1]), ints([0, 1, 2])])) == (
        "shape mismatch: indexing tensors could not be broadcast together with shapes [2], [3]")
    assert message(lambda: x.index_tensors([None, None])) == "advanced indexing needs at least one index tensor"
    assert message(lambda: x.index_put_tensors([ints([0])], tensor(np.zeros(5, dtype=np.float32), DT.F32, [5]), False)) == (
        "shape mismatch: value tensor of shape [5] cannot be broadcast to indexing result of shape [1, 3, 4]")
    assert message(lambda: x.index_put_tensors([ints([0])], tensor(np.zeros(4, dtype=np.int32), DT.I32, [4]), False)) == (
        "Index put requires the source and destination dtypes match, got f32 for the destination and i32 for the source.")
    empty = tensor(np.zeros(0, dtype=np.float32), DT.F32, [0, 3])
    assert message(lambda: empty.index_tensors([ints([0])])) == "index is out of bounds for dimension with size 0"
    # Checked even when the result is empty.
    assert message(lambda: x.index_tensors([ints([5]), None, ints(np.zeros([0], dtype=np.int64))])) == (
        "index 5 is out of bounds for dimension 0 with size 2")


# ---- the GPU against the CPU --------------------------------------------------------------------------------------


def operand_layouts(dtype, shape, seed):
    n = int(np.prod(shape))
    rev, perm = list(reversed(shape)), list(reversed(range(len(shape))))
    base = tensor(values(dtype, n, seed), dtype)
    wide = tensor(values(dtype, 2 * n + 3, seed + 1), dtype)
    views = [("contiguous", lambda b, w: b.reshape(shape)), ("permuted", lambda b, w: b.reshape(rev).permute(perm)),
             ("strided", lambda b, w: w.narrow(0, 3, 2 * n).reshape([n, 2]).select(1, 1).reshape(shape))]
    bg, wg = base.to(GPU), wide.to(GPU)
    return [(name, f(base, wide), f(bg, wg)) for name, f in views]


def placed(indices, device, mixed):
    """Every index tensor on `device`, or alternately on the GPU and on the CPU (ref: rocm_index.rs:319-337)."""
    out, k = [], 0
    for i in indices:
        if i is None:
            out.append(None)
            continue
        k += 1
        out.append(as_index(i, "cpu" if mixed and k % 2 == 0 else device))
    return out


@pytest.mark.gpu
def test_advanced_indexing_matches_the_cpu():
    for s, dtype in enumerate(DTYPES):
        for sname, cpu, gpu in operand_layouts(dtype, [5, 6, 7], 500 + s):
            for name, cut, indices, _ in cases():
                c, g = (cpu, gpu) if cut is None else (cpu.narrow(*cut), gpu.narrow(*cut))
                want = c.index_tensors([as_index(i, "cpu") for i in indices])
                for where, device, mixed in [("GPU indices", GPU, False), ("CPU indices", "cpu", False), ("mixed", GPU, True)]:
                    got = g.index_tensors(placed(indices, device, mixed))
                    assert_same(got, want, f"{dtype} {sname} {name}, {where}")


@pytest.mark.gpu
def test_index_put_matches_the_cpu():
    for s, dtype in enumerate(DTYPES):
        for sname, cpu, gpu in operand_layouts(dtype, [5, 6, 7], 600 + s):
            for name, cut, indices, _ in cases():
                if cut is not None:
                    continue
                shape = cpu.index_tensors([as_index(i, "cpu") for i in indices]).shape
                n = int(np.prod(shape))
                v = tensor(values(dtype, n, 700 + s), dtype, shape)
                for where, device, mixed in [("GPU indices", GPU, False), ("mixed", GPU, True)]:
                    ci, gi = [as_index(i, "cpu") for i in indices], placed(indices, device, mixed)
                    what = f"{dtype} {sname} {name}, {where}"
                    assert_same(gpu.index_put_tensors(gi, v.to(GPU), False), cpu.index_put_tensors(ci, v, False), f"index_put {what}")
                    assert_bitwise(gpu.index_put_tensors(gi, v.to(GPU), True), cpu.index_put_tensors(ci, v, True),
                                   f"index_put accumulate {what}")
                    if n > 0:
                        one = v.reshape([-1]).narrow(0, 0, 1).reshape([])
                        assert_same(gpu.index_put_tensors(gi, one.to(GPU), False), cpu.index_put_tensors(ci, one, False),
                                    f"index_put broadcast {what}")


@pytest.mark.gpu
def test_large_masks_compact_in_order():
    """More true elements than one tile and than one chunk of the scan of the tiles' counts, in several layouts
    (ref: tests/rocm_index.rs:406-449)."""
    rows, cols = 3001, 1709
    m = words(42, rows * cols) % np.uint64(5) < 3
    mt = bools(m.reshape(rows, cols))
    x = np.arange(rows * cols, dtype=np.int64).reshape(rows, cols)
    gx = tensor(x, DT.I64, [rows, cols], GPU)
    got = gx.index_tensors([mt.to(GPU)])
    assert np.array_equal(array(got), x[m.reshape(rows, cols)])
    got = gx.transpose(0, 1).index_tensors([mt.transpose(0, 1).to(GPU)])
    assert np.array_equal(array(got), x.T[m.reshape(rows, cols).T])
    for fill in (False, True):
        full = bools(np.full((rows, cols), fill))
        got = gx.index_tensors([full.to(GPU)])
        assert np.array_equal(array(got), x[np.full((rows, cols), fill)])
    # A tile boundary inside the mask, a mask of one dimension and one of three over a strided target.
    for n in (1, 4095, 4096, 4097, 1000):
        m1 = m[:n]
        x1 = tensor(np.arange(n, dtype=np.float32), DT.F32, [n], GPU)
        assert np.array_equal(array(x1.index_tensors([bools(m1).to(GPU)])), np.arange(n, dtype=np.float32)[m1])
    m3 = m[:60].reshape(3, 4, 5)
    x3 = np.arange(120, dtype=np.float32).reshape(3, 4, 10)
    g3 = tensor(x3, DT.F32, [3, 4, 10], GPU).narrow(2, 3, 5)
    got = g3.index_tensors([bools(m3).to(GPU)])
    assert got.shape == [int(m3.sum())] and np.array_equal(array(got), x3[:, :, 3:8][m3])
    # The coordinates themselves, as the CPU gives them.
    for view in (lambda t: t, lambda t: t.transpose(0, 1)):
        gc, cc = view(mt.to(GPU)).mask_coordinates(), view(mt).mask_coordinates()
        for g, c in zip(gc, cc):
            assert_same(g, c, "mask coordinates")


def _a_mask_alone(device):
    """A mask as the only index - over leading dimensions, over all of them, behind full slices, as a view - read,
    assigned one value, assigned as many values as it selects, and accumulated into: numpy's results. (The host layer
    takes a contiguous mask that stands alone as linear positions, and one value for all of it as a select.)"""
    rng = np.random.default_rng(11)
    for dtype, npdt in ((DT.F32, np.float32), (DT.I64, np.int64), (DT.BF16, np.uint16)):
        for shape, mshape, start in (([6, 5, 4], [6, 5], 0), ([6, 5, 4], [6], 0), ([6, 5, 4], [6, 5, 4], 0), ([6, 5, 4], [5], 1),
                                     ([6, 5, 4], [5, 4], 1), ([70, 130], [70, 130], 0), ([9000], [9000], 0)):
            a = rng.integers(0, 30000, shape).astype(npdt)
            m = rng.random(mshape) < 0.5
            x, mt = tensor(a, dtype, shape, device), bools(m).to(device)
            at = (slice(None),) * start + (m,)
            idx = [None] * start + [mt]
            assert np.array_equal(array(x.index_tensors(idx)), a[at]), (dtype, shape, mshape)
            one = np.array([7], dtype=npdt)
            for vshape in ([], [1]):
                got = x.index_put_tensors(idx, tensor(one, dtype, vshape, device), False)
                want = a.copy()
                want[at] = one[0]
                assert np.array_equal(array(got), want), (dtype, shape, mshape, vshape)
            many = rng.integers(0, 30000, a[at].shape).astype(npdt)
            got = x.index_put_tensors(idx, tensor(many, dtype, list(many.shape), device), False)
            want = a.copy()
            want[at] = many
            assert np.array_equal(array(got), want), (dtype, shape, mshape, "values")
            if dtype == DT.I64:
                got = x.index_put_tensors(idx, tensor(one, dtype, [], device), True)
                want = a.copy()
                want[at] += one[0]
                assert np.array_equal(array(got), want), (dtype, shape, mshape, "accumulate")
            if len(mshape) == 2:
                view = bools(np.ascontiguousarray(m.T)).to(device).transpose(0, 1)
                got = x.index_put_tensors([None] * start + [view], tensor(one, dtype, [], device), False)
                want = a.copy()
                want[at] = one[0]
                assert np.array_equal(array(got), want), (dtype, shape, mshape, "view")
                assert np.array_equal(array(x.index_tensors([None] * start + [view])), a[at])


    # Masks that are views: expanded along a dimension, and cut out of a larger one.
    a = rng.integers(0, 30000, [6, 5, 4]).astype(np.float32)
    x = tensor(a, DT.F32, [6, 5, 4], device)
    seven = tensor(np.array([7.0], dtype=np.float32), DT.F32, [], device)
    row = rng.random([5]) < 0.5
    wide = rng.random([8, 7]) < 0.5
    views = [(bools(row.reshape(1, 5)).to(device).expand([6, 5]), np.broadcast_to(row, (6, 5))),
             (bools(wide).to(device).narrow(0, 1, 6).narrow(1, 2, 5), wide[1:7, 2:7])]
    for view, m in views:
        assert np.array_equal(array(x.index_tensors([view])), a[m])
        want = a.copy()
        want[m] = 7.0
        assert np.array_equal(array(x.index_put_tensors([view], seven, False)), want)
        many = np.arange(int(m.sum()) * 4, dtype=np.float32).reshape(-1, 4)
        want = a.copy()
        want[m] = many
        assert np.array_equal(array(x.index_put_tensors([view], tensor(many, DT.F32, list(many.shape), device), False)), want)


def test_a_mask_alone_follows_numpy():
    _a_mask_alone("cpu")


@pytest.mark.gpu
def test_a_mask_alone_follows_numpy_on_the_device():
    _a_mask_alone(GPU)


@pytest.mark.gpu
def test_overwrites_of_rows_keep_the_last_of_repeated_positions():
    """Rows that copy as 16-byte tiles and rows that don't, many repeats of few positions."""
    for dtype, width in [(DT.BF16, 256), (DT.F32, 64), (DT.F32, 7), (DT.U8, 48), (DT.I64, 5)]:
        rows, m = 37, 1000
        x = tensor(values(dtype, rows * width, 1), dtype, [rows, width])
        v = tensor(values(dtype, m * width, 2), dtype, [m, width])
        pos = (words(3, m) % np.uint64(rows)).astype(np.int64)
        got = x.to(GPU).index_put_tensors([ints(pos).to(GPU)], v.to(GPU), False)
        want = array(x).copy()
        va = array(v)
        for i, p in enumerate(pos):
            want[p] = va[i]
        assert np.array_equal(array(got).view(np.uint8), want.view(np.uint8)), (dtype, width)


@pytest.mark.gpu
def test_positions_out_of_range_report_what_the_cpu_reports():
    x = tensor(values(DT.F32, 24, 1), DT.F32, [2, 3, 4])
    gx = x.to(GPU)
    for indices in ([np.array([0, 2])], [np.array([0]), np.array([1, -4])], [np.array([0, 5, 7]), np.array([9, 1, 1])],
                    [np.array([0]), None, np.array([4])], [np.array([5]), None, np.zeros([0], dtype=np.int64)]):
        with pytest.raises(h.HomuraError) as c:
            x.index_tensors([as_index(i, "cpu") for i in indices])
        for device in (GPU, "cpu"):
            with pytest.raises(h.HomuraError) as g:
                gx.index_tensors([as_index(i, device) for i in indices])
            assert str(g.value) == str(c.value)
        with pytest.raises(h.HomuraError) as g:
            gx.index_put_tensors([as_index(i, GPU) for i in indices], tensor(np.zeros(1, dtype=np.float32), DT.F32, []).to(GPU), True)
        assert str(g.value) == str(c.value)
    # A failed write leaves the target unchanged (the work happens on a copy).
    assert_same(gx, x, "the target of a failed index_put")


@pytest.mark.gpu
def test_the_c_abi_of_positions_masks_and_overwrites():
    from ctypes import byref, c_int64

    from homura_amd import capi
    L = capi.lib
    ctx = capi.Context(0)
    try:
        # hmr_index_positions: two passes over a [2, 3] broadcast shape: rows (I32, negative wraps) x stride 4, columns.
        rows = ctx.upload(np.array([-1, 0], dtype=np.int32))
        cols = ctx.upload(np.array([3, -4, 1], dtype=np.int64))
        out = ctx.upload(np.full(6, -7, dtype=np.int64))
        O = capi.make_desc(out.ptr, capi.I64, [2, 3], [3, 1], 0)
        R = capi.make_desc(rows.ptr, capi.I32, [2, 3], [1, 0], 0)
        C = capi.make_desc(cols.ptr, capi.I64, [2, 3], [0, 1], 0)
        capi.check(L.hmr_index_positions(ctx.handle, byref(O), byref(R), 3, 4, 1))
        capi.check(L.hmr_index_positions(ctx.handle, byref(O), byref(C), 4, 1, 0))
        ctx.synchronize()
        assert out.download(np.int64, 6).tolist() == [11, 8, 9, 3, 0, 1]
        F = capi.make_desc(out.ptr, capi.F64, [2, 3], [3, 1], 0)
        assert L.hmr_index_positions(ctx.handle, byref(F), byref(R), 3, 4, 1) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "index_positions: the positions are I64"
        assert L.hmr_index_positions(ctx.handle, byref(O), byref(F), 3, 4, 1) == capi.HMR_INVALID
        # Masks: an offset per tile of 4096 elements and the total after them, then (up to 65 536 tiles) the tiles' raw
        # counts, which the scan by many workgroups keeps apart from the offsets it writes.
        n = 3 * 4096 + 5
        bytes_, word = c_int64(), c_int64()
        capi.check(L.hmr_mask_workspace(n, byref(bytes_), byref(word)))
        assert (bytes_.value, word.value) == ((5 + 4) * 8, 4)
        big, big_word = c_int64(), c_int64()
        capi.check(L.hmr_mask_workspace(65537 * 4096, byref(big), byref(big_word)))
        assert (big.value, big_word.value) == (65538 * 8, 65537)
        m = words(9, n) % np.uint64(4) == 0
        dm = ctx.upload(m.astype(np.uint8))
        ws = ctx.malloc(bytes_.value)
        M = capi.make_desc(dm.ptr, capi.BOOL, [n], [1], 0)
        assert L.hmr_mask_count(ctx.handle, byref(M), ws.ptr, 8) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "mask_count: the workspace is too small"
        capi.check(L.hmr_mask_count(ctx.handle, byref(M), ws.ptr, bytes_.value))
        ctx.synchronize()
        counts = ws.download(np.uint64, 5)
        tiles = [int(m[k * 4096:(k + 1) * 4096].sum()) for k in range(4)]
        assert counts.tolist() == [0, tiles[0], sum(tiles[:2]), sum(tiles[:3]), int(m.sum())]
        total = int(m.sum())
        coords = ctx.malloc(total * 8)
        K = capi.make_desc(coords.ptr, capi.I64, [1, total], [total, 1], 0)
        capi.check(L.hmr_mask_coordinates(ctx.handle, byref(M), ws.ptr, bytes_.value, byref(K)))
        ctx.synchronize()
        assert np.array_equal(coords.download(np.int64, total), np.nonzero(m)[0])
        U = capi.make_desc(dm.ptr, capi.U8, [n], [1], 0)
        assert L.hmr_mask_count(ctx.handle, byref(U), ws.ptr, bytes_.value) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "mask_count: the mask is BOOL"
        # hmr_index_overwrite: a word per position of out along dim; the last of repeated positions wins.
        capi.check(L.hmr_index_overwrite_workspace(10, byref(bytes_)))
        assert bytes_.value == 80
        x = ctx.upload(np.arange(10, dtype=np.float32))
        v = ctx.upload(np.array([1, 2, 3], dtype=np.float32))
        p = ctx.upload(np.array([3, 3, 7], dtype=np.int64))
        w = ctx.malloc(80)
        X = capi.make_desc(x.ptr, capi.F32, [10], [1], 0)
        V = capi.make_desc(v.ptr, capi.F32, [3], [1], 0)
        P = capi.make_desc(p.ptr, capi.I64, [3], [1], 0)
        assert L.hmr_index_overwrite(ctx.handle, byref(X), byref(V), byref(P), 0, w.ptr, 79) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "index_overwrite: the workspace is too small"
        capi.check(L.hmr_index_overwrite(ctx.handle, byref(X), byref(V), byref(P), 0, w.ptr, 80))
        ctx.synchronize()
        assert x.download(np.float32, 10).tolist() == [0.0, 1.0, 2.0, 2.0, 4.0, 5.0, 6.0, 3.0, 8.0, 9.0]
    finally:
        ctx.close()


@pytest.mark.gpu
def test_masked_reads_and_empty_cache_from_two_threads_do_not_deadlock():
    """`x[mask]` allocates inside the device's execution lock (and so looks the device up) while empty_cache walks
    the devices and takes each execution lock: the two orders must not cross. The thread is joined with a
    time limit, so a regression fails here instead of hanging the run."""
    import threading

    x = tensor(values(DT.F32, 4096, 77), DT.F32, [64, 64]).to(GPU)
    keep = bools(mask([64, 64], 78)).to(GPU)
    want = array(x.index_tensors([keep]))
    failures = []

    def reads():
        try:
            for _ in range(200):
                if not same(array(x.index_tensors([keep])), want):
                    failures.append("a masked read changed")
        except Exception as e:  # pragma: no cover
            failures.append(repr(e))

    worker = threading.Thread(target=reads, daemon=True)
    worker.start()
    for _ in range(200):
        h.empty_cache()
    worker.join(timeout=60)
    assert not worker.is_alive(), "x[mask] and empty_cache wait for each other"
    assert not failures, failures


def random_indices(rng, shape):
    """A list of None / integer arrays / bool masks for a tensor of `shape`, as numpy arrays: integer tensors of one
    broadcast shape with repeats and negatives, or one mask over one or two dimensions with scalar indices beside."""
    nd = len(shape)
    out = []
    if rng.integers(0, 3) == 0 and nd >= 1:
        # one mask, placed at a random dimension
        span = int(rng.integers(1, min(2, nd) + 1))
        at = int(rng.integers(0, nd - span + 1))
        density = float(rng.choice([0.0, 0.05, 0.5, 0.95, 1.0]))
        m = rng.random(shape[at:at + span]) < density
        d = 0
        while d < nd:
            if d == at:
                out.append(m)
                d += span
            else:
                pick = rng.integers(0, 3) == 0
                out.append(np.array(int(rng.integers(-shape[d], shape[d]))) if pick else None)
                d += 1
    else:
        bshape = [int(rng.choice([1, 2, 3, 17, 300])) for _ in range(int(rng.integers(0, 3)))]
        some = False
        for d in range(nd):
            if rng.integers(0, 2) == 0 and not (d == nd - 1 and not some):
                out.append(None)
                continue
            some = True
            ishape = [n if rng.integers(0, 4) else 1 for n in bshape]
            out.append(rng.integers(-shape[d], shape[d], ishape).astype(np.int64))
    while out and out[-1] is None:
        out.pop()
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(10))
def test_random_index_expressions_match_the_cpu(seed):
    """Index expressions drawn from a seeded generator over tensors of random shapes and layouts: reading, writing
    (the last of repeated positions wins) and accumulating (added in the CPU's order), with the indices on the GPU."""
    rng = np.random.default_rng(0x5EED4000 + seed)
    every = [DT.F32, DT.BF16, DT.I64, DT.U8, DT.F64, DT.Bool, DT.F16, DT.I32]
    sizes = [1, 2, 3, 5, 8, 17, 64, 130]
    for case in range(60):
        dtype = every[int(rng.integers(0, len(every)))]
        shape = [int(rng.choice(sizes)) for _ in range(int(rng.integers(1, 5)))]
        if int(np.prod(shape)) > 200000:
            continue
        indices = random_indices(rng, shape)
        if not any(i is not None for i in indices):
            continue
        layouts = operand_layouts(dtype, shape, 9000 * seed + case)
        sname, cpu, gpu = layouts[int(rng.integers(0, len(layouts)))]
        what = f"seed {seed} case {case}: {dtype} {shape} {sname} " + str([None if i is None else (str(i.dtype), i.shape) for i in indices])
        itype = DT.I64 if rng.integers(0, 2) else DT.I32
        ci = [as_index(i, "cpu", itype) for i in indices]
        gi = [as_index(i, GPU, itype) for i in indices]
        want = cpu.index_tensors(ci)
        assert_same(gpu.index_tensors(gi), want, f"{what}: read")
        n = int(np.prod(want.shape))
        v = tensor(values(dtype, n, 9500 + case), dtype, list(want.shape))
        assert_same(gpu.index_put_tensors(gi, v.to(GPU), False), cpu.index_put_tensors(ci, v, False), f"{what}: index_put")
        assert_bitwise(gpu.index_put_tensors(gi, v.to(GPU), True), cpu.index_put_tensors(ci, v, True), f"{what}: accumulate")
        if n > 0 and len(want.shape) >= 1:
            # a value that broadcasts: the result's last dimension alone
            tail = tensor(values(dtype, want.shape[-1], 9600 + case), dtype, [want.shape[-1]])
            assert_same(gpu.index_put_tensors(gi, tail.to(GPU), False), cpu.index_put_tensors(ci, tail, False), f"{what}: broadcast value")


@pytest.mark.parametrize("seed", range(10))
def test_random_index_expressions_follow_numpy(seed):
    """The same generator on the CPU against numpy's advanced indexing: reading, and assignment where no position
    repeats (numpy leaves the winner of repeated positions open, the reference does not)."""
    rng = np.random.default_rng(0x5EED4000 + seed)
    sizes = [1, 2, 3, 5, 8, 17, 64, 130]
    for case in range(60):
        dtype = [DT.F32, DT.I64, DT.U8, DT.F64][int(rng.integers(0, 4))]
        shape = [int(rng.choice(sizes)) for _ in range(int(rng.integers(1, 5)))]
        if int(np.prod(shape)) > 200000:
            continue
        indices = random_indices(rng, shape)
        if not any(i is not None for i in indices):
            continue
        x = values(dtype, int(np.prod(shape)), 9000 * seed + case).reshape(shape)
        t = tensor(x, dtype, shape)
        key = tuple(slice(None) if i is None else i for i in indices)
        want = x[key]
        got = t.index_tensors([as_index(i, "cpu") for i in indices])
        what = f"seed {seed} case {case}: {dtype} {shape} " + str([None if i is None else (str(i.dtype), i.shape) for i in indices])
        assert same(array(got), want), what
