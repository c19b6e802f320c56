"""Tensors of more than 4 GiB and of more than 2^32 elements: byte offsets and element counts that do not fit 32 bits.

Every kernel family of the path runs once on an operand of 5 GiB (or, for bytes, of 2^32 + 4099 elements) and its
result is judged where that is cheap: integer results element for element with numpy, floating-point ones in
windows - the first rows, the rows on both sides of byte 2^32 and the last rows - against the CPU backend run on
those rows only (rows and columns of these ops do not depend on each other). Inputs repeat with a period of
1 000 003 elements (prime), so that a result taken from an offset that wrapped would differ.
"""
import numpy as np
import pytest

from tests import oracle
from tests.support import DT, GPU, NP, assert_bitwise, f32_to_bf16_bits, h, tensor, words
from tests.test_rocm_reduce import check_softmax

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())

PERIOD = 1_000_003
FOUR_GIB = 1 << 32


def array(t):
    """The elements of a tensor as a read-only numpy array over the bytes that came back (no second copy)."""
    return np.frombuffer(t.to_bytes(), dtype=NP[t.dtype]).reshape(t.shape)


def ints_pattern(n, mul, dtype):
    base = ((np.arange(PERIOD, dtype=np.uint64) * np.uint64(mul)) >> np.uint64(7)).astype(dtype)
    return np.resize(base, n)


def floats_pattern(n, seed, spread=2.0):
    """f32 values in (-spread, spread), none of them equal to its neighbours."""
    w = words(seed, PERIOD)
    base = (((w >> np.uint64(11)).astype(np.float64) / float(1 << 53)) * 2.0 - 1.0) * spread
    return np.resize(base.astype(np.float32), n)


def windows(rows, row_bytes, height):
    """Row ranges [start, start + height): the first rows, those around byte 2^32 and the last ones."""
    middle = FOUR_GIB // row_bytes - height // 2
    assert 0 < middle and middle + height < rows
    return [0, middle, rows - height]


def test_byte_offsets_past_four_gib_in_contiguous_ops_folds_and_copies():
    n = 5 * (1 << 28) + 4099  # i32: 5 GiB and a ragged last tile
    a, b = ints_pattern(n, 2654435761, np.int32), ints_pattern(n, 40503, np.int32)
    x, y = tensor(a, DT.I32, [n], GPU), tensor(b, DT.I32, [n], GPU)
    got = array(x.add(y))
    assert np.array_equal(got, a + b)
    got = array(x.greater(y))
    assert np.array_equal(got, (a > b).astype(np.uint8))
    del got, y, b
    assert int(array(x.sum()).reshape(-1)[0]) == int(a.sum(dtype=np.int64))
    half = (n - 1) // 2
    rows, rows_np = x.narrow(0, 1, n - 1).reshape([2, half]), a[1:].reshape(2, half)
    assert array(rows.sum_dim(1, False)).tolist() == rows_np.sum(axis=1, dtype=np.int64).tolist()
    got = array(rows.sum_dim(0, False))
    assert np.array_equal(got, rows_np.sum(axis=0, dtype=np.int64))
    # A copy out of the transposed view, and the elements in reverse order.
    got = array(rows.transpose(0, 1).contiguous())
    assert got.shape == (half, 2) and np.array_equal(got, rows_np.T)
    got = array(x.flip([0]))
    assert np.array_equal(got, a[::-1])


def test_more_than_two_to_the_32_elements():
    n = FOUR_GIB + 4099
    a, b = ints_pattern(n, 2654435761, np.uint8), ints_pattern(n, 40503, np.uint8)
    x, y = tensor(a, DT.U8, [n], GPU), tensor(b, DT.U8, [n], GPU)
    got = array(x.add(y))
    assert got.shape == (n,) and np.array_equal(got, a + b)
    got = array(x.less(y))
    assert np.array_equal(got, (a < b).astype(np.uint8))
    del got
    assert int(array(x.sum()).reshape(-1)[0]) == int(a.sum(dtype=np.int64))
    # A sparse mask over all of it: the coordinates of its true elements, in order, and the elements picked by it.
    m = (a == 201) & (b < 16)
    m[[FOUR_GIB - 1, FOUR_GIB, n - 1]] = True
    mask = tensor(m.astype(np.uint8), DT.Bool, [n], GPU)
    where = np.flatnonzero(m)
    assert where.size > 1000 and where[-1] > FOUR_GIB
    assert np.array_equal(array(mask.mask_coordinates()[0]), where)
    assert np.array_equal(array(y.index_tensors([mask])), b[where])


def test_softmax_and_row_folds_of_five_gib():
    rows, cols = 1281 * 256, 4096  # f32: 5.004 GiB; as [1281, 2^20] the same bytes give columns 4 MiB apart
    a = floats_pattern(rows * cols, 5).reshape(rows, cols)
    x = tensor(a, DT.F32, [rows, cols], GPU)
    for log in (False, True):
        g = x.log_softmax(1) if log else x.softmax(1)
        for start in windows(rows, cols * 4, 32):
            part = tensor(a[start:start + 32], DT.F32)
            c = part.log_softmax(1) if log else part.softmax(1)
            check_softmax(g.narrow(0, start, 32), c, part.to(DT.F64), 1, log, f"rows from {start} log {log}")
        del g
    # Row and column sums and maxima against numpy in f64 (the sums to the accuracy of an f64 accumulation).
    exact = a.sum(axis=1, dtype=np.float64)
    got = array(x.sum_dim(1, False)).astype(np.float64)
    assert np.all(np.abs(got - exact) <= np.spacing(np.abs(exact).astype(np.float32)).astype(np.float64))
    exact = a.sum(axis=0, dtype=np.float64)
    got = array(x.sum_dim(0, False)).astype(np.float64)
    assert np.all(np.abs(got - exact) <= np.spacing(np.abs(exact).astype(np.float32)).astype(np.float64) + 1e-6)
    assert np.array_equal(array(x.max_dim(1, False)[0]), a.max(axis=1))
    assert np.array_equal(array(x.max_dim(0, False)[0]), a.max(axis=0))
    where = array(x.max_dim(1, False)[1])
    assert np.array_equal(a[np.arange(rows), where], a.max(axis=1))
    # The same bytes as 1281 positions of 2^20 rows each: a softmax across memory whose positions span 5 GiB.
    wide = 1 << 20
    tall, tall_np = x.reshape([1281, wide]), a.reshape(1281, wide)
    for log in (False, True):
        g = tall.log_softmax(0) if log else tall.softmax(0)
        for start in (0, wide // 2 - 32, wide - 64):
            part = tensor(np.ascontiguousarray(tall_np[:, start:start + 64]), DT.F32)
            c = part.log_softmax(0) if log else part.softmax(0)
            check_softmax(g.narrow(1, start, 64), c, part.to(DT.F64), 0, log, f"columns from {start} log {log}")
        del g


def test_bf16_softmax_across_memory_and_lookups_of_five_gib():
    outer, n, inner = 40, 1024, 65536  # bf16: 5 GiB; positions 128 KiB apart, the last outer slices past byte 2^32
    a = np.resize(f32_to_bf16_bits(floats_pattern(PERIOD, 9, 3.0)), outer * n * inner).reshape(outer, n, inner)
    x = tensor(a, DT.BF16, [outer, n, inner], GPU)
    for log in (False, True):
        g = x.log_softmax(1) if log else x.softmax(1)
        for o, start in ((0, 0), (31, inner - 128), (32, 0), (outer - 1, inner - 128)):
            part = tensor(np.ascontiguousarray(a[o:o + 1, :, start:start + 128]), DT.BF16)
            c = part.log_softmax(1) if log else part.softmax(1)
            check_softmax(g.narrow(0, o, 1).narrow(2, start, 128), c, part.to(DT.F64), 1, log,
                          f"outer {o} columns from {start} log {log}")
        del g
    # A 16-bit unary op is a lookup: the flat walk, and the walk of a permuted view (heads before positions).
    total, length = outer * n * inner, 1 << 20
    flat = x.reshape([total]).silu()
    for start in (0, FOUR_GIB // 2 - length // 2, total - length):
        part = tensor(a.reshape(-1)[start:start + length], DT.BF16)
        assert_bitwise(flat.narrow(0, start, length), part.silu(), f"silu of elements from {start}")
    del flat
    heads = [80, 2048, 32, 512]
    swapped = x.reshape(heads).permute([0, 2, 1, 3]).gelu()
    assert swapped.shape == [80, 32, 2048, 512]
    by_heads = a.reshape(heads)
    for b, head in ((0, 0), (63, 31), (64, 0), (79, 31)):
        part = tensor(np.ascontiguousarray(by_heads[b, :, head, :]), DT.BF16)
        assert_bitwise(swapped.narrow(0, b, 1).narrow(1, head, 1).reshape([2048, 512]), part.gelu(),
                       f"gelu of batch {b} head {head}")


def test_index_ops_on_a_table_of_five_gib():
    rows, width, picks = 5 * (1 << 18) + 3, 1024, 4096  # f32 rows of 4 KiB: row 2^20 starts at byte 2^32
    a = floats_pattern(rows * width, 21).reshape(rows, width)
    table = tensor(a, DT.F32, [rows, width], GPU)
    w = words(33, picks)
    ids_np = (w % np.uint64(rows)).astype(np.int64)
    ids_np[:8] = [0, rows - 1, (1 << 20) - 1, 1 << 20, (1 << 20) + 1, rows - 2, 1, 5 * (1 << 18)]
    ids_np = np.unique(ids_np)  # distinct rows: sums and writes do not depend on an order
    ids_np = ids_np[np.argsort(words(36, ids_np.size), kind="stable")]
    ids = tensor(ids_np, DT.I64, [ids_np.size], GPU)
    assert np.array_equal(array(table.index_select(0, ids)), a[ids_np])
    assert np.array_equal(array(table.index_tensors([ids])), a[ids_np])
    signed = np.where(np.arange(ids_np.size) % 2 == 0, ids_np, ids_np - rows)  # every other one counted from the end
    assert np.array_equal(array(table.index_tensors([tensor(signed, DT.I64, [signed.size], GPU)])), a[ids_np])
    src_np = floats_pattern(ids_np.size * width, 34).reshape(ids_np.size, width)
    src = tensor(src_np, DT.F32, list(src_np.shape), GPU)
    expected = a.copy()
    expected[ids_np] += src_np
    got = array(table.index_add(0, ids, src))
    assert np.array_equal(got, expected)
    expected[ids_np] = src_np
    got = array(table.index_put_tensors([ids], src, False))
    assert np.array_equal(got, expected)
    del got, expected
    # Single elements by position, enough of them (every 13th: 412 MB) for the stores that go past the caches.
    every = np.arange(0, rows * width, 13, dtype=np.int64)
    got = array(table.reshape([rows * width]).index_select(0, tensor(every, DT.I64, [every.size], GPU)))
    assert np.array_equal(got, a.reshape(-1)[::13])
    del got, every
    # gather and scatter_add along the rows: four distinct columns of every row.
    r = np.arange(rows, dtype=np.int64)[:, None]
    cols_np = (r * 7 + np.arange(4, dtype=np.int64)[None, :] * 259) % width
    cols = tensor(cols_np, DT.I64, [rows, 4], GPU)
    assert np.array_equal(array(table.gather(1, cols)), np.take_along_axis(a, cols_np, axis=1))
    add_np = floats_pattern(rows * 4, 35).reshape(rows, 4)
    got = array(table.scatter_add(1, cols, tensor(add_np, DT.F32, [rows, 4], GPU)))
    expected = a.copy()
    np.put_along_axis(expected, cols_np, np.take_along_axis(a, cols_np, axis=1) + add_np, axis=1)
    assert np.array_equal(got, expected)


def test_layout_ops_and_scans_of_five_gib():
    batch, side = 321, 2048  # f32 [321, 2048, 2048]: matrix 256 starts at byte 2^32
    a = floats_pattern(batch * side * side, 41).reshape(batch, side, side)
    x = tensor(a, DT.F32, [batch, side, side], GPU)
    upper, lower, turned, mirrored = x.triu(1), x.tril(0), x.flip([1]), x.flip([2])
    moved = x.transpose(1, 2).contiguous()
    for m in (0, 255, 256, batch - 1):
        assert np.array_equal(array(upper.narrow(0, m, 1))[0], np.triu(a[m], 1)), f"triu of matrix {m}"
        assert np.array_equal(array(lower.narrow(0, m, 1))[0], np.tril(a[m], 0)), f"tril of matrix {m}"
        assert np.array_equal(array(turned.narrow(0, m, 1))[0], a[m, ::-1]), f"rows of matrix {m} reversed"
        assert np.array_equal(array(mirrored.narrow(0, m, 1))[0], a[m, :, ::-1]), f"matrix {m} mirrored"
        assert np.array_equal(array(moved.narrow(0, m, 1))[0], a[m].T), f"matrix {m} transposed"
    del upper, lower, turned, mirrored, moved
    # One transpose of the whole: [41088, 32768] -> [32768, 41088], judged in bands of eight result rows.
    tall = batch * side * side // 32768
    flat_np = a.reshape(tall, 32768)
    across = x.reshape([tall, 32768]).transpose(0, 1).contiguous()
    for start in (0, 16384, 32760):
        assert np.array_equal(array(across.narrow(0, start, 8)), flat_np[:, start:start + 8].T), f"band {start}"
    del across
    # permute(2, 0, 1) of [80, 4108, 4096] (the same bytes less a tail): result[k] = x[:, :, k].
    cube_np = a.reshape(-1)[:80 * 4108 * 4096].reshape(80, 4108, 4096)
    cube = x.reshape([batch * side * side]).narrow(0, 0, 80 * 4108 * 4096).reshape([80, 4108, 4096])
    turned = cube.permute([2, 0, 1]).contiguous()
    for k in (0, 2047, 4095):
        assert np.array_equal(array(turned.narrow(0, k, 1))[0], cube_np[:, :, k]), f"plane {k}"
    del turned, cube
    # Exclusive running products of factors near 1, along rows and along columns of [328 704, 4096].
    rows = batch * side * side // 4096
    f_np = (1.0 + a.reshape(rows, 4096) * np.float32(2.0 ** -9)).astype(np.float32)
    f = tensor(f_np, DT.F32, [rows, 4096], GPU)
    along = h.exclusive_cumprod(f, 1, False)
    for start in windows(rows, 4096 * 4, 16):
        part = tensor(f_np[start:start + 16], DT.F32)
        assert_bitwise(along.narrow(0, start, 16), h.exclusive_cumprod(part, 1, False), f"rows from {start}")
    del along
    down = h.exclusive_cumprod(f, 0, True)
    for start in (0, 2048, 4088):
        part = tensor(np.ascontiguousarray(f_np[:, start:start + 8]), DT.F32)
        assert_bitwise(down.narrow(1, start, 8), h.exclusive_cumprod(part, 0, True), f"columns from {start}")


def test_random_fills_of_five_gib():
    n = 5 * (1 << 28) + 4099
    h.manual_seed(77)
    g = h.rand([n], DT.F32, GPU)
    h.manual_seed(77)
    c = h.rand([n], DT.F32, "cpu")
    assert np.array_equal(array(g), array(c))
    del g, c
    m = 5 * (1 << 27) + 4099  # i64: 5 GiB
    h.manual_seed(78)
    g = h.randint(-5, 6, [m], DT.I64, GPU)
    h.manual_seed(78)
    c = h.randint(-5, 6, [m], DT.I64, "cpu")
    assert np.array_equal(array(g), array(c))
