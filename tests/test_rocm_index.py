"""index_select, gather, index_add and scatter_add on the GPU against the CPU oracle, through the host layer and the
C ABI: the same bytes for the reads, the same bits for the adds, whose sums follow the CPU's order
(ref: tests/rocm_index.rs:35-278, 451-500, 616-639)."""
from ctypes import byref, c_int64

import numpy as np
import pytest

from homura_amd import capi
from tests import oracle
from tests.support import DT, DTYPES, GPU, NP, array, assert_bitwise, assert_same, bits, h, layouts, tensor, values, words

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())
L = capi.lib


def ints(v, shape=None, dtype=DT.I64):
    a = np.asarray(v, dtype=np.int64)
    return tensor(a.astype(NP[dtype]), dtype, list(a.shape) if shape is None else shape)


def random_positions(n, size, seed):
    return (words(seed, n) % np.uint64(size)).astype(np.int64)


def index_layouts(v, shape):
    """The same positions as I64, as I32 and as every other element of a wider I64 tensor (ref: rocm_index.rs:47-69)."""
    v = np.asarray(v, dtype=np.int64)
    t = ints(v, shape)
    wide = np.zeros(2 * v.size, dtype=np.int64)
    wide[1::2] = v
    strided = tensor(wide, DT.I64, [max(v.size, 0), 2]).select(1, 1).reshape(shape)
    assert array(strided).reshape(-1).tolist() == v.tolist()
    return [("I64", t), ("I32", t.to(DT.I32)), ("strided I64", strided)]


def operand_layouts(dtype, shape, seed):
    """A tensor of `shape` in three layouts: contiguous, permuted, every other element of a buffer with an offset
    (ref: rocm_index.rs:94-133)."""
    n = int(np.prod(shape))
    rev, perm = list(reversed(shape)), list(reversed(range(len(shape))))
    base = tensor(values(dtype, n, seed), dtype)
    wide = tensor(values(dtype, 2 * n + 3, seed + 1), dtype)
    views = [("contiguous", lambda b, w: b.reshape(shape)), ("permuted", lambda b, w: b.reshape(rev).permute(perm)),
             ("strided", lambda b, w: w.narrow(0, 3, 2 * n).reshape([n, 2]).select(1, 1).reshape(shape))]
    bg, wg = base.to(GPU), wide.to(GPU)
    return [(name, f(base, wide), f(bg, wg)) for name, f in views]


def test_index_select_matches_the_cpu():
    checked = 0
    for s, dtype in enumerate(DTYPES):
        for pair in layouts(dtype, 10 + s):
            shape = pair.cpu.shape
            for dim in range(len(shape)):
                n = shape[dim]
                picks = [] if n == 0 else [n - 1, 0, n - 1, n // 2]
                for iname, index in index_layouts(picks, [len(picks)]):
                    assert_same(pair.gpu.index_select(dim, index.to(GPU)), pair.cpu.index_select(dim, index),
                                f"{dtype} {pair.name} dim {dim} {iname}")
                    checked += 1
    assert checked > 500


@pytest.mark.parametrize("dtype", [DT.U8, DT.BF16, DT.F32, DT.I64])
def test_index_select_of_rows_that_vectorise(dtype):
    """An embedding lookup (rows of whole 16-byte tiles picked along dim 0, many repeats), the same from a wider
    table (row stride beyond the row), along a middle dimension, and along the innermost one (single elements)."""
    table = tensor(values(dtype, 5000 * 96, 31), dtype).reshape([5000, 96])
    tg = table.to(GPU)
    picks = ints(random_positions(20000, 5000, 32))
    assert_same(tg.index_select(0, picks.to(GPU)), table.index_select(0, picks), f"{dtype} embedding")
    assert_same(tg.narrow(1, 32, 64).index_select(0, picks.to(GPU)), table.narrow(1, 32, 64).index_select(0, picks), f"{dtype} wider table")
    cube, cg = table.reshape([50, 100, 96]), tg.reshape([50, 100, 96])
    mid = ints(random_positions(333, 100, 33), dtype=DT.I32)
    assert_same(cg.index_select(1, mid.to(GPU)), cube.index_select(1, mid), f"{dtype} middle dimension")
    inner = ints(random_positions(70, 96, 34))
    assert_same(cg.index_select(2, inner.to(GPU)), cube.index_select(2, inner), f"{dtype} innermost dimension")
    odd = table.narrow(1, 1, 64)  # rows that start off a 16-byte boundary for the narrow dtypes
    assert_same(tg.narrow(1, 1, 64).index_select(0, picks.to(GPU)), odd.index_select(0, picks), f"{dtype} unaligned rows")


def test_gather_matches_the_cpu():
    shape = [4, 5, 6]
    for s, dtype in enumerate(DTYPES):
        for sname, cpu, gpu in operand_layouts(dtype, shape, 100 + s):
            for dim in range(3):
                ishape = list(shape)  # longer than the source along dim, shorter in one other dimension
                ishape[dim] = 7
                ishape[(dim + 1) % 3] -= 1
                picks = random_positions(int(np.prod(ishape)), shape[dim], 7 * s + dim)
                for iname, index in index_layouts(picks, ishape):
                    assert_same(gpu.gather(dim, index.to(GPU)), cpu.gather(dim, index), f"{dtype} {sname} dim {dim} {iname}")
    x = tensor(values(DT.F32, 300 * 1000, 41), DT.F32).reshape([300, 1000])
    idx = ints(random_positions(300 * 64, 1000, 42), [300, 64])
    assert_same(x.to(GPU).gather(1, idx.to(GPU)), x.gather(1, idx), "gather [300, 64] of [300, 1000]")
    zero = tensor(np.array([2.5], dtype=np.float32), DT.F32).reshape([])
    assert_same(zero.to(GPU).gather(0, ints(0, []).to(GPU)), zero.gather(0, ints(0, [])), "0-dim gather")


def test_scatter_add_and_index_add_match_the_cpu():
    shape = [4, 5, 6]
    for s, dtype in enumerate(DTYPES):
        for sname, cpu, gpu in operand_layouts(dtype, shape, 200 + s):
            for dim in range(3):
                # scatter_add: an index smaller than self in the other dimensions, a source larger than the index.
                ishape = list(shape)
                ishape[dim] = 9
                ishape[(dim + 2) % 3] -= 2
                sshape = list(ishape)
                sshape[(dim + 1) % 3] += 1
                sshape[dim] += 2
                picks = random_positions(int(np.prod(ishape)), shape[dim], 11 * s + dim)
                src = tensor(values(dtype, int(np.prod(sshape)), 300 + s), dtype).reshape(sshape)
                for iname, index in index_layouts(picks, ishape):
                    assert_bitwise(gpu.scatter_add(dim, index.to(GPU), src.to(GPU)), cpu.scatter_add(dim, index, src),
                                   f"scatter_add {dtype} {sname} dim {dim} {iname}")
                # index_add: a vector of 9 positions with repeats.
                picks = random_positions(9, shape[dim], 13 * s + dim)
                sshape = list(shape)
                sshape[dim] = 9
                src = tensor(values(dtype, int(np.prod(sshape)), 400 + s), dtype).reshape(sshape)
                src_t = src.transpose(0, 2).contiguous().transpose(0, 2)
                for iname, index in index_layouts(picks, [9]):
                    for srcname, source in (("source", src), ("transposed source", src_t)):
                        assert_bitwise(gpu.index_add(dim, index.to(GPU), source.to(GPU)), cpu.index_add(dim, index, source),
                                       f"index_add {dtype} {sname} dim {dim} {iname} {srcname}")
    x = h.full([3], 0.0, DT.F32, "cpu")
    i, v = ints(2, []), tensor(np.array([5.0], dtype=np.float32), DT.F32)
    assert_same(x.to(GPU).index_add(0, i.to(GPU), v.to(GPU)), x.index_add(0, i, v), "0-dim index_add")


def order_sensitive(n):
    """Values whose f64 sum depends on the order: 2^53 + 1 + 1 - 2^53 is 0 from the left and 2 when the ones come
    first (ref: rocm_index.rs:210-221)."""
    big = 2.0 ** 53
    return np.array([big if i % 4 == 0 else (-big if i % 4 == 3 else 1.0) for i in range(n)])


def test_repeated_positions_add_in_the_cpus_order():
    n = 4000
    v = order_sensitive(n)
    src = tensor(v, DT.F64)
    picks = np.array([(i // 4) % 2 for i in range(n)], dtype=np.int64)
    index, reversed_index = ints(picks), ints(picks[::-1].copy())
    src_rev = tensor(v[::-1].copy(), DT.F64)
    x = h.full([2], 0.0, DT.F64, "cpu")
    for name, i, s in (("forward", index, src), ("reversed", reversed_index, src_rev)):
        assert_same(x.to(GPU).scatter_add(0, i.to(GPU), s.to(GPU)), x.scatter_add(0, i, s), f"scatter_add {name}")
        assert_same(x.to(GPU).index_add(0, i.to(GPU), s.to(GPU)), x.index_add(0, i, s), f"index_add {name}")
    forward = array(x.to(GPU).scatter_add(0, index.to(GPU), src.to(GPU))).tolist()
    backward = array(x.to(GPU).scatter_add(0, reversed_index.to(GPU), src_rev.to(GPU))).tolist()
    assert forward != backward, "the same pairs in the other order sum differently"
    # Many more pairs than one chunk of the sort, and targets spread over 17 bits.
    big = 3 * 2048 + 17
    w = tensor(order_sensitive(big), DT.F64)
    picks = ints(random_positions(big, 70000, 5))
    x = h.full([70000], 0.0, DT.F64, "cpu")
    assert_same(x.to(GPU).scatter_add(0, picks.to(GPU), w.to(GPU)), x.scatter_add(0, picks, w), "scatter_add over several chunks")


def test_large_scatters_and_long_groups():
    n, size = 200000, (1 << 25) + 5
    picks = ints(random_positions(n, size, 77))
    src = tensor(values(DT.U8, n, 78), DT.U8)
    x = tensor(values(DT.U8, size, 79), DT.U8)
    assert_same(x.to(GPU).scatter_add(0, picks.to(GPU), src.to(GPU)), x.scatter_add(0, picks, src), "scatter_add into 2^25 elements")
    picks = ints(random_positions(n, 300, 80))
    s = tensor(order_sensitive(n), DT.F64)
    x = h.full([300], 0.0, DT.F64, "cpu")
    assert_same(x.to(GPU).index_add(0, picks.to(GPU), s.to(GPU)), x.index_add(0, picks, s), "index_add with long groups")
    # Millions of positions (a histogram table of several scan chunks), three digits of targets, sums that show
    # any change of order.
    n, size = 3_000_001, 70_000
    picks = ints(random_positions(n, size, 83))
    s = tensor(order_sensitive(n), DT.F64)
    x = h.full([size], 0.0, DT.F64, "cpu")
    assert_same(x.to(GPU).scatter_add(0, picks.to(GPU), s.to(GPU)), x.scatter_add(0, picks, s), "scatter_add of 3M positions")
    # The gradient of an embedding: 30 000 token rows of 256 bf16 added into a table of 8 000 rows.
    rows = tensor(values(DT.BF16, 30000 * 256, 81), DT.BF16).reshape([30000, 256])
    rows = rows.masked_fill(rows.abs().greater(1e30), 1.0).masked_fill(rows.not_equal(rows), 0.5)
    tokens = ints(random_positions(30000, 8000, 82))
    table = h.full([8000, 256], 0.0, DT.BF16, "cpu")
    assert_bitwise(table.to(GPU).index_add(0, tokens.to(GPU), rows.to(GPU)), table.index_add(0, tokens, rows), "embedding gradient")


def test_positions_out_of_range_report_what_the_cpu_reports():
    x = tensor(np.arange(30, dtype=np.float32), DT.F32).reshape([5, 6])
    for d in ("cpu", GPU):
        xd = x.to(d)
        cases = [
            ("index -1 is out of bounds for dimension 0 with size 5", lambda: xd.index_select(0, ints([1, -1, 9]).to(d))),
            ("index 6 is out of bounds for dimension 1 with size 6", lambda: xd.gather(1, ints([[0, 6], [7, 0]]).to(d))),
            # The logical order of a transposed index, not its memory order.
            ("index 8 is out of bounds for dimension 0 with size 5",
             lambda: xd.narrow(1, 0, 2).gather(0, ints([[0, 9], [8, 0]]).to(d).transpose(0, 1))),
            ("index 7 is out of bounds for dimension 0 with size 5",
             lambda: xd.index_add(0, ints([0, 7, -2]).to(d), h.full([3, 6], 1.0, DT.F32, d))),
            ("index -2 is out of bounds for dimension 0 with size 5",
             lambda: xd.scatter_add(0, ints([[0], [-2]]).to(d), h.full([2, 1], 1.0, DT.F32, d))),
        ]
        for message, call in cases:
            with pytest.raises(Exception, match=message):
                call()
        # A rejected add leaves its target as it was.
        before = bits(xd)
        with pytest.raises(Exception, match="out of bounds"):
            xd.index_add(0, ints([9]).to(d), h.full([1, 6], 1.0, DT.F32, d))
        assert (bits(xd) == before).all()
    # The checks of the front end, the same on both devices.
    g = x.to(GPU)
    for message, call in [
        ("index_select\\(\\): Index is supposed to be a vector", lambda: g.index_select(0, ints([[0]]).to(GPU))),
        ("index_select\\(\\): Expected dtype i32 or i64 for index, got f32", lambda: g.index_select(0, g.narrow(0, 0, 1).reshape([6]))),
        ("Index tensor must have the same number of dimensions as input tensor", lambda: g.gather(0, ints([0]).to(GPU))),
        ("index_add\\(\\): Number of indices \\(2\\) should be equal to source.size\\(dim\\): \\(3\\), for dim: 0",
         lambda: g.index_add(0, ints([0, 1]).to(GPU), h.full([3, 6], 1.0, DT.F32, GPU))),
        ("scatter_add\\(\\): Expected self.dtype to be equal to src.dtype",
         lambda: g.scatter_add(0, ints([[0]]).to(GPU), h.full([1, 1], 1.0, DT.F64, GPU))),
    ]:
        with pytest.raises(Exception, match=message):
            call()


def sort_bytes(n):
    """The workspace of the adds: two buffers of n 64-bit words, a 256-entry histogram per tile of 2048 words and a
    word per 4096 histogram entries, rounded up to 256 bytes."""
    tiles = -(-n // 2048)
    chunks = -(-tiles * 256 // 4096)
    return -(-(16 * n + 4 * 256 * tiles + 4 * chunks) // 256) * 256


def test_the_c_abi_of_the_index_kernels():
    ctx = capi.Context(0)
    try:
        # hmr_index_check: the first offender in logical order of a strided index, its position and value.
        idx = np.array([[3, 99, 1], [-4, 2, 77]], dtype=np.int64)
        di = ctx.upload(idx)
        slot = ctx.malloc(16)
        transposed = capi.make_desc(di.ptr, capi.I64, [3, 2], [1, 3], 0)
        capi.check(L.hmr_index_check(ctx.handle, byref(transposed), 0, 10, 0, 0, slot.ptr))
        ctx.synchronize()
        assert slot.download(np.int64, 2).tolist() == [1, -4]  # logical order: 3, -4, 99, 2, 1, 77
        capi.check(L.hmr_index_check(ctx.handle, byref(transposed), -10, 100, 0, 0, slot.ptr))
        ctx.synchronize()
        assert slot.download(np.uint64, 2).tolist() == [2 ** 64 - 1, 0]
        capi.check(L.hmr_index_check(ctx.handle, byref(transposed), 0, 10, 1, -4, slot.ptr))  # -4 is exempt
        ctx.synchronize()
        assert slot.download(np.int64, 2).tolist() == [2, 99]
        # More elements than the single-workgroup form takes: the first offender of several, then none.
        big = (np.arange(200000) % 1000).astype(np.int32)
        big[[77777, 150000, 199999]] = [1000, -1, 5000]
        db = ctx.upload(big)
        B = capi.make_desc(db.ptr, capi.I32, [200000], [1], 0)
        capi.check(L.hmr_index_check(ctx.handle, byref(B), 0, 1000, 0, 0, slot.ptr))
        ctx.synchronize()
        assert slot.download(np.int64, 2).tolist() == [77777, 1000]
        capi.check(L.hmr_index_check(ctx.handle, byref(B), -1, 5001, 0, 0, slot.ptr))
        ctx.synchronize()
        assert slot.download(np.uint64, 2).tolist() == [2 ** 64 - 1, 0]
        # The last element of a single-workgroup check, and of a wave's share.
        for n, bad in ((65536, 65535), (65536, 1023), (1000, 999)):
            small = np.zeros(n, dtype=np.int64)
            small[bad] = 7
            dsm = ctx.upload(small)
            S_ = capi.make_desc(dsm.ptr, capi.I64, [n], [1], 0)
            capi.check(L.hmr_index_check(ctx.handle, byref(S_), 0, 7, 0, 0, slot.ptr))
            ctx.synchronize()
            assert slot.download(np.int64, 2).tolist() == [bad, 7]
        f = capi.make_desc(di.ptr, capi.F64, [6], [1], 0)
        assert L.hmr_index_check(ctx.handle, byref(f), 0, 1, 0, 0, slot.ptr) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "index_check: unsupported dtype"
        # hmr_scatter_add: the workspace it asks for, and too small a one.
        n = 5000
        need = c_int64()
        capi.check(L.hmr_scatter_add_workspace(n, byref(need)))
        assert need.value == sort_bytes(n) == 83200
        capi.check(L.hmr_index_add_workspace(100, 7, byref(need)))
        assert need.value == sort_bytes(100) == 2816
        assert L.hmr_index_add_workspace(1 << 31, 7, byref(need)) == capi.HMR_INVALID
        out = ctx.upload(np.zeros(16, dtype=np.float32))
        src = ctx.upload(np.ones(n, dtype=np.float32))
        picks = ctx.upload((np.arange(n) % 16).astype(np.int32))
        ws = ctx.malloc(sort_bytes(n))
        O = capi.make_desc(out.ptr, capi.F32, [16], [1], 0)
        S = capi.make_desc(src.ptr, capi.F32, [n], [1], 0)
        I = capi.make_desc(picks.ptr, capi.I32, [n], [1], 0)
        assert L.hmr_scatter_add(ctx.handle, byref(O), byref(S), byref(I), 0, ws.ptr, 100) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "scatter_add: the workspace is too small"
        capi.check(L.hmr_scatter_add(ctx.handle, byref(O), byref(S), byref(I), 0, ws.ptr, sort_bytes(n)))
        ctx.synchronize()
        want = np.bincount(np.arange(n) % 16, minlength=16).astype(np.float32)
        np.testing.assert_array_equal(out.download(np.float32, 16), want)
    finally:
        ctx.close()


def test_values_are_read_at_large_logical_positions():
    """hmr_test_index_value: the second step of a position check alone, at logical positions as large as a shape
    allows (below 2^63) in two-element views with zero strides; the kernel computes offsets in 64 bits
    (ref: src/backend/rocm/tests.rs:1213-1261, the same five cases)."""
    import ctypes

    from homura_amd import capi

    ctx = capi.Context(0)
    try:
        for np_dtype, code in ((np.int64, capi.I64), (np.int32, capi.I32)):
            base = ctx.upload(np.array([11, 22], dtype=np_dtype))
            cases = [([2, 1 << 60], [1, 0], 1 << 60, 22), ([2, 1 << 60], [1, 0], (1 << 60) - 1, 11),
                     ([2, 1 << 60], [1, 0], (1 << 61) - 1, 22), ([1 << 62, 2], [0, 1], (1 << 63) - 1, 22),
                     ([1 << 62, 2], [0, 1], (1 << 63) - 2, 11)]
            for shape, strides, position, expected in cases:
                slots = ctx.upload(np.array([position, 0], dtype=np.uint64))
                desc = capi.make_desc(base.ptr, code, shape, strides)
                capi.check(capi.lib.hmr_test_index_value(ctx.handle, ctypes.byref(desc), slots.ptr))
                ctx.synchronize()
                assert list(slots.download(np.uint64, 2)) == [position, expected], (shape, position)
            # UINT64_MAX means "no position": nothing is written.
            slots = ctx.upload(np.array([2**64 - 1, 7], dtype=np.uint64))
            desc = capi.make_desc(base.ptr, code, [2], [1])
            capi.check(capi.lib.hmr_test_index_value(ctx.handle, ctypes.byref(desc), slots.ptr))
            ctx.synchronize()
            assert list(slots.download(np.uint64, 2)) == [2**64 - 1, 7]
        bad = capi.make_desc(base.ptr, capi.F32, [2], [1])
        assert capi.lib.hmr_test_index_value(ctx.handle, ctypes.byref(bad), slots.ptr) == capi.HMR_INVALID
        assert capi.lib.hmr_last_error().decode() == "index tensors must be I32 or I64"
    finally:
        ctx.close()


def test_a_sort_whose_histogram_table_needs_several_rounds_of_the_totals_scan():
    """34.6 M positions are 16 895 tiles of 2048 words, so the digit histogram has 4.3 M entries in 1056 chunks of
    4096: more than the 1024 totals one round of the last scan takes, which then carries over. Order-sensitive f64
    values into a few targets: a word out of place or out of order changes a sum."""
    n, size = 34_600_000, 300
    pattern = np.array([2.0 ** 53, 1.0, 1.0, -(2.0 ** 53)])
    src = tensor(np.tile(pattern, n // 4), DT.F64)
    picks = tensor(random_positions(n, size, 91).astype(np.int32), DT.I32, [n])
    x = h.full([size], 0.0, DT.F64, "cpu")
    want = array(x.scatter_add(0, picks, src))
    got = array(x.to(GPU).scatter_add(0, picks.to(GPU), src.to(GPU)))
    wrong = np.flatnonzero(got.view(np.uint64) != want.view(np.uint64))
    assert wrong.size == 0, f"first difference at target {wrong[0]}: {got[wrong[0]]} != {want[wrong[0]]}"


def test_sorts_too_large_to_size_fail_before_any_kernel():
    """Indices and sources of 2^58 elements (views of one element with zero strides): the size of the sort's
    workspace is refused before anything is queued, and the tensor the call was made on is unchanged
    (ref: tests/rocm_index.rs:461-477; the reference words it "the workspace is too large", this library names
    its limit of 2^31 - 1 positions)."""
    n = 1 << 58
    x = tensor(np.arange(4, dtype=np.float32), DT.F32, [4], GPU)
    index = tensor(np.array([1], dtype=np.int64), DT.I64, [1], GPU).expand([n])
    src = tensor(np.ones(1, dtype=np.float32), DT.F32, [1], GPU).expand([n])
    for call, message in ((lambda: x.index_add(0, index, src), "index_add: more than 2^31 - 1 positions"),
                          (lambda: x.scatter_add(0, index, src), "scatter_add: more than 2^31 - 1 positions")):
        with pytest.raises(h.HomuraError) as e:
            call()
        assert message in str(e.value), str(e.value)
    assert array(x).tolist() == [0.0, 1.0, 2.0, 3.0]


def test_zero_dimensional_gpu_indices_select():
    """A zero-dimensional integer tensor on the GPU selects like an integer (its value is read back); out of range,
    the CPU's message (ref: tests/rocm_index.rs:577-589)."""
    x = tensor(np.arange(12, dtype=np.float32), DT.F32, [3, 4])
    g = x.to(GPU)
    for i in (2, -1):
        zero_dim = tensor(np.array([i], dtype=np.int64), DT.I64, [])
        assert_same(g.index_tensors([zero_dim.to(GPU)]), x.index_tensors([zero_dim]), f"x[{i}]")
    bad = tensor(np.array([3], dtype=np.int64), DT.I64, [])
    with pytest.raises(h.HomuraError) as c:
        x.index_tensors([bad])
    with pytest.raises(h.HomuraError) as e:
        g.index_tensors([bad.to(GPU)])
    assert str(e.value) == str(c.value)


@pytest.mark.parametrize("seed", range(6))
def test_random_gathers_and_scatter_adds_around_the_line_kernels_limits(seed):
    """gather and scatter_add along a random dimension of random shapes whose line counts, line lengths and numbers of
    positions straddle what the per-line kernels accept (128 lines, 64 to 2048 positions, 64 KiB of line), with
    contiguous and permuted operands, I32 and I64 positions, repeated targets in every density: the CPU's bits."""
    rng = np.random.default_rng(0x1D0000 + seed)
    for case in range(12):
        dtype = [DT.F32, DT.BF16, DT.I64, DT.F64, DT.U8][int(rng.integers(0, 5))]
        lines = int(rng.choice([1, 7, 127, 128, 129, 300]))
        length = int(rng.choice([5, 63, 64, 100, 1000, 2048, 4096, 20000]))
        count = int(rng.choice([1, 63, 64, 65, 500, 2047, 2048, 2049]))
        if lines * max(length, count) > 3000000:
            lines = 128
        dim = int(rng.integers(0, 2))
        shape = [lines, length] if dim == 1 else [length, lines]
        ishape = [lines, count] if dim == 1 else [count, lines]
        what = f"seed {seed} case {case}: {dtype} {shape} dim {dim}, {count} positions a line"
        x = tensor(values(dtype, lines * length, 500 + case), dtype, shape)
        if rng.integers(0, 3) == 0:   # the other dimension contiguous
            x = x.transpose(0, 1).contiguous().transpose(0, 1)
        spread = int(rng.choice([length, max(1, length // 50), 1 + length // 3]))   # few targets: long runs of repeats
        picks = (words(600 + 31 * seed + case, lines * count) % np.uint64(spread)).astype(np.int64)
        index = ints(picks, ishape, DT.I32 if rng.integers(0, 2) else DT.I64)
        g = x.to(GPU)
        assert_same(g.gather(dim, index.to(GPU)), x.gather(dim, index), f"gather {what}")
        src = tensor(values(dtype, lines * count, 700 + case), dtype, ishape)
        assert_bitwise(g.scatter_add(dim, index.to(GPU), src.to(GPU)), x.scatter_add(dim, index, src), f"scatter_add {what}")


def test_a_contiguous_index_off_the_16_byte_boundary_is_checked_like_any_other():
    """An index that is one contiguous run starting 1 to 3 elements into its buffer (its head lies before the first
    16-byte boundary, its end may be ragged): the first position out of range is reported wherever it lies, with the
    CPU's message, and a valid index selects the CPU's rows."""
    x = tensor(values(DT.F32, 50 * 3, 9), DT.F32, [50, 3])
    g = x.to(GPU)
    for dtype in (DT.I32, DT.I64):
        for offset in (1, 2, 3):
            for n in (70001, 65537 + offset):
                picks = random_positions(n + offset, 50, 10 * offset + n % 7)
                for bad_at in (None, 0, 1, 2, n // 2, n - 2, n - 1):
                    v = picks.copy()
                    if bad_at is not None:
                        v[offset + bad_at] = 50 + bad_at % 5
                        v[min(offset + bad_at + 3, n + offset - 1)] = -7 if bad_at % 2 else 99   # a later one must not win
                    index = ints(v, [n + offset], dtype).narrow(0, offset, n)
                    what = f"{dtype} offset {offset} n {n} bad at {bad_at}"
                    if bad_at is None:
                        assert_same(g.index_select(0, index.to(GPU)), x.index_select(0, index), what)
                        continue
                    with pytest.raises(h.HomuraError) as c:
                        x.index_select(0, index)
                    with pytest.raises(h.HomuraError) as e:
                        g.index_select(0, index.to(GPU))
                    assert str(e.value) == str(c.value), what


def test_the_first_bad_position_is_found_at_every_index_length():
    """Index lengths on both sides of the limits at which the position check changes form (one workgroup up to 16 384
    positions, a grid that meets at a counter beyond; whole 16-byte vectors or a ragged end), contiguous and every
    other element of a longer buffer: a bad value at the front, in the middle and at the very end, with a later bad
    value behind it that must not win, gives the CPU's message; a valid index the CPU's rows. Two checks in a row on
    one context also show that the counters of the first are back at rest."""
    x = tensor(values(DT.F32, 40 * 2, 11), DT.F32, [40, 2])
    g = x.to(GPU)
    lengths = (1, 2, 63, 64, 1023, 1024, 1025, 8191, 8192, 8193, 16383, 16384, 16385, 16400, 40000, 262147)
    for dtype in (DT.I32, DT.I64):
        for n in lengths:
            for strided in (False, True):
                picks = random_positions(n * (2 if strided else 1), 40, n % 13 + (7 if strided else 0))
                for bad_at in (None, 0, n // 2, n - 1):
                    v = picks.copy()
                    step = 2 if strided else 1
                    if bad_at is not None:
                        v[bad_at * step] = 40 + bad_at % 3
                        if bad_at + 1 < n:
                            v[(n - 1) * step] = -9   # a later one must not win
                    whole = ints(v, [len(v)], dtype)
                    view = (lambda t: t.reshape([n, 2]).select(1, 0)) if strided else (lambda t: t)   # a view made on the device
                    what = f"{dtype} n {n} strided {strided} bad at {bad_at}"
                    if bad_at is None:
                        assert_same(g.index_select(0, view(whole.to(GPU))), x.index_select(0, view(whole)), what)
                        continue
                    with pytest.raises(h.HomuraError) as c:
                        x.index_select(0, view(whole))
                    with pytest.raises(h.HomuraError) as e:
                        g.index_select(0, view(whole.to(GPU)))
                    assert str(e.value) == str(c.value), what
