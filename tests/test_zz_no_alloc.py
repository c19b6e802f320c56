"""hmr_reduce_static: hmr_reduce for callers that cannot allocate (no workspace argument; the partial
results go to a block inside the library's code object). It has no counterpart in the reference; the
bar is the existing entry point's own output, bit for bit, on the same device buffers.

Two calls in a row share the block, the second with a smaller input: what the first left there must
not leak into the second. Collected last (the file name sorts after every other test file)."""
from ctypes import byref, c_int64

import numpy as np
import pytest

from homura_amd import capi
from tests.support import normal

pytestmark = pytest.mark.gpu
L = capi.lib
LIMIT = 8 * 1024 * 1024  # HMR_REDUCE_STATIC_BYTES


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def matrix_reduction(src, dtype, rows, cols, dim):
    """(kept, red, nout) of a reduction over dimension `dim` of a contiguous [rows, cols] matrix."""
    if dim == 0:
        return (capi.make_desc(src.ptr, dtype, [cols], [1]), capi.make_desc(src.ptr, dtype, [rows], [cols]), cols)
    if dim == 1:
        return (capi.make_desc(src.ptr, dtype, [rows], [cols]), capi.make_desc(src.ptr, dtype, [cols], [1]), rows)
    return (capi.make_desc(src.ptr, dtype, [], []), capi.make_desc(src.ptr, dtype, [rows * cols], [1]), 1)


def workspace_bytes(kept, red):
    need = c_int64(-1)
    capi.check(L.hmr_reduce_workspace(byref(kept), byref(red), 0, byref(need)))
    return need.value


def both_ways(ctx, src, dtype, np_dtype, rows, cols, dim, op):
    """The reduction through hmr_reduce (caller's workspace) and through hmr_reduce_static: raw output bits."""
    kept, red, nout = matrix_reduction(src, dtype, rows, cols, dim)
    need = workspace_bytes(kept, red)
    assert need <= LIMIT
    size = np.dtype(np_dtype).itemsize
    results = []
    for static in (False, True):
        out = ctx.malloc(nout * size)
        capi.check(L.hmr_memset(ctx.handle, out.ptr, 0xA5, nout * size))
        o = capi.make_desc(out.ptr, dtype, [nout] if dim in (0, 1) else [], [1] if dim in (0, 1) else [])
        if static:
            capi.check(L.hmr_reduce_static(ctx.handle, capi.REDUCE[op], byref(o), byref(kept), byref(red)))
        else:
            work = ctx.malloc(max(need, 1))
            capi.check(L.hmr_memset(ctx.handle, work.ptr, 0xFF, max(need, 1)))
            capi.check(L.hmr_reduce(ctx.handle, capi.REDUCE[op], byref(o), byref(kept), byref(red), work.ptr, need))
        ctx.synchronize()
        results.append(out.download(np.uint8, nout * size))
    return need, results


@pytest.mark.parametrize("op", ["sum", "mean", "max", "prod"])
def test_two_calls_in_a_row_match_the_entry_point_with_a_workspace(ctx, op):
    big_rows, big_cols = 8192, 1024
    values = normal(0x5A11 + len(op), big_rows * big_cols).astype(np.float32)
    if op == "prod":
        values = (1.0 + values * 1e-3).astype(np.float32)
    src = ctx.upload(values)
    staged = 0
    # The larger input first, then smaller ones over the same block: columns, a full reduction, rows.
    for rows, cols, dim in ((big_rows, big_cols, 0), (2048, 512, 0), (big_rows, big_cols, None), (1024, 96, None),
                            (64, 65536, 1), (300, 64, 0)):
        need, (with_workspace, with_block) = both_ways(ctx, src, capi.F32, np.float32, rows, cols, dim, op)
        staged += need > 0
        assert np.array_equal(with_workspace, with_block), (op, rows, cols, dim)
    assert staged >= 3, "the cases are meant to stage partial results"
    # Against a plain float64 fold too, so that two equal wrong answers do not pass.
    kept, red, nout = matrix_reduction(src, capi.F32, 2048, 512, 0)
    out = ctx.malloc(nout * 4)
    o = capi.make_desc(out.ptr, capi.F32, [nout], [1])
    capi.check(L.hmr_reduce_static(ctx.handle, capi.REDUCE[op], byref(o), byref(kept), byref(red)))
    ctx.synchronize()
    got = out.download(np.float32, nout).astype(np.float64)
    x = values[:2048 * 512].reshape(2048, 512).astype(np.float64)
    want = {"sum": x.sum(0), "mean": x.mean(0), "max": x.max(0), "prod": x.prod(0)}[op]
    np.testing.assert_allclose(got, want, rtol=3e-7, atol=1e-30)


def test_integer_sums_and_the_other_dtypes(ctx):
    rows, cols = 4096, 2048
    ints = (np.arange(rows * cols, dtype=np.int64) * 2654435761 % 2001 - 1000).astype(np.int32)
    src = ctx.upload(ints)
    for r, c, dim in ((rows, cols, 0), (1000, 256, 0), (rows, cols, None)):
        kept, red, nout = matrix_reduction(src, capi.I32, r, c, dim)
        shape, strides = ([nout], [1]) if dim is not None else ([], [])
        outs = []
        for static in (False, True):
            out = ctx.malloc(nout * 8)
            o = capi.make_desc(out.ptr, capi.I64, shape, strides)
            if static:
                capi.check(L.hmr_reduce_static(ctx.handle, capi.REDUCE["sum"], byref(o), byref(kept), byref(red)))
            else:
                need = workspace_bytes(kept, red)
                work = ctx.malloc(max(need, 1))
                capi.check(L.hmr_reduce(ctx.handle, capi.REDUCE["sum"], byref(o), byref(kept), byref(red), work.ptr, need))
            ctx.synchronize()
            outs.append(out.download(np.int64, nout))
        assert np.array_equal(outs[0], outs[1])
        x = ints[:r * c].reshape(r, c).astype(np.int64)
        assert np.array_equal(outs[1], x.sum(0) if dim == 0 else np.array([x.sum()]))


def test_a_plan_beyond_the_block_is_refused_and_queues_nothing(ctx):
    # Many one-byte columns: 64 slices of 32 768 partial sums of 16 bytes.
    rows, cols = 16384, 32768
    src = ctx.malloc(rows * cols)
    kept, red, nout = matrix_reduction(src, capi.I8, rows, cols, 0)
    need = workspace_bytes(kept, red)
    assert need > LIMIT, "this shape is meant to stage more than the block holds; pick a wider one if the plan changed"
    out = ctx.malloc(nout * 8)
    capi.check(L.hmr_memset(ctx.handle, out.ptr, 0x5C, nout * 8))
    o = capi.make_desc(out.ptr, capi.I64, [nout], [1])
    assert L.hmr_reduce_static(ctx.handle, capi.REDUCE["sum"], byref(o), byref(kept), byref(red)) == capi.HMR_INVALID
    message = L.hmr_last_error().decode()
    assert message.startswith("hmr_reduce_static: this reduction stages %d bytes" % need) and str(LIMIT) in message
    ctx.synchronize()
    assert (out.download(np.uint8, nout * 8) == 0x5C).all()
    # The same errors as hmr_reduce for a bad call.
    bad = capi.make_desc(out.ptr, capi.I64, [nout + 1], [1])
    assert L.hmr_reduce_static(ctx.handle, capi.REDUCE["sum"], byref(bad), byref(kept), byref(red)) == capi.HMR_INVALID
    assert L.hmr_last_error().decode() == "a reduction's output is not contiguous with its sizes"


def test_the_block_belongs_to_one_context_per_gpu(ctx):
    """A second context of the same GPU (another stream) is refused while the first one holds the block, with
    nothing queued, and takes it over once the first is destroyed; a null context is refused, not followed."""
    rows, cols = 4096, 2048
    src = ctx.upload(np.arange(rows * cols, dtype=np.int32) % 7)
    kept, red, nout = matrix_reduction(src, capi.I32, rows, cols, 0)
    assert workspace_bytes(kept, red) > 0, "this shape is meant to stage partial results"
    out = ctx.malloc(nout * 8)
    o = capi.make_desc(out.ptr, capi.I64, [nout], [1])
    capi.check(L.hmr_reduce_static(ctx.handle, capi.REDUCE["sum"], byref(o), byref(kept), byref(red)))
    ctx.synchronize()
    want = out.download(np.int64, nout)
    other = capi.Context(0)
    try:
        capi.check(L.hmr_memset(other.handle, out.ptr, 0x5C, nout * 8))
        other.synchronize()
        assert L.hmr_reduce_static(other.handle, capi.REDUCE["sum"], byref(o), byref(kept), byref(red)) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == ("hmr_reduce_static: the static block of rocm:0 is in use by another context; "
                                               "call hmr_reduce with a workspace")
        other.synchronize()
        assert (out.download(np.uint8, nout * 8) == 0x5C).all()
        # A reduction that stages nothing needs no block and runs on any context.
        kept1, red1, nout1 = matrix_reduction(src, capi.I32, 64, 512, 1)
        assert workspace_bytes(kept1, red1) == 0
        small = capi.make_desc(out.ptr, capi.I64, [nout1], [1])
        capi.check(L.hmr_reduce_static(other.handle, capi.REDUCE["sum"], byref(small), byref(kept1), byref(red1)))
        other.synchronize()
    finally:
        other.close()
    assert L.hmr_reduce_static(None, capi.REDUCE["sum"], byref(o), byref(kept), byref(red)) == capi.HMR_INVALID
    assert L.hmr_last_error().decode() == "hmr_reduce_static: null context"
    # The owner is still the owner.
    capi.check(L.hmr_reduce_static(ctx.handle, capi.REDUCE["sum"], byref(o), byref(kept), byref(red)))
    ctx.synchronize()
    assert np.array_equal(out.download(np.int64, nout), want)
