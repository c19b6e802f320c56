"""The C ABI called directly (ctypes, no host layer): operand contract, in-place operands, empty
operands, error behaviour and the reduction / softmax entry points with caller-provided workspaces
(ref: csrc/homura_rocm.h:26-40, 148-155, 297-346, 612-626; csrc/kernel.hpp:62-154;
src/backend/rocm/tests.rs)."""
import ctypes
from ctypes import byref

import numpy as np
import pytest

from homura_amd import capi
from tests import oracle
from tests.support import DT, array, from_f64, h, normal, tensor, to_f64

pytestmark = pytest.mark.gpu
L = capi.lib


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def last_error():
    return L.hmr_last_error().decode()


def desc(buf, dtype, sizes, strides=None, offset=0):
    if strides is None:
        strides, s = [], 1
        for n in reversed(sizes):
            strides.insert(0, s)
            s *= n
    return capi.make_desc(buf.ptr if buf is not None else 0, dtype, sizes, strides, offset)


def test_in_place_operands(ctx):
    n = 100003
    a = np.linspace(-4, 4, n).astype(np.float32)
    b = np.linspace(1, 2, n).astype(np.float32)
    da, db = ctx.upload(a), ctx.upload(b)
    A, B = desc(da, capi.F32, [n]), desc(db, capi.F32, [n])
    capi.check(L.hmr_binary(ctx.handle, capi.BINARY["mul"], byref(A), byref(A), byref(B)))      # a *= b
    capi.check(L.hmr_binary(ctx.handle, capi.BINARY["sub"], byref(B), byref(A), byref(B)))      # b = a - b
    capi.check(L.hmr_unary(ctx.handle, capi.UNARY["neg"], byref(A), byref(A)))                  # a = -a
    capi.check(L.hmr_binary_scalar(ctx.handle, capi.BINARY["mul"], byref(A), byref(A), 0.5, 0))
    ctx.synchronize()
    prod = a * b
    np.testing.assert_array_equal(db.download(np.float32, n), prod - b)
    np.testing.assert_array_equal(da.download(np.float32, n), -prod * np.float32(0.5))
    # where with the output aliasing a branch.
    cond = (np.arange(n) % 3 == 0).astype(np.uint8)
    dc = ctx.upload(cond)
    C = desc(dc, capi.BOOL, [n])
    capi.check(L.hmr_where(ctx.handle, byref(A), byref(C), byref(A), byref(B)))
    ctx.synchronize()
    np.testing.assert_array_equal(da.download(np.float32, n), np.where(cond != 0, -prod * np.float32(0.5), prod - b))


def test_empty_operands_queue_nothing(ctx):
    z = desc(None, capi.F32, [0, 5])
    assert L.hmr_unary(ctx.handle, capi.UNARY["exp"], byref(z), byref(z)) == capi.HMR_OK
    assert L.hmr_binary(ctx.handle, capi.BINARY["add"], byref(z), byref(z), byref(z)) == capi.HMR_OK
    assert L.hmr_copy(ctx.handle, byref(z), byref(z)) == capi.HMR_OK
    assert L.hmr_fill(ctx.handle, byref(z), 0) == capi.HMR_OK
    rows = desc(None, capi.F32, [0])
    assert L.hmr_softmax(ctx.handle, byref(rows), byref(rows), 8, 1, 1, 0, None, 0) == capi.HMR_OK
    assert L.hmr_softmax(ctx.handle, byref(desc(None, capi.F32, [4], [0])), byref(desc(None, capi.F32, [4], [0])), 0, 1, 1, 0,
                         None, 0) == capi.HMR_OK


def test_invalid_descriptions_are_refused_with_a_message(ctx):
    buf = ctx.malloc(4096)
    good = desc(buf, capi.F32, [16])
    bad_dtype = desc(buf, 10, [16])
    assert L.hmr_unary(ctx.handle, 0, byref(good), byref(bad_dtype)) == capi.HMR_INVALID
    assert last_error() == "invalid dtype 10"
    many = desc(buf, capi.F32, [16])
    many.ndim = 26
    assert L.hmr_unary(ctx.handle, 0, byref(many), byref(many)) == capi.HMR_INVALID
    assert last_error() == "invalid number of dimensions 26"
    neg = desc(buf, capi.F32, [-1])
    assert L.hmr_copy(ctx.handle, byref(neg), byref(neg)) == capi.HMR_INVALID and last_error() == "negative size"
    back = desc(buf, capi.F32, [16], [-1], 15)
    assert L.hmr_copy(ctx.handle, byref(good), byref(back)) == capi.HMR_INVALID and last_error() == "negative stride"
    other = desc(buf, capi.F32, [4, 4])
    assert L.hmr_binary(ctx.handle, 0, byref(good), byref(good), byref(other)) == capi.HMR_INVALID
    assert last_error() == "kernel operands have different sizes"
    # Unsupported op / dtype combinations: "<entry>: unsupported dtype".
    ints = desc(buf, capi.I32, [16])
    assert L.hmr_unary(ctx.handle, capi.UNARY["exp"], byref(ints), byref(ints)) == capi.HMR_INVALID
    assert last_error() == "unary: unsupported dtype"
    assert L.hmr_unary(ctx.handle, 99, byref(good), byref(good)) == capi.HMR_INVALID
    assert L.hmr_binary(ctx.handle, capi.BINARY["bitwise_and"], byref(good), byref(good), byref(good)) == capi.HMR_INVALID
    assert last_error() == "binary: unsupported dtype"
    boolean = desc(buf, capi.BOOL, [16])
    assert L.hmr_binary(ctx.handle, capi.BINARY["add"], byref(boolean), byref(good), byref(good)) == capi.HMR_INVALID
    assert L.hmr_where(ctx.handle, byref(good), byref(good), byref(good), byref(good)) == capi.HMR_INVALID  # cond not bool
    # A refused call leaves the context usable, and a good call clears nothing it should not.
    assert L.hmr_unary(ctx.handle, capi.UNARY["neg"], byref(good), byref(good)) == capi.HMR_OK
    ctx.synchronize()


def test_injected_failures_queue_nothing(ctx):
    n = 1 << 12
    src = ctx.upload(np.ones(n, dtype=np.float32))
    dst = ctx.upload(np.full(n, 7, dtype=np.float32))
    S, D = desc(src, capi.F32, [n]), desc(dst, capi.F32, [n])
    L.hmr_test_fail_data(1, 1)
    assert L.hmr_unary(ctx.handle, capi.UNARY["neg"], byref(D), byref(S)) == capi.HMR_OUT_OF_MEMORY
    L.hmr_test_fail_data(1, 0)
    assert L.hmr_copy(ctx.handle, byref(D), byref(S)) == capi.HMR_HIP_ERROR
    assert "hipGetLastError()" in last_error()
    ctx.synchronize()
    np.testing.assert_array_equal(dst.download(np.float32, n), np.full(n, 7, dtype=np.float32))
    assert L.hmr_copy(ctx.handle, byref(D), byref(S)) == capi.HMR_OK
    ctx.synchronize()
    np.testing.assert_array_equal(dst.download(np.float32, n), np.ones(n, dtype=np.float32))


def test_the_callers_current_device_is_restored(ctx):
    dev = ctypes.c_int32(-1)
    capi.check(L.hmr_test_current_device(byref(dev)))
    before = dev.value
    buf = ctx.malloc(64)
    d = desc(buf, capi.F32, [16])
    capi.check(L.hmr_fill(ctx.handle, byref(d), 0))
    capi.check(L.hmr_test_current_device(byref(dev)))
    assert dev.value == before


def reduce_through_the_abi(ctx, op, x, kept_dims, red_dims, out_dtype=None, var=None, arg=None):
    """x: numpy array (storage of dtype code `code`); returns the downloaded output(s)."""
    arr, code = x
    strides = [s // arr.itemsize for s in arr.strides]
    src = ctx.upload(arr)
    kept = capi.make_desc(src.ptr, code, [arr.shape[d] for d in kept_dims], [strides[d] for d in kept_dims])
    red = capi.make_desc(src.ptr, code, [arr.shape[d] for d in red_dims], [strides[d] for d in red_dims])
    nout = int(np.prod([arr.shape[d] for d in kept_dims])) if kept_dims else 1
    need = ctypes.c_int64(-1)
    capi.check(L.hmr_reduce_workspace(byref(kept), byref(red), 1 if var is not None else 0, byref(need)))
    ws = ctx.malloc(max(need.value, 1))
    out_code = code if out_dtype is None else out_dtype
    out = ctx.malloc(max(nout * capi.DTYPE_SIZE[out_code], 1))
    O = desc(out, out_code, [arr.shape[d] for d in kept_dims])
    if var is not None:
        capi.check(L.hmr_var(ctx.handle, byref(O), byref(kept), byref(red), float(var), 0, ws.ptr, need.value))
    elif arg is not None:
        idx = ctx.malloc(max(nout * 8, 1))
        I = desc(idx, capi.I64, [arr.shape[d] for d in kept_dims])
        capi.check(L.hmr_arg_reduce(ctx.handle, byref(O), byref(I), byref(kept), byref(red), int(arg), ws.ptr, need.value))
        ctx.synchronize()
        return out.download(capi.DTYPE_NP[out_code], nout), idx.download(np.int64, nout), need.value
    else:
        capi.check(L.hmr_reduce(ctx.handle, capi.REDUCE[op], byref(O), byref(kept), byref(red), ws.ptr, need.value))
    ctx.synchronize()
    return out.download(capi.DTYPE_NP[out_code], nout), need.value


def test_reductions_with_caller_workspaces(ctx):
    h.register_cpu_backend(oracle.backend_address())
    rows, cols = 96, 20000
    x = normal(5, rows * cols).astype(np.float32).reshape(rows, cols)
    cpu = tensor(x, DT.F32, [rows, cols])
    # Few long rows: the plan cuts them and needs a workspace.
    got, need = reduce_through_the_abi(ctx, "sum", (x, capi.F32), [0], [1])
    assert need > 0
    want = array(cpu.sum_dim(-1, False)).reshape(-1)
    assert np.all(np.abs(got.astype(np.float64) - want) <= np.spacing(np.abs(want)))
    # Column direction: kept stride 1, reduced stride `cols`.
    got, _ = reduce_through_the_abi(ctx, "mean", (x, capi.F32), [1], [0])
    want = array(cpu.mean_dim(0, False)).reshape(-1)
    assert np.all(np.abs(got.astype(np.float64) - want) <= np.spacing(np.abs(want)))
    got, _ = reduce_through_the_abi(ctx, None, (x, capi.F32), [0], [1], var=1)
    want = array(cpu.var_dim(-1, 1, False)).reshape(-1)
    assert np.all(np.abs(got.astype(np.float64) - want) <= np.spacing(np.abs(want)))
    vals, idx, _ = reduce_through_the_abi(ctx, None, (x, capi.F32), [0], [1], arg=1)
    np.testing.assert_array_equal(idx, x.argmax(axis=1))
    np.testing.assert_array_equal(vals, x.max(axis=1))
    # Everything into one output.
    got, need = reduce_through_the_abi(ctx, "sum", (x, capi.F32), [], [0, 1])
    want = array(cpu.sum()).reshape(-1)
    assert abs(float(got[0]) - float(want[0])) <= np.spacing(abs(want[0]))
    # Integers: exact, written as I64.
    xi = (np.arange(rows * cols, dtype=np.int64).reshape(rows, cols) * 2654435761 % 1000 - 500).astype(np.int32)
    got, _ = reduce_through_the_abi(ctx, "sum", (xi, capi.I32), [0], [1], out_dtype=capi.I64)
    np.testing.assert_array_equal(got, xi.astype(np.int64).sum(axis=1))


def test_a_workspace_that_is_too_small_is_refused(ctx):
    rows, cols = 4, 1 << 20
    src = ctx.malloc(rows * cols * 4)
    capi.check(L.hmr_memset(ctx.handle, src.ptr, 0, rows * cols * 4))
    kept = capi.make_desc(src.ptr, capi.F32, [rows], [cols])
    red = capi.make_desc(src.ptr, capi.F32, [cols], [1])
    need = ctypes.c_int64(0)
    capi.check(L.hmr_reduce_workspace(byref(kept), byref(red), 0, byref(need)))
    assert need.value > 0
    out = ctx.malloc(rows * 4)
    capi.check(L.hmr_memset(ctx.handle, out.ptr, 0x7F, rows * 4))
    O = desc(out, capi.F32, [rows])
    ws = ctx.malloc(need.value)
    assert L.hmr_reduce(ctx.handle, 0, byref(O), byref(kept), byref(red), ws.ptr, need.value - 1) == capi.HMR_INVALID
    assert "workspace" in last_error()
    assert L.hmr_reduce(ctx.handle, 0, byref(O), byref(kept), byref(red), None, 0) == capi.HMR_INVALID
    ctx.synchronize()
    assert (out.download(np.uint32, rows) == 0x7F7F7F7F).all(), "a refused call must not write"
    # Reductions check their operands too.
    wrong = desc(out, capi.F32, [rows + 1])
    assert L.hmr_reduce(ctx.handle, 0, byref(wrong), byref(kept), byref(red), ws.ptr, need.value) == capi.HMR_INVALID
    as_int = desc(out, capi.I64, [rows])
    assert L.hmr_reduce(ctx.handle, 0, byref(as_int), byref(kept), byref(red), ws.ptr, need.value) == capi.HMR_INVALID
    empty_red = capi.make_desc(src.ptr, capi.F32, [0], [1])
    assert L.hmr_reduce(ctx.handle, capi.REDUCE["max"], byref(O), byref(kept), byref(empty_red), None, 0) == capi.HMR_INVALID


def test_softmax_rows_with_strides(ctx):
    """Rows that are columns of a matrix (element stride = row length) and rows inside a wider buffer."""
    h.register_cpu_backend(oracle.backend_address())
    r, c = 300, 77
    x = normal(6, r * c, 0.0, 3.0).astype(np.float32).reshape(r, c)
    src = ctx.upload(x)
    out = ctx.malloc(r * c * 4)
    # softmax along dim 0: c rows of r elements, element stride c, row stride 1.
    rows_s = capi.make_desc(src.ptr, capi.F32, [c], [1])
    rows_o = capi.make_desc(out.ptr, capi.F32, [c], [1])
    need = ctypes.c_int64(-1)
    capi.check(L.hmr_softmax_workspace(byref(rows_s), r, c, byref(need)))
    ws = ctx.malloc(max(need.value, 1))
    for log in (0, 1):
        capi.check(L.hmr_softmax(ctx.handle, byref(rows_o), byref(rows_s), r, c, c, log, ws.ptr, need.value))
        ctx.synchronize()
        got = out.download(np.float32, r * c).reshape(r, c)
        cpu = tensor(x, DT.F32, [r, c])
        want = array(cpu.log_softmax(0) if log else cpu.softmax(0)).reshape(r, c)
        assert np.all(np.abs(got.astype(np.float64) - want) <= np.spacing(np.maximum(np.abs(want), np.abs(got))))
    bad = capi.make_desc(src.ptr, capi.I32, [c], [1])
    assert L.hmr_softmax(ctx.handle, byref(rows_o), byref(bad), r, c, c, 0, None, 0) == capi.HMR_INVALID
