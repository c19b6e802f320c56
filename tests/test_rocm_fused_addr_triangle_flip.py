"""hmr_fused, hmr_addr, hmr_triangle and hmr_flip on the GPU against the CPU oracle, through the host layer and
through the C ABI directly. All four are bit-exact: a fused step is IEEE arithmetic with the FMAs where the CPU has
them (ref: src/backend/cpu/mod.rs:509-569), addr rounds every step to the dtype (ref: src/backend/cpu/linalg.rs:
224-388, tests/gemm_writeback.rs:301-375), the other two move bits. Modelled on ref: src/backend/rocm/tests.rs:886-935
(fused_steps_match_the_cpu) and tests/rocm_elementwise.rs:674-718 (triangles_are_bitwise, flips_are_bitwise)."""
from ctypes import byref

import numpy as np
import pytest

from homura_amd import capi
from tests import oracle
from tests.support import (DT, DTYPES, FLOATS, GPU, NP, array, assert_bitwise, bits, from_f64, h, large_layouts, layouts,
                           mixed_floats, tensor, values)

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())
L = capi.lib

COEFFICIENTS = [0.1, -0.3, 0.49999, 0.5, 0.9, 1.0 + 1e-4, -1.7, 1.0 / 3.0, 1e-30]
STEPS = {"scaled_add": lambda a, b, c, v: h.scaled_add(a, b, v), "lerp": lambda a, b, c, v: h.lerp_step(a, b, v),
         "addcmul": lambda a, b, c, v: h.addcmul_step(a, b, c, v), "addcdiv": lambda a, b, c, v: h.addcdiv_step(a, b, c, v)}


@pytest.mark.parametrize("dtype", FLOATS)
def test_fused_steps_match_the_cpu(dtype):
    a, b, c = (mixed_floats(dtype, 1031, seed) for seed in (2, 3, 4))
    ag, bg, cg = (t.to(GPU) for t in (a, b, c))
    for v in COEFFICIENTS:
        for name, f in STEPS.items():
            assert_bitwise(f(ag, bg, cg, v), f(a, b, c, v), f"{dtype} {name} {v}")


@pytest.mark.parametrize("dtype", FLOATS)
def test_fused_steps_on_special_values_and_random_bits(dtype):
    """Infinities, NaNs, signed zeros, subnormals and arbitrary bit patterns in every operand position."""
    n = 4099
    a, b, c = (tensor(values(dtype, n, seed), dtype) for seed in (11, 12, 13))
    # Rotate so that special values meet ordinary ones, not only each other.
    b = tensor(np.roll(array(b), 7), dtype)
    c = tensor(np.roll(array(c), 19), dtype)
    ag, bg, cg = (t.to(GPU) for t in (a, b, c))
    for v in (0.25, -0.75, 3.0, 0.0, float("inf"), float("nan")):
        for name, f in STEPS.items():
            assert_bitwise(f(ag, bg, cg, v), f(a, b, c, v), f"{dtype} {name} {v}")


def test_fused_steps_on_every_layout_and_on_large_tensors():
    for dtype in FLOATS:
        for p in layouts(dtype, 60):
            for name, f in STEPS.items():
                what = f"{dtype} {name} {p.name}"
                # The same view in every position, then a contiguous partner.
                assert_bitwise(f(p.gpu, p.gpu, p.gpu, 0.3), f(p.cpu, p.cpu, p.cpu, 0.3), what)
                q = p.cpu.mul(2).contiguous()
                assert_bitwise(f(p.gpu, q.to(GPU), p.gpu, -0.7), f(p.cpu, q, p.cpu, -0.7), what + " mixed")
    for dtype in (DT.BF16, DT.F32):
        for p in large_layouts(dtype, 61):
            for name, f in STEPS.items():
                assert_bitwise(f(p.gpu, p.gpu, p.gpu, 0.6), f(p.cpu, p.cpu, p.cpu, 0.6), f"{dtype} {name} {p.name}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_addr_matches_the_cpu(dtype):
    from tests.test_oracle_kats import addr_cases
    checked = 0
    for (what, inp, v1, v2, beta, alpha), (_, ginp, g1, g2, _, _) in zip(addr_cases(dtype), addr_cases(dtype, GPU)):
        assert_bitwise(ginp.addr(g1, g2, beta, alpha), inp.addr(v1, v2, beta, alpha), what)
        checked += 1
    assert checked >= 24


def test_addr_of_sizes_that_vectorise_and_of_sizes_that_do_not():
    for dtype, beta, alpha in ((DT.BF16, 0.5, -1.5), (DT.F32, 1, 0.1), (DT.F64, 0, 2.0), (DT.I16, 3, -1), (DT.U8, 1, 2),
                               (DT.Bool, True, True)):
        for n, m in ((1031, 257), (64, 4096), (1, 1), (3, 0), (2048, 2048)):
            v1 = tensor(values(dtype, n, 71), dtype)
            v2 = tensor(values(dtype, m, 72), dtype)
            for inp in (tensor(values(dtype, n * m, 73), dtype).reshape([n, m]), tensor(values(dtype, m, 74), dtype)):
                got = inp.to(GPU).addr(v1.to(GPU), v2.to(GPU), beta, alpha)
                assert_bitwise(got, inp.addr(v1, v2, beta, alpha), f"{dtype} [{n}, {m}] input {inp.shape}")


def test_triangles_are_bitwise():
    checked = 0
    for dtype in DTYPES:
        for p in layouts(dtype, 40):
            if len(p.cpu.shape) < 2:
                continue
            for diagonal in (-3, -1, 0, 1, 2, 300, -(1 << 62), (1 << 62)):
                what = f"{dtype} {p.name} diagonal {diagonal}"
                assert_bitwise(p.gpu.triu(diagonal), p.cpu.triu(diagonal), "triu " + what)
                assert_bitwise(p.gpu.tril(diagonal), p.cpu.tril(diagonal), "tril " + what)
                checked += 2
    assert checked > 1000
    with pytest.raises(Exception, match="triu: input tensor must have at least 2 dimensions"):
        h.full([4], 1.0, DT.F32, GPU).triu(0)
    with pytest.raises(Exception, match="tril: input tensor must have at least 2 dimensions"):
        h.full([], 1.0, DT.F32, GPU).tril(0)


@pytest.mark.parametrize("dtype", [DT.U8, DT.BF16, DT.F32, DT.I64])
def test_triangles_of_matrices_that_vectorise(dtype):
    """Rows of whole 16-byte tiles, where tiles outside the triangle aren't read, next to rows that aren't."""
    for shape in ([3, 64, 128], [2, 2, 33, 48], [130, 256], [5, 7, 19], [1, 1, 16]):
        n = int(np.prod(shape))
        base = tensor(values(dtype, n, 41), dtype).reshape(shape)
        g = base.to(GPU)
        for diagonal in (-40, -1, 0, 1, 17, 100):
            what = f"{dtype} {shape} diagonal {diagonal}"
            assert_bitwise(g.triu(diagonal), base.triu(diagonal), "triu " + what)
            assert_bitwise(g.tril(diagonal), base.tril(diagonal), "tril " + what)
        # A transposed matrix (column stride != 1) and a batch of rows out of a wider buffer.
        assert_bitwise(g.transpose(-1, -2).triu(1), base.transpose(-1, -2).triu(1), f"transposed {dtype} {shape}")
        if shape[-1] >= 32:
            w = shape[-1] // 2
            assert_bitwise(g.narrow(-1, 16, w).tril(0), base.narrow(-1, 16, w).tril(0), f"narrowed {dtype} {shape}")


def test_flips_are_bitwise():
    checked = 0
    for dtype in DTYPES:
        for p in layouts(dtype, 50):
            n = len(p.cpu.shape)
            choices = [[d] for d in range(n)] + [list(range(n))]
            if n >= 2:
                choices += [[0, n - 1], [n - 2, n - 1]]
            for dims in choices:
                assert_bitwise(p.gpu.flip(dims), p.cpu.flip(dims), f"flip {dtype} {p.name} {dims}")
                checked += 1
    assert checked > 300
    for p in large_layouts(DT.I16, 51):
        assert_bitwise(p.gpu.flip([0]), p.cpu.flip([0]), p.name)
    # A flip is its own inverse, and flipping nothing copies.
    x = tensor(values(DT.F32, 2 * 3 * 1024, 52), DT.F32).reshape([2, 3, 1024]).to(GPU)
    assert (bits(x.flip([0, 2]).flip([2, 0])) == bits(x)).all()
    assert (bits(x.flip([])) == bits(x)).all()
    assert (bits(x.flip([1])) == bits(tensor(array(x)[:, ::-1, :].copy(), DT.F32))).all()


# ---- the C ABI directly ---------------------------------------------------------------------------------


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def desc(buf, dtype, sizes, strides=None, offset=0):
    if strides is None:
        strides, s = [], 1
        for n in reversed(sizes):
            strides.insert(0, s)
            s *= n
    return capi.make_desc(buf.ptr if buf is not None else 0, dtype, sizes, strides, offset)


def last_error():
    return L.hmr_last_error().decode()


def test_fused_through_the_c_abi_in_place_and_its_errors(ctx):
    n = 70001
    rng = np.random.default_rng(5)
    p, g = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    dp, dg = ctx.upload(p), ctx.upload(g)
    P, G = desc(dp, capi.F32, [n]), desc(dg, capi.F32, [n])
    lr = float(np.float32(-0.01))
    # p = fma(g, -lr, p), written over p.
    capi.check(L.hmr_fused(ctx.handle, 0, byref(P), byref(P), byref(G), None, lr, 0))
    ctx.synchronize()
    expected = (p.astype(np.float64) + g.astype(np.float64) * lr).astype(np.float32)  # exact product, one rounding
    np.testing.assert_array_equal(dp.download(np.float32, n), expected)
    # addcmul over its third operand: g = fma(c * p, g, p) with c * p rounded to f32 first.
    p1 = dp.download(np.float32, n)
    capi.check(L.hmr_fused(ctx.handle, 2, byref(G), byref(P), byref(P), byref(G), 0.5, 0))
    ctx.synchronize()
    cb = (np.float32(0.5) * p1).astype(np.float64)
    np.testing.assert_array_equal(dg.download(np.float32, n), (p1.astype(np.float64) + cb * g.astype(np.float64)).astype(np.float32))
    assert L.hmr_fused(ctx.handle, 4, byref(P), byref(P), byref(G), None, 1.0, 0) == capi.HMR_INVALID
    assert last_error() == "fused: unknown step"
    assert L.hmr_fused(ctx.handle, 2, byref(P), byref(P), byref(G), None, 1.0, 0) == capi.HMR_INVALID
    assert last_error() == "fused: the step needs three operands"
    assert L.hmr_fused(ctx.handle, 1, byref(P), byref(P), byref(G), byref(G), 1.0, 0) == capi.HMR_INVALID
    assert last_error() == "fused: the step takes two operands"
    di = ctx.upload(np.arange(n, dtype=np.int32))
    I = desc(di, capi.I32, [n])
    assert L.hmr_fused(ctx.handle, 0, byref(I), byref(I), byref(I), None, 1.0, 0) == capi.HMR_INVALID
    assert last_error() == "fused: unsupported dtype"
    assert L.hmr_fused(ctx.handle, 0, byref(P), byref(P), byref(I), None, 1.0, 0) == capi.HMR_INVALID
    assert last_error() == "fused: unsupported dtype"
    short = desc(dg, capi.F32, [n - 1])
    assert L.hmr_fused(ctx.handle, 0, byref(P), byref(P), byref(short), None, 1.0, 0) == capi.HMR_INVALID
    # Nothing above wrote anything.
    np.testing.assert_array_equal(dp.download(np.float32, n), expected)
    # No elements: nothing to do, whatever the pointers are.
    E = desc(None, capi.F32, [0, 4])
    capi.check(L.hmr_fused(ctx.handle, 3, byref(E), byref(E), byref(E), byref(E), 1.0, 0))


def test_addr_through_the_c_abi_and_its_errors(ctx):
    n, m = 300, 200
    rng = np.random.default_rng(9)
    v1, v2 = rng.standard_normal(n).astype(np.float32), rng.standard_normal(m).astype(np.float32)
    c = rng.standard_normal((n, m)).astype(np.float32)
    d1, d2, dc = ctx.upload(v1), ctx.upload(v2), ctx.upload(c)
    O = desc(dc, capi.F32, [n, m])
    V1, V2 = desc(d1, capi.F32, [n, m], [1, 0]), desc(d2, capi.F32, [n, m], [0, 1])
    alpha, beta = np.float32(0.75), np.float32(-2.0)
    # In place over the input: every step rounded to f32.
    capi.check(L.hmr_addr(ctx.handle, byref(O), byref(V1), byref(V2), byref(O), float(alpha), float(beta), 0, 0))
    ctx.synchronize()
    want = (c * beta) + (v1 * alpha)[:, None] * v2[None, :]
    np.testing.assert_array_equal(dc.download(np.float32, n * m).reshape(n, m), want)
    # beta == 0: the input isn't read and may be missing.
    capi.check(L.hmr_addr(ctx.handle, byref(O), byref(V1), byref(V2), None, 1.0, 0.0, 0, 0))
    ctx.synchronize()
    np.testing.assert_array_equal(dc.download(np.float32, n * m).reshape(n, m), v1[:, None] * v2[None, :])
    assert L.hmr_addr(ctx.handle, byref(O), byref(V1), byref(V2), None, 1.0, 1.0, 0, 0) == capi.HMR_INVALID
    assert last_error() == "addr: beta isn't zero but there is no input"
    flat = desc(dc, capi.F32, [n * m])
    assert L.hmr_addr(ctx.handle, byref(flat), byref(flat), byref(flat), None, 1.0, 0.0, 0, 0) == capi.HMR_INVALID
    assert last_error() == "addr: the output must have two dimensions"
    H = desc(d1, capi.F16, [n, m], [1, 0])
    assert L.hmr_addr(ctx.handle, byref(O), byref(H), byref(V2), None, 1.0, 0.0, 0, 0) == capi.HMR_INVALID
    assert last_error() == "addr: unsupported dtype"
    # Integers wrap in the element's width.
    a8, b8 = np.arange(-100, 100, dtype=np.int8), np.arange(-60, 68, dtype=np.int8)
    c8 = np.full((200, 128), 7, dtype=np.int8)
    da, db, dcc = ctx.upload(a8), ctx.upload(b8), ctx.upload(c8)
    O8 = desc(dcc, capi.I8, [200, 128])
    capi.check(L.hmr_addr(ctx.handle, byref(O8), byref(desc(da, capi.I8, [200, 128], [1, 0])),
                          byref(desc(db, capi.I8, [200, 128], [0, 1])), byref(O8), 0.0, 0.0, -3, 5))
    ctx.synchronize()
    want8 = (c8.astype(np.int64) * 5 + a8.astype(np.int64)[:, None] * b8.astype(np.int64)[None, :] * -3).astype(np.int8)
    np.testing.assert_array_equal(dcc.download(np.int8, 200 * 128).reshape(200, 128), want8)


def test_triangle_and_flip_through_the_c_abi_and_their_errors(ctx):
    rows, cols = 37, 64
    m = np.arange(2 * rows * cols, dtype=np.float32).reshape(2, rows, cols) + 1
    dm = ctx.upload(m)
    dout = ctx.upload(np.zeros_like(m))
    M, O = desc(dm, capi.F32, [2, rows, cols]), desc(dout, capi.F32, [2, rows, cols])
    capi.check(L.hmr_triangle(ctx.handle, byref(O), byref(M), 3, 1))
    ctx.synchronize()
    np.testing.assert_array_equal(dout.download(np.float32, m.size).reshape(m.shape), np.triu(m, 3))
    # In place, the lower triangle.
    capi.check(L.hmr_triangle(ctx.handle, byref(M), byref(M), -2, 0))
    ctx.synchronize()
    np.testing.assert_array_equal(dm.download(np.float32, m.size).reshape(m.shape), np.tril(m, -2))
    V = desc(dm, capi.F32, [rows * cols * 2])
    assert L.hmr_triangle(ctx.handle, byref(V), byref(V), 0, 1) == capi.HMR_INVALID
    assert last_error() == "triangle needs two dimensions"
    H = desc(dm, capi.F16, [2, rows, cols])
    assert L.hmr_triangle(ctx.handle, byref(O), byref(H), 0, 1) == capi.HMR_INVALID
    assert last_error() == "triangle: unsupported dtype"
    R = desc(dm, capi.F32, [2, rows, cols], [rows * cols, cols, -1], cols - 1)
    assert L.hmr_triangle(ctx.handle, byref(O), byref(R), 0, 1) == capi.HMR_INVALID
    # flip: the source read backwards along both matrix dimensions, from its last element.
    x = np.arange(rows * cols, dtype=np.int64).reshape(rows, cols)
    dx, dy = ctx.upload(x), ctx.upload(np.zeros_like(x))
    Y = desc(dy, capi.I64, [rows, cols])
    X = desc(dx, capi.I64, [rows, cols], [-cols, -1], rows * cols - 1)
    capi.check(L.hmr_flip(ctx.handle, byref(Y), byref(X)))
    ctx.synchronize()
    np.testing.assert_array_equal(dy.download(np.int64, x.size).reshape(x.shape), x[::-1, ::-1])
    # Only flip reads through negative strides, and only its source may have them.
    assert L.hmr_flip(ctx.handle, byref(X), byref(Y)) == capi.HMR_INVALID
    before = last_error()
    assert "negative" in before
    assert L.hmr_copy(ctx.handle, byref(Y), byref(X)) == capi.HMR_INVALID
    assert "negative" in last_error()
    assert L.hmr_unary(ctx.handle, capi.UNARY["neg"], byref(Y), byref(X)) == capi.HMR_INVALID
    np.testing.assert_array_equal(dy.download(np.int64, x.size).reshape(x.shape), x[::-1, ::-1])
