"""hmr_copy / hmr_fill on the GPU against the CPU oracle, byte for byte, NaN payloads included
(ref: tests/rocm_copy.rs:12-130, src/dtype.rs:186-277, csrc/elem.hpp:276-287)."""
import numpy as np
import pytest

from tests import oracle
from tests.support import DT, DTYPES, GPU, NP, array, assert_same, bits, h, large_layouts, layouts, tensor, values, words

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())


def test_every_conversion_matches_the_cpu_in_every_layout():
    for k, src in enumerate(DTYPES):
        for pair in layouts(src, 10 + k):
            assert_same(pair.gpu.contiguous(), pair.cpu.contiguous(), f"{src} {pair.name} copied")
            for dst in DTYPES:
                what = f"{src} -> {dst}, {pair.name}"
                gpu, cpu = pair.gpu.to(dst), pair.cpu.to(dst)
                assert_same(gpu, cpu, what)
                if dst != src:
                    assert gpu.is_contiguous(), what


def test_nan_payloads_convert_like_the_cpu():
    n = 1 << 16
    r, r32, r16, rb16 = (words(99 + k, n) for k in range(4))
    f64s = ((r & np.uint64(0x800FFFFFFFFFFFFF)) | np.uint64(0x7FF0000000000001)).view(np.float64)
    f32s = ((r32.astype(np.uint32) & np.uint32(0x807FFFFF)) | np.uint32(0x7F800001)).view(np.float32)
    f16s = (r16.astype(np.uint16) & np.uint16(0x83FF)) | np.uint16(0x7C01)
    bf16s = (rb16.astype(np.uint16) & np.uint16(0x807F)) | np.uint16(0x7F81)
    for arr, dtype in ((f64s, DT.F64), (f32s, DT.F32), (f16s, DT.F16), (bf16s, DT.BF16)):
        cpu = tensor(arr, dtype, [n])
        gpu = cpu.to(GPU)
        for dst in DTYPES:
            assert_same(gpu.to(dst), cpu.to(dst), f"NaNs {dtype} -> {dst}")


def test_conversions_of_large_tensors_take_several_grid_rounds():
    for src, dst in ((DT.F32, DT.BF16), (DT.F64, DT.F16), (DT.I64, DT.F32), (DT.U8, DT.U8), (DT.BF16, DT.F32)):
        for pair in large_layouts(src, 7):
            assert_same(pair.gpu.to(dst), pair.cpu.to(dst), f"{src} -> {dst}, {pair.name}")


def test_conversion_counterexamples():
    def f(v, dtype):
        return array(tensor(np.array([v], dtype=np.float32), DT.F32, [1], GPU).to(dtype)).item()

    assert f(300.0, DT.U8) == 44
    assert f(-129.9, DT.I8) == 127
    assert f(np.inf, DT.I32) == -1
    assert f(np.inf, DT.I64) == np.iinfo(np.int64).max
    assert f(1e30, DT.I16) == -1
    assert f(np.nan, DT.I32) == 0
    assert array(tensor(np.array([0xC100], dtype=np.uint16), DT.F16, [1], GPU).to(DT.U8)).item() == 254   # -2.5

    def g(v, dtype):
        return array(tensor(np.array([v], dtype=np.float64), DT.F64, [1], GPU).to(dtype)).item()

    p = lambda e: 2.0 ** e
    assert array(tensor(np.array([1.0 + p(-8) + p(-21)]), DT.F64, [1], GPU).to(DT.F32).to(DT.BF16)).item() == 0x3F81
    assert g(1.0 + p(-8) + p(-40), DT.BF16) == 0x3F80
    assert g(1.0 + p(-11) + p(-40), DT.F16) == 0x3C00
    i = tensor(np.array([(1 << 24) + (1 << 16) + 1], dtype=np.int64), DT.I64, [1], GPU)
    assert array(i.to(DT.BF16)).item() == 0x4B80                                                       # 2^24
    b = tensor(np.array([0.0, -0.0, 0.1, np.nan, -3.0]), DT.F64, [5], GPU).to(DT.Bool)
    assert array(b).tolist() == [0, 0, 1, 1, 1]
    assert array(b.to(DT.U8)).tolist() == [0, 0, 1, 1, 1]


def test_fill_writes_every_dtype_and_layout():
    for dtype, v in ((DT.Bool, True), (DT.U8, 200), (DT.I8, -3), (DT.I16, -30000), (DT.I32, 1 << 30), (DT.I64, -(1 << 40)),
                     (DT.F16, 1.5), (DT.BF16, -2.5), (DT.F32, 3.25), (DT.F64, 1e-300)):
        for shape in ([], [1], [7], [1031], [3, 257], [0, 4]):
            gpu, cpu = h.full(shape, v, dtype, GPU), h.full(shape, v, dtype, "cpu")
            assert_same(gpu, cpu, f"full {dtype} {shape}")
            n = int(np.prod(shape)) if shape else 1
            if n:
                want = array(cpu).reshape(-1)
                assert (want == want[0]).all() and want.dtype == NP[dtype]


def test_fill_writes_exactly_its_span_at_every_offset_and_length():
    """hmr_fill through the C ABI into the middle of a buffer: every alignment of the first element, every tail
    after the last 16-byte tile, a span of several workgroups, a strided destination; the elements on both
    sides keep their guard pattern."""
    from ctypes import byref

    from homura_amd import capi
    L = capi.lib
    ctx = capi.Context(0)
    try:
        for code, npdt, value, guard in ((capi.U8, np.uint8, 0xA5, 0x11), (capi.I16, np.int16, -1234, 0x1111),
                                         (capi.F32, np.float32, 3.25, 7.0), (capi.I64, np.int64, -(1 << 40), 5)):
            total = 70000
            bits = int(np.array([value], dtype=npdt).view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[
                np.dtype(npdt).itemsize])[0])
            spans = [(o, n) for o in range(0, 18) for n in (0, 1, 2, 3, 15, 16, 17, 33, 1023, 1031, 5000)] + [(3, 69000), (16, 65536)]
            clean = np.full(total, guard, dtype=npdt)
            buf = ctx.upload(clean)
            for offset, n in spans:
                capi.check(L.hmr_copy_from_host(ctx.handle, buf.ptr, clean.ctypes.data, clean.nbytes))
                d = capi.make_desc(buf.ptr, code, [n], [1], offset)
                capi.check(L.hmr_fill(ctx.handle, byref(d), bits))
                ctx.synchronize()
                got = buf.download(npdt, total)
                want = np.full(total, guard, dtype=npdt)
                want[offset:offset + n] = value
                assert np.array_equal(got, want), f"{npdt.__name__} offset {offset} length {n}"
            capi.check(L.hmr_copy_from_host(ctx.handle, buf.ptr, clean.ctypes.data, clean.nbytes))
            d = capi.make_desc(buf.ptr, code, [100, 30], [600, 2], 8)
            capi.check(L.hmr_fill(ctx.handle, byref(d), bits))
            ctx.synchronize()
            want = np.full(total, guard, dtype=npdt)
            want[8:8 + 100 * 600].reshape(100, 600)[:, 0:60:2] = value
            assert np.array_equal(buf.download(npdt, total), want), f"{npdt.__name__} strided"
            buf.free()
    finally:
        ctx.close()


def test_moves_between_the_cpu_and_the_gpu():
    """ref: tests/rocm_copy.rs:126-157"""
    for k, dtype in enumerate(DTYPES):
        for pair in layouts(dtype, 100 + k):
            what = f"{dtype}, {pair.name}"
            up = pair.cpu.to(GPU)
            assert_same(up, pair.cpu, what)
            assert up.is_contiguous(), what
            down = pair.gpu.to("cpu")
            assert str(down.device) == "cpu" and np.array_equal(bits(down), bits(pair.cpu)), what
            assert np.array_equal(bits(up.to("cpu")), bits(pair.cpu)), what
            for to in (DT.F16, DT.I32, DT.Bool, DT.F64):
                expected = pair.cpu.to(to)
                assert_same(pair.cpu.to(to).to(GPU), expected, f"{what} -> {to}")
                down = pair.gpu.to(to).to("cpu")
                assert str(down.device) == "cpu" and np.array_equal(bits(down), bits(expected)), f"{what} -> {to} on the cpu"


def test_copy_into_strided_targets():
    """A transposed target, a broadcast source of another dtype, on the same device and across devices; a copy onto
    an overlapping part of itself goes through a copy (ref: tests/rocm_copy.rs:160-184)."""
    for k, src_dtype in enumerate(DTYPES):
        for to in (DT.F32, DT.I8, DT.BF16, src_dtype):
            src = tensor(values(src_dtype, 5, 300 + k), src_dtype, [5])
            zeros = np.zeros(15, dtype=NP[to])
            cpu = tensor(zeros, to, [5, 3]).transpose(0, 1)
            gpu = tensor(zeros, to, [5, 3], GPU).transpose(0, 1)
            cpu.copy_(src.reshape([1, 5]))
            gpu.copy_(src.to(GPU).reshape([1, 5]))
            what = f"{src_dtype} -> {to}"
            assert_same(gpu, cpu, what)
            gpu = tensor(zeros, to, [5, 3], GPU).transpose(0, 1)
            gpu.copy_(src.reshape([1, 5]))
            assert_same(gpu, cpu, f"{what}, cpu source")
            back = tensor(zeros, to, [5, 3]).transpose(0, 1)
            back.copy_(src.to(GPU).reshape([1, 5]))
            assert np.array_equal(bits(back), bits(cpu)), f"{what}, gpu source"
    x = tensor(np.arange(6, dtype=np.int64), DT.I64, [6], GPU)
    x.narrow(0, 1, 5).copy_(x.narrow(0, 0, 5))
    assert array(x).tolist() == [0, 0, 1, 2, 3, 4]
    # A large strided target: every other row of a matrix takes rows of another dtype.
    rows = tensor(values(DT.F32, 512 * 384, 7), DT.F32, [512, 384])
    for to in (DT.F32, DT.BF16):
        zeros = np.zeros(1024 * 384, dtype=NP[to])
        cpu, gpu = tensor(zeros, to, [1024, 384]), tensor(zeros, to, [1024, 384], GPU)
        cpu.slice(0, 1, None, 2).copy_(rows)
        gpu.slice(0, 1, None, 2).copy_(rows.to(GPU))
        assert_same(gpu, cpu, f"every other row <- f32 as {to}")
        cpu.transpose(0, 1).narrow(0, 5, 300).fill_(2.5)
        gpu.transpose(0, 1).narrow(0, 5, 300).fill_(2.5)
        assert_same(gpu, cpu, f"fill_ of a transposed part, {to}")


def test_strided_gpu_tensors_read_back_directly():
    """ref: tests/rocm_copy.rs:265-283"""
    cpu = tensor(np.arange(12, dtype=np.float32), DT.F32, [3, 4])
    gpu = cpu.to(GPU)
    ct, gt = cpu.transpose(0, 1), gpu.transpose(0, 1)
    assert not gt.is_contiguous()
    assert array(gt).tolist() == array(ct).tolist()
    assert array(gpu.select(1, 2).select(0, 1)).item() == 6.0
    half = gpu.to(DT.F16).transpose(0, 1).narrow(0, 1, 2)
    assert np.array_equal(bits(half), bits(cpu.to(DT.F16).transpose(0, 1).narrow(0, 1, 2)))
    b = h.full([2, 3], True, DT.Bool, GPU).expand([4, 2, 3]).transpose(0, 2)
    assert array(b).reshape(-1).tolist() == [1] * 24
