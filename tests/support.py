"""Helpers of the parity tests, modelled on the reference's tests/common/rocm.rs: inputs made of
special values followed by pseudo-random bit patterns, the same tensor on the CPU (oracle) and on
the GPU in a range of layouts, and judges that compare raw bits or count ulps."""
import json
import math
import os
import struct

import numpy as np

import homura_amd

h = homura_amd.load_host()
DT = h.DType
DTYPES = [DT.Bool, DT.U8, DT.I8, DT.I16, DT.I32, DT.I64, DT.F16, DT.BF16, DT.F32, DT.F64]
FLOATS = [DT.F16, DT.BF16, DT.F32, DT.F64]
INTS = [DT.U8, DT.I8, DT.I16, DT.I32, DT.I64]
NP = {DT.Bool: np.uint8, DT.U8: np.uint8, DT.I8: np.int8, DT.I16: np.int16, DT.I32: np.int32, DT.I64: np.int64,
      DT.F16: np.uint16, DT.BF16: np.uint16, DT.F32: np.float32, DT.F64: np.float64}
SIZE = {d: np.dtype(NP[d]).itemsize for d in DTYPES}
GPU = "rocm:0"
MASK64 = (1 << 64) - 1


class Words:
    """SplitMix64 (ref: tests/common/rocm.rs:27-42)."""

    def __init__(self, seed):
        self.s = seed & MASK64

    def next(self):
        self.s = (self.s + 0x9E3779B97F4A7C15) & MASK64
        z = self.s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
        return z ^ (z >> 31)


def words(seed, n):
    """n SplitMix64 words as a uint64 array (vectorised, same stream as Words)."""
    idx = np.arange(1, n + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed & MASK64) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def p2(e):
    return math.ldexp(1.0, e)


def f64_from_bits(b):
    return struct.unpack("<d", struct.pack("<Q", b))[0]


def special_f64():
    """ref: tests/common/rocm.rs:62-122"""
    f32_min_sub = float(np.frombuffer(struct.pack("<I", 1), dtype=np.float32)[0])
    v = [0.0, -0.0, 1.0, -1.0, 0.5, -2.5, 2.5, 255.9, -0.5, 300.0, -129.9, 1e30, -1e30, 65504.0, 65520.0, -65536.0,
         math.inf, -math.inf, math.nan, -math.nan, f64_from_bits(0x7FF0000000000001), f64_from_bits(0xFFF4000000001234),
         f64_from_bits(0x7FF8000020000000), 2.2250738585072014e-308, -2.2250738585072014e-308 / 3.0, f64_from_bits(1),
         1.7976931348623157e308, -1.7976931348623157e308, 3.4028234663852886e38, 1.1754943508222875e-38, f32_min_sub,
         f32_min_sub / 2.0, f32_min_sub * 0.75, 6.0e-8, p2(-24) * 1.5, p2(-133), 9.2e18, -9.3e18, p2(63), -p2(63),
         p2(63) - 1024.0, p2(31), -p2(31) - 1.0, p2(53) + 1.0, 1.0 + p2(-8) + p2(-21), 1.0 + p2(-8) + p2(-40),
         1.0 + p2(-11) + p2(-40), 1.0 + p2(-11), 1.0 + p2(-8), 1.0 + p2(-24), 1.0 + p2(-24) + p2(-52),
         -(1.0 + p2(-8) + p2(-21))]
    v += [(i - 20.0) * 0.37 for i in range(40)]
    return v


def special_i64():
    """ref: tests/common/rocm.rs:124-160"""
    v = [0, 1, -1, 2, 127, 128, -128, -129, 255, 256, -255, 300, 32767, 32768, -32769, 65535, 65536, 2**31 - 1, -2**31,
         2**31, 2**63 - 1, -2**63, 2**63 - 2, (1 << 24) + 1, (1 << 24) + (1 << 16) + 1, (1 << 53) + 1,
         (1 << 53) + (1 << 30) + 1, 65504, 65520, 70000]
    v += [i * 7 - 140 for i in range(40)]
    return v


# ---- conversions between dtype storage and f64, in numpy (independent of the code under test) ----

def f32_to_bf16_bits(a):
    """f32 array -> bf16 patterns, round to nearest even, NaN quiet (the textbook rule)."""
    x = np.asarray(a, dtype=np.float32).view(np.uint32)
    nan = (x & 0x7FFFFFFF) > 0x7F800000
    r = ((x + 0x7FFF + ((x >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((x >> 16) | 0x40).astype(np.uint16), r)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_f64(arr, dtype):
    """The elements of a storage array as exact f64 values."""
    if dtype == DT.F16:
        return arr.view(np.float16).astype(np.float64)
    if dtype == DT.BF16:
        return bf16_bits_to_f32(arr).astype(np.float64)
    return arr.astype(np.float64)


def from_f64(values, dtype):
    """f64 values -> storage array of dtype, converted as homura's from_f64 (halves through f32)."""
    v = np.asarray(values, dtype=np.float64)
    with np.errstate(all="ignore"):
        if dtype == DT.F64:
            return v.copy()
        if dtype == DT.F32:
            return v.astype(np.float32)
        if dtype == DT.F16:
            return v.astype(np.float32).astype(np.float16).view(np.uint16)
        if dtype == DT.BF16:
            return f32_to_bf16_bits(v.astype(np.float32))
        if dtype == DT.Bool:
            return (v != 0).astype(np.uint8)
        # integers: truncate, saturate to i64 (NaN -> 0), wrap
        t = np.where(np.isnan(v), 0.0, v)
        t = np.clip(np.trunc(t), -9.223372036854775808e18, 9.223372036854775807e18)
        i = np.where(t >= 9.223372036854775807e18, np.int64(2**63 - 1), t.astype(np.int64))
        return i.astype(NP[dtype])


def values(dtype, n, seed):
    """n elements of dtype: the special values first, then random bit patterns
    (ref: tests/common/rocm.rs:162-211). Returns the storage array."""
    w = words(seed, n)
    if dtype == DT.Bool:
        special = np.array([0, 1], dtype=np.uint8)
        rnd = (w & np.uint64(1)).astype(np.uint8)
    elif dtype in INTS:
        special = np.array([x & MASK64 for x in special_i64()], dtype=np.uint64).astype(NP[dtype])
        rnd = w.astype(NP[dtype]) if dtype != DT.I64 else w.view(np.int64)
    elif dtype == DT.F64:
        special = np.array(special_f64(), dtype=np.float64)
        rnd = w.view(np.float64)
    elif dtype == DT.F32:
        with np.errstate(all="ignore"):
            special = np.array(special_f64(), dtype=np.float64).astype(np.float32)
        rnd = w.astype(np.uint32).view(np.float32)
    else:
        special = from_f64(special_f64(), dtype)
        rnd = w.astype(np.uint16)
    out = np.empty(n, dtype=NP[dtype])
    k = min(n, len(special))
    out[:k] = special[:k]
    # the reference draws one word per non-special element, starting at the first word
    out[k:] = rnd[: n - k]
    return out


def mixed_floats(dtype, n, seed):
    """A mix of magnitudes, signs, zeros and values that overflow or vanish in F16
    (ref: src/backend/rocm/tests.rs:809-830)."""
    s, out = seed, np.empty(n, dtype=np.float64)
    for i in range(n):
        s = (s * 6364136223846793005 + 1442695040888963407) & ((1 << 64) - 1)
        u = (s >> 11) / float(1 << 53)
        e = ((s >> 3) % 40) - 20
        out[i] = {0: 0.0, 1: -0.0, 2: 7e4, 3: 1e-7}.get(i % 17, (u * 2.0 - 1.0) * 2.0 ** e)
    return tensor(from_f64(out, dtype), dtype)


def normal(seed, n, mean=0.0, std=1.0):
    """Box-Muller in f64 from SplitMix64 words (the bench and config inputs)."""
    w = words(seed, 2 * ((n + 1) // 2))
    u = ((w >> np.uint64(11)).astype(np.float64) + 0.5) / float(1 << 53)
    u1, u2 = u[0::2], u[1::2]
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([r * np.cos(2 * math.pi * u2), r * np.sin(2 * math.pi * u2)])[:n]
    return mean + std * z


def uniform(seed, n, lo=0.0, hi=1.0):
    w = words(seed, n)
    u = (w >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    return lo + (hi - lo) * u


def tensor(arr, dtype, shape=None, device="cpu"):
    arr = np.ascontiguousarray(arr)
    return h.Tensor.from_bytes(arr, dtype, list(arr.shape if shape is None else shape), device)


def array(t):
    """The elements of a tensor (any device) as a numpy storage array of its shape."""
    a = np.frombuffer(t.to_bytes(), dtype=NP[t.dtype]).copy()
    return a.reshape(t.shape)


def bits(t):
    a = array(t).reshape(-1)
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize]).astype(np.uint64)


# ---- layouts (ref: tests/common/rocm.rs:273-325) ----------------------------------------------------

VIEWS = [
    ("contiguous [3, 5]", 15, lambda t: t.reshape([3, 5])),
    ("contiguous with an offset [7]", 10, lambda t: t.narrow(0, 2, 7)),
    ("transposed [5, 3]", 15, lambda t: t.reshape([3, 5]).transpose(0, 1)),
    ("broadcast [4, 3, 5] (stride 0)", 15, lambda t: t.reshape([1, 3, 5]).expand([4, 3, 5])),
    ("narrow with an offset [2, 3]", 20, lambda t: t.reshape([4, 5]).narrow(0, 1, 2).narrow(1, 1, 3)),
    ("0-dim", 1, lambda t: t.reshape([])),
    ("empty [0, 3]", 0, lambda t: t.reshape([0, 3])),
    ("odd [1031]", 1031, lambda t: t),
    ("permuted [5, 4, 3, 2]", 120, lambda t: t.reshape([2, 3, 4, 5]).permute([3, 2, 1, 0])),
    ("every other [600]", 1200, lambda t: t.reshape([600, 2]).select(1, 1)),
    ("past one block [3, 257]", 771, lambda t: t.reshape([3, 257]).transpose(0, 1)),
    # Layouts the gfx950 kernels special-case: rows that vectorise, bias / per-row broadcasts.
    ("rows [9, 64] of a wider buffer", 9 * 80, lambda t: t.reshape([9, 80]).narrow(1, 16, 64)),
    ("inner broadcast [7, 48]", 48, lambda t: t.reshape([1, 48]).expand([7, 48])),
    ("row broadcast [6, 40]", 6, lambda t: t.reshape([6, 1]).expand([6, 40])),
    ("permuted heads [2, 4, 3, 32]", 2 * 3 * 4 * 32, lambda t: t.reshape([2, 3, 4, 32]).permute([0, 2, 1, 3])),
    # Large enough for the rows kernel to walk the transposed pair of dimensions in tiles of 8.
    ("permuted heads [2, 8, 24, 32]", 2 * 24 * 8 * 32, lambda t: t.reshape([2, 24, 8, 32]).permute([0, 2, 1, 3])),
]


class Pair:
    def __init__(self, name, cpu, gpu):
        self.name, self.cpu, self.gpu = name, cpu, gpu


def layouts(dtype, seed, views=VIEWS):
    out = []
    for name, n, view in views:
        base = tensor(values(dtype, n, seed), dtype, [n])
        cpu = view(base)
        gpu = view(base.to(GPU))
        assert gpu.strides == cpu.strides and gpu.offset == cpu.offset, name
        out.append(Pair(name, cpu, gpu))
    return out


def large_layouts(dtype, seed):
    """More elements than one pass of any launch grid covers (ref: tests/common/rocm.rs:327-344)."""
    n = (1 << 24) + 1000
    base = tensor(values(dtype, 2 * n, seed), dtype, [2 * n])
    g = base.to(GPU)
    return [Pair("large contiguous", base.narrow(0, 0, n), g.narrow(0, 0, n)),
            Pair("large strided", base.reshape([n, 2]).select(1, 1), g.reshape([n, 2]).select(1, 1))]


# ---- judges -----------------------------------------------------------------------------------------------

def is_nan_bits(dtype, b):
    if dtype == DT.F16:
        return (b & 0x7FFF) > 0x7C00
    if dtype == DT.BF16:
        return (b & 0x7FFF) > 0x7F80
    if dtype == DT.F32:
        return (b & 0x7FFFFFFF) > 0x7F800000
    if dtype == DT.F64:
        return (b & np.uint64(0x7FFFFFFFFFFFFFFF)) > np.uint64(0x7FF0000000000000)
    return np.zeros(b.shape, dtype=bool)


def _header(gpu, cpu, what):
    assert gpu.device == GPU, f"{what}: device {gpu.device}"
    assert gpu.shape == cpu.shape, f"{what}: shape {gpu.shape} vs {cpu.shape}"
    assert gpu.dtype == cpu.dtype, f"{what}: dtype {gpu.dtype} vs {cpu.dtype}"


def assert_same(gpu, cpu, what):
    """Same shape, dtype and bits, NaN payloads included (ref: tests/common/rocm.rs:253-271)."""
    _header(gpu, cpu, what)
    g, c = bits(gpu), bits(cpu)
    bad = np.nonzero(g != c)[0]
    assert bad.size == 0, (f"{what}: element {bad[0]} differs: gpu {int(g[bad[0]]):#x}, cpu {int(c[bad[0]]):#x} "
                           f"({bad.size} of {g.size} differ)")


def assert_bitwise(gpu, cpu, what):
    """Same bits, except that a NaN only has to meet a NaN (ref: tests/common/rocm.rs:357-377)."""
    _header(gpu, cpu, what)
    g, c = bits(gpu), bits(cpu)
    same = (g == c) | (is_nan_bits(cpu.dtype, g) & is_nan_bits(cpu.dtype, c))
    bad = np.nonzero(~same)[0]
    assert bad.size == 0, (f"{what}: element {bad[0]} differs: gpu {int(g[bad[0]]):#x}, cpu {int(c[bad[0]]):#x} "
                           f"({bad.size} of {g.size} differ)")


def ulp_of(dtype, v):
    """Spacing of dtype at |v| (ref: tests/common/rocm.rs:388-407)."""
    man, min_exp = {DT.F16: (10, -14), DT.BF16: (7, -126), DT.F32: (23, -126), DT.F64: (52, -1022)}[dtype]
    v = np.abs(np.asarray(v, dtype=np.float64))
    biased = (v.view(np.uint64) >> np.uint64(52)).astype(np.int64)
    e = np.where(biased == 0, -1023, biased - 1023)
    return np.ldexp(1.0, (np.maximum(e, min_exp) - man).astype(np.int64))


def ordered(b, dtype):
    """Bit patterns mapped to integers that are monotonic in the value."""
    nbits = {DT.F16: 16, DT.BF16: 16, DT.F32: 32, DT.F64: 64}[dtype]
    b = b.astype(np.uint64)
    sign = np.uint64(1) << np.uint64(nbits - 1)
    mag = (b & (sign - np.uint64(1))).astype(np.float64) if nbits == 64 else (b & (sign - np.uint64(1))).astype(np.int64)
    neg = (b & sign) != 0
    return np.where(neg, -mag, mag)


def check_within(gpu, cpu, extra=0.0, max_ulp=1, what=""):
    """|gpu - cpu| <= extra + max_ulp * ulp_out(max(|gpu|,|cpu|)); NaN must meet NaN, an infinity the
    same infinity (ref: tests/common/rocm.rs:486-537, with max_ulp = 1 there). Returns
    (number of differing elements, largest distance in ulps)."""
    _header(gpu, cpu, what)
    dtype = cpu.dtype
    ga, ca = array(gpu).reshape(-1), array(cpu).reshape(-1)
    g, c = to_f64(ga, dtype), to_f64(ca, dtype)
    special = np.isnan(g) | np.isnan(c) | np.isinf(g) | np.isinf(c)
    ok_special = (np.isnan(g) & np.isnan(c)) | (g == c)
    bad = np.nonzero(special & ~ok_special)[0]
    assert bad.size == 0, f"{what}: element {bad[0]}: gpu {g[bad[0]]!r}, cpu {c[bad[0]]!r} (classification)"
    fin = ~special & (g != c)
    if not fin.any():
        return 0, 0
    extra = np.broadcast_to(np.asarray(extra, dtype=np.float64), g.shape)
    with np.errstate(all="ignore"):
        bound = extra + max_ulp * ulp_of(dtype, np.maximum(np.abs(g), np.abs(c)))
        over = fin & ~(np.abs(g - c) <= bound)
    bad = np.nonzero(over)[0]
    assert bad.size == 0, (f"{what}: element {bad[0]}: gpu {g[bad[0]]!r}, cpu {c[bad[0]]!r}: |diff| "
                           f"{abs(g[bad[0]] - c[bad[0]])!r} > bound {bound[bad[0]]!r} ({bad.size} of {g.size} over)")
    gb = ga.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[ga.dtype.itemsize])
    cb = ca.view(gb.dtype)
    dist = np.abs(ordered(gb[fin], dtype) - ordered(cb[fin], dtype))
    return int(fin.sum()), int(dist.max())


# ---- golden vectors (tests/golden/ops.safetensors, the reference's own PyTorch outputs) -------------

ST_DTYPES = {"BOOL": DT.Bool, "U8": DT.U8, "I8": DT.I8, "I16": DT.I16, "I32": DT.I32, "I64": DT.I64, "F16": DT.F16,
             "BF16": DT.BF16, "F32": DT.F32, "F64": DT.F64}


def load_golden(path=None):
    """{case: {name: (storage array shaped, dtype)}} parsed from the safetensors file (header JSON +
    raw little-endian data; nothing in the file is executed)."""
    path = path or os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ops.safetensors")
    with open(path, "rb") as f:
        raw = f.read()
    n = struct.unpack("<Q", raw[:8])[0]
    header = json.loads(raw[8:8 + n])
    data = raw[8 + n:]
    cases = {}
    for key, meta in header.items():
        if key == "__metadata__":
            continue
        case, name = key.split("/", 1)
        dtype = ST_DTYPES[meta["dtype"]]
        lo, hi = meta["data_offsets"]
        arr = np.frombuffer(data[lo:hi], dtype=NP[dtype]).copy().reshape(meta["shape"])
        cases.setdefault(case, {})[name] = (arr, dtype)
    return cases
