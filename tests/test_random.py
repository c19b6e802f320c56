"""Random sampling from the Philox4x32-10 generator (ref: src/ops/random.rs; tests/random.rs; tests/rocm_random.rs).

Without a GPU this pins the oracle: the Random123 known-answer vectors the reference itself tests (ref:
src/ops/random.rs:478-497), the reference's one concrete sample (`0.6159043529544902` after seed 6 and a rejected-
words randint, ref: tests/rocm_random.rs:100-104), closed forms built from the published first block (seed 0 is the
all-zero key and counter), the value ranges of ref: src/ops/random.rs:499-531 and the statistics and generator rules of
tests/random.rs. On the GPU: uniform samples and integers are the CPU's bit for bit for every dtype, size, interval and
device interleaving; normal samples stay within 6 * 2^-53 * M plus one output ulp (ref: tests/rocm_random.rs:145-222).
"""
import ctypes
import math

import numpy as np
import pytest

from tests import oracle
from tests.support import DT, FLOATS, GPU, array, assert_bitwise, bits, check_within, h, tensor, to_f64

h.register_cpu_backend(oracle.backend_address())
SIZES = [0, 1, 2, 3, 5, 1031, 4096, (1 << 20) + 3]
KAT0 = [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]  # counter 0, key 0
I64_MIN, I64_MAX = -(1 << 63), (1 << 63) - 1


def philox(counter, key):
    """Philox4x32-10 as published (Salmon et al., SC11), written independently of the oracle and checked against the
    same known answers."""
    c, k = list(counter), list(key)
    for r in range(10):
        if r > 0:
            k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
        p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
    return c


def block(seed, n):
    return philox([n & 0xFFFFFFFF, n >> 32, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])


def test_philox_known_answers():
    lib = oracle.lib()
    vectors = [([0] * 4, [0] * 2, KAT0),
               ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
               ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
                [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1])]
    for counter, key, want in vectors:
        out = (ctypes.c_uint32 * 4)()
        lib.orc_philox((ctypes.c_uint32 * 4)(*counter), (ctypes.c_uint32 * 2)(*key), out)
        assert list(out) == want
        assert philox(counter, key) == want


def test_the_first_block_reaches_the_samples_in_order():
    """Seed 0, offset 0 is the published vector: element j of a narrow float takes word j's top bits, an F64 element
    takes two words, a normal pair the whole block, an integer a 64-bit word (high word first)."""
    for dtype, digits in ((DT.F16, 11), (DT.BF16, 8), (DT.F32, 24)):
        h.manual_seed(0)
        got = to_f64(array(h.rand([4], dtype, "cpu")), dtype)
        assert got.tolist() == [(w >> (32 - digits)) / float(1 << digits) for w in KAT0], dtype
    unit = lambda hi, lo: float((hi << 21) ^ (lo >> 11)) / float(1 << 53)
    h.manual_seed(0)
    assert array(h.rand([2], DT.F64, "cpu")).tolist() == [unit(KAT0[0], KAT0[1]), unit(KAT0[2], KAT0[3])]
    h.manual_seed(0)
    u1, u2 = 1.0 - unit(KAT0[0], KAT0[1]), unit(KAT0[2], KAT0[3])
    r, theta = math.sqrt(-2.0 * math.log(u1)), 2.0 * math.pi * u2
    got = array(h.randn([2], DT.F64, "cpu")).tolist()
    assert got == pytest.approx([r * math.cos(theta), r * math.sin(theta)], rel=1e-15, abs=1e-16)
    h.manual_seed(0)
    words = [(KAT0[0] << 32) | KAT0[1], (KAT0[2] << 32) | KAT0[3]]
    assert array(h.randint(0, 1 << 40, [2], DT.I64, "cpu")).tolist() == [w % (1 << 40) for w in words]
    h.manual_seed(0)
    assert array(h.randint(-5, 6, [2], DT.I64, "cpu")).tolist() == [-5 + w % 11 for w in words]  # neither is rejected


def test_the_references_sample():
    """ref: tests/rocm_random.rs:100-104 (the sequence is the same on every device): about half of the words of
    [i64::MIN, 1) are rejected, three blocks go for one value, and the next F64 sample is this one."""
    h.manual_seed(6)
    h.randint(I64_MIN, 1, [1], DT.I64, "cpu")
    assert array(h.rand([1], DT.F64, "cpu")).item() == 0.6159043529544902


def expected_ints(seed, n, low, high):
    """sample_int of ref: src/ops/random.rs:228-258 over the independent Philox; returns the values and the blocks used."""
    rng = high - low
    threshold = ((1 << 64) - rng) % rng
    out, offset = [], 0
    while len(out) < n:
        blocks = (n - len(out) + 1) // 2
        for i in range(blocks):
            b = block(seed, offset + i)
            for w in ((b[0] << 32) | b[1], (b[2] << 32) | b[3]):
                if w >= threshold and len(out) < n:
                    out.append(low + w % rng)
        offset += blocks
    return out, offset


@pytest.mark.parametrize("low,high", [(0, 2), (-5, 6), (0, 3), (I64_MIN, 1), (I64_MIN, I64_MAX), (-(1 << 62) - 1, 1 << 62),
                                      (I64_MAX - 1, I64_MAX)])
def test_integer_sampling_against_the_independent_generator(low, high):
    for n in (1, 2, 7, 300):
        h.manual_seed(11)
        want, used = expected_ints(11, n, low, high)
        assert array(h.randint(low, high, [n], DT.I64, "cpu")).tolist() == want
        # The next call starts at the block after the ones the batches reserved.
        b = block(11, used)
        assert array(h.rand([4], DT.F32, "cpu")).tolist() == [(w >> 8) / float(1 << 24) for w in b]


def test_later_blocks_and_intervals_against_the_independent_generator():
    h.manual_seed(1234567890123)
    n = 37
    got = array(h.uniform([n], -3.0, 5.0, DT.F32, "cpu")).tolist()
    words = [w for i in range((n + 3) // 4) for w in block(1234567890123, i)][:n]
    assert got == [float(np.float32(-3.0 + ((w >> 8) / float(1 << 24)) * 8.0)) for w in words]
    used = (n + 3) // 4
    got = array(h.normal([5], 3.0, 0.5, DT.F64, "cpu")).tolist()
    want = []
    for i in range(3):
        b = block(1234567890123, used + i)
        u1 = 1.0 - float((b[0] << 21) ^ (b[1] >> 11)) / float(1 << 53)
        u2 = float((b[2] << 21) ^ (b[3] >> 11)) / float(1 << 53)
        r, theta = math.sqrt(-2.0 * math.log(u1)), 2.0 * math.pi * u2
        want += [3.0 + 0.5 * r * math.cos(theta), 3.0 + 0.5 * r * math.sin(theta)]
    assert got == pytest.approx(want[:5], rel=4e-16)


def test_unit_ranges_and_the_excluded_upper_bound():
    """ref: src/ops/random.rs:499-516, 279-286: samples are below 1 in every dtype; a sample that rounds to `to` becomes
    `from`."""
    for dtype, digits in ((DT.F16, 11), (DT.BF16, 8), (DT.F32, 24), (DT.F64, 53)):
        h.manual_seed(3)
        v = to_f64(array(h.rand([20000], dtype, "cpu")), dtype)
        assert v.min() >= 0.0 and v.max() < 1.0 and v.max() >= 1.0 - 2.0 ** -7
        assert (v * 2.0 ** digits == np.floor(v * 2.0 ** digits)).all()  # k / 2^digits, exactly
        h.manual_seed(3)
        w = to_f64(array(h.uniform([20000], 1.0, 1.125, dtype, "cpu")), dtype)
        assert w.min() >= 1.0 and w.max() < 1.125
    # BF16 has 16 values in [1, 1.125): every one is reached, and the 8 of 256 levels that round up to 1.125 land on 1.0.
    h.manual_seed(3)
    v = to_f64(array(h.uniform([20000], 1.0, 1.125, DT.BF16, "cpu")), DT.BF16)
    assert set(v.tolist()) == {1.0 + k / 128.0 for k in range(16)}


def seeded_sampling(device):
    """ref: tests/random.rs:7-64, 80-139"""
    h.manual_seed(42)
    a = h.rand([1000], DT.F32, device)
    n = h.randn([10001], DT.F32, device)
    h.manual_seed(42)
    b = h.rand([1000], DT.F32, device)
    assert (bits(a) == bits(b)).all(), "same seed must give the same numbers"
    assert not (bits(a) == bits(h.rand([1000], DT.F32, device))).all()
    lo, hi = array(a).min(), array(a).max()
    assert 0.0 <= lo < 0.01 and 0.99 <= hi < 1.0
    mean, std = array(n).mean(), array(n).std(ddof=1)
    assert abs(mean) < 0.05 and abs(std - 1.0) < 0.05
    r = h.randint(-3, 4, [2000], DT.I64, device)
    assert r.dtype == DT.I64 and (array(r).min(), array(r).max()) == (-3, 3)
    assert h.randn([100], DT.BF16, device).dtype == DT.BF16
    x = array(h.uniform([3, 400], 2.0, 3.0, DT.F32, device))
    assert ((x >= 2.0) & (x < 3.0)).all()
    assert abs(array(h.normal([3, 400], 5.0, 0.1, DT.F32, device)).mean() - 5.0) < 0.02
    assert array(h.randint(0, 2, [64], DT.Bool, device)).max() == 1
    assert h.randint(-100, 100, [3, 333], DT.F16, device).dtype == DT.F16
    # Rejected calls don't advance the generator.
    h.manual_seed(7)
    expected = bits(h.rand([4], DT.F32, device))
    h.manual_seed(7)
    rejected = [
        (lambda: h.uniform([4], -1e308, 1e308, DT.F64, device), "uniform_ expects to - from <= "),
        (lambda: h.randint(70000, 70001, [4], DT.F16, device), r"random_ expects \[from, to\) to lie inside \[-2048, 2048\] for f16"),
        (lambda: h.uniform([4], 1.0, 0.5, DT.F32, device), r"uniform_ expects to return a \[from, to\) range, but found from=1 > to=0.5"),
        (lambda: h.uniform([4], 0.0, 1e5, DT.F16, device), "uniform_ expects to to be a finite value of f16, but got to=100000"),
        (lambda: h.normal([4], 0.0, -1.0, DT.F32, device), "normal expects std >= 0.0, but found std -1"),
        (lambda: h.randint(3, 3, [4], DT.I64, device), "random_ expects 'from' to be less than 'to', but got from=3 >= to=3"),
        (lambda: h.randint(0, 300, [4], DT.U8, device), r"random_ expects \[from, to\) to lie inside \[0, 255\] for u8"),
        (lambda: h.rand([4], DT.I32, device), "random floating point sampling is not implemented for i32 tensors"),
    ]
    for call, message in rejected:
        with pytest.raises(Exception, match=message):
            call()
    assert (bits(h.rand([4], DT.F32, device)) == expected).all()


def test_seeded_sampling_on_cpu_oracle():
    seeded_sampling("cpu")


def test_integer_sampling_covers_extreme_ranges():
    """ref: src/ops/random.rs:518-531"""
    h.manual_seed(5)
    v = array(h.randint(I64_MIN, I64_MAX, [64], DT.I64, "cpu"))
    assert (v < I64_MAX).all() and len(set(v.tolist())) == 64
    assert array(h.randint(I64_MAX - 1, I64_MAX, [8], DT.I64, "cpu")).tolist() == [I64_MAX - 1] * 8
    assert set(array(h.randint(0, 3, [500], DT.I64, "cpu")).tolist()) == {0, 1, 2}


# ---- the GPU ------------------------------------------------------------------------------------------------------


def both(seed, f):
    """f(device) after seeding, on the CPU and on the GPU (ref: tests/rocm_random.rs:25-32)."""
    h.manual_seed(seed)
    cpu = f("cpu")
    h.manual_seed(seed)
    return f(GPU), cpu


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", FLOATS)
def test_uniform_samples_are_the_cpus(dtype):
    for n in SIZES:
        g, c = both(7, lambda d: h.rand([n], dtype, d))
        assert_bitwise(g, c, f"rand {dtype} [{n}]")
        # The excluded upper bound: in F16 and BF16 many samples of [1, 1 + 2^-3) round up to it.
        for lo, hi in ((-3.0, 5.0), (1.0, 1.125), (-1e-3, 0.0), (0.0, 65504.0)):
            g, c = both(8, lambda d: h.uniform([n], lo, hi, dtype, d))
            assert_bitwise(g, c, f"uniform {dtype} [{n}] [{lo}, {hi})")
    g, c = both(9, lambda d: h.uniform([4, 6, 5], 0.0, 1.0, dtype, d))
    assert_bitwise(g, c, f"uniform {dtype} [4, 6, 5]")


@pytest.mark.gpu
def test_integer_samples_are_the_cpus():
    ranges = [(0, 2), (0, 1 << 40), (-5, 6), (0, 3), (I64_MIN, 1), (I64_MIN, I64_MAX), (-(1 << 62) - 1, 1 << 62),
              (I64_MAX - 1, I64_MAX)]
    for low, high in ranges:
        for n in SIZES:
            g, c = both(6, lambda d: h.randint(low, high, [n], DT.I64, d))
            assert_bitwise(g, c, f"randint [{low}, {high}) [{n}]")

            def after(d):
                h.randint(low, high, [n], DT.I64, d)
                return h.rand([5], DT.F64, "cpu").to(GPU)  # shows that both advanced the generator by the same blocks

            g, c = both(6, after)
            assert_bitwise(g, c.to("cpu"), f"after randint [{low}, {high}) [{n}]")
    for dtype in (DT.U8, DT.I16, DT.F16, DT.BF16, DT.F32, DT.F64):
        low = 0 if dtype == DT.U8 else -100
        g, c = both(10, lambda d: h.randint(low, 100, [3, 333], dtype, d))
        assert_bitwise(g, c, f"randint {dtype}")
    h.manual_seed(6)
    h.randint(I64_MIN, 1, [1], DT.I64, GPU)
    assert array(h.rand([1], DT.F64, "cpu")).item() == 0.6159043529544902


@pytest.mark.gpu
def test_alternating_devices_follow_one_sequence():
    """ref: tests/rocm_random.rs:106-129 (without the dropout call, which is outside this library)."""
    def run(devices):
        h.manual_seed(42)
        return [h.randint(I64_MIN, 1, [7], DT.I64, devices[0]).to("cpu"), h.rand([9], DT.F32, devices[1]).to("cpu"),
                h.randn([1001], DT.F64, devices[2]).to("cpu"), h.randint(0, 7, [13], DT.I64, devices[3]).to("cpu")]
    cpu = run(["cpu"] * 4)
    for devices in ([GPU] * 4, [GPU, "cpu", GPU, "cpu"], ["cpu", GPU, "cpu", GPU]):
        for i, (m, c) in enumerate(zip(run(devices), cpu)):
            if i == 2:
                check_within(m.to(GPU), c, extra=1e-14, what=f"{devices}: call {i}")
            else:
                assert_bitwise(m.to(GPU), c, f"{devices}: call {i}")


NORMAL_K, NORMAL_U = 6.0, 2.0 ** -53


def normal_sizes(seed, n, mean, std):
    """M = |mean| + |std| r (1 + 2 pi) per sample, r from the CPU's unrounded f64 pair (ref: tests/rocm_random.rs:
    150-167)."""
    h.manual_seed(seed)
    y = array(h.normal([n + n % 2], mean, std, DT.F64, "cpu")).astype(np.float64)
    a, b = (y[0::2] - mean) / std, (y[1::2] - mean) / std
    r = np.sqrt(a * a + b * b) * (1.0 + 2.0 ** -40) + 2.0 ** -40 * abs(mean) / std
    return np.repeat(abs(mean) + std * r * (1.0 + 2.0 * math.pi), 2)[:n]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", FLOATS)
def test_normal_samples_stay_within_the_bound(dtype):
    worst = 0
    for mean, std in ((0.0, 1.0), (3.0, 0.5), (-1e3, 10.0), (0.0, 1e-3)):
        for n in (1, 2, 7, 4096, (1 << 20) + 1):
            g, c = both(12, lambda d: h.normal([n], mean, std, dtype, d))
            m = normal_sizes(12, n, mean, std)
            differ, ulps = check_within(g, c, extra=NORMAL_K * NORMAL_U * m, what=f"normal {dtype} ({mean}, {std}) [{n}]")
            worst = max(worst, ulps)
            # The judge rejects one element off by twice the bound's first term plus 3 output ulps.
            ys = to_f64(array(c), dtype).copy()
            i = n // 2
            from tests.support import from_f64, ulp_of
            ys[i] += 2.0 * NORMAL_K * NORMAL_U * m[i] + 3.0 * float(ulp_of(dtype, np.array([abs(ys[i])]))[0])
            bad = tensor(from_f64(ys, dtype), dtype)
            with pytest.raises(AssertionError):
                check_within(g, bad, extra=NORMAL_K * NORMAL_U * m, what="off by more than the bound")
    print(f"normal {dtype}: the largest distance is {worst} ulp")

    def after(d):
        h.randn([5], dtype, d)
        return h.rand([3], DT.F64, "cpu").to(GPU)

    g, c = both(13, after)
    assert_bitwise(g, c.to("cpu"), f"after randn {dtype}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [DT.F32, DT.BF16, DT.F16])
def test_normal_samples_hold_the_bound_where_mean_and_deviation_cancel(dtype):
    """A sample is mean + std z: where the two cancel the result is small, its ulp with it, and the bound is left
    with its first term, 6 * 2^-53 * M: an f64 evaluation's accuracy. Millions of samples of distributions whose
    mean lies a fraction of a deviation from zero, so that thousands of them land next to zero."""
    for seed, (mean, std) in enumerate(((3.0, 10.0), (-250.0, 1000.0), (1.0, 1.0), (0.001, 0.01))):
        n = 1 << 22
        g, c = both(40 + seed, lambda d: h.normal([n], mean, std, dtype, d))
        m = normal_sizes(40 + seed, n, mean, std)
        check_within(g, c, extra=NORMAL_K * NORMAL_U * m, what=f"normal {dtype} ({mean}, {std}) [{n}]")


@pytest.mark.gpu
def test_seeded_sampling_on_gpu():
    seeded_sampling(GPU)


@pytest.mark.gpu
def test_sampling_through_the_c_abi_at_odd_offsets_and_its_errors():
    from ctypes import byref

    from homura_amd import capi
    L = capi.lib
    ctx = capi.Context(0)
    try:
        total = 5000
        guard = np.full(total, -7.0, dtype=np.float32)
        buf = ctx.upload(guard)
        for offset, n in ((0, 16), (1, 7), (3, 1030), (5, 4093)):
            capi.check(L.hmr_copy_from_host(ctx.handle, buf.ptr, guard.ctypes.data, guard.nbytes))
            d = capi.make_desc(buf.ptr, capi.F32, [n], [1], offset)
            capi.check(L.hmr_random_uniform(ctx.handle, byref(d), 99, 1000, 0.0, 1.0))
            ctx.synchronize()
            want = guard.copy()
            words = [w for i in range((n + 3) // 4) for w in block(99, 1000 + i)][:n]
            want[offset:offset + n] = [np.float32((w >> 8) / float(1 << 24)) for w in words]
            assert np.array_equal(buf.download(np.float32, total), want), (offset, n)
        strided = capi.make_desc(buf.ptr, capi.F32, [10], [2], 0)
        assert L.hmr_random_uniform(ctx.handle, byref(strided), 1, 0, 0.0, 1.0) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "random sampling writes a contiguous tensor"
        ints = capi.make_desc(buf.ptr, capi.I32, [10], [1], 0)
        assert L.hmr_random_normal(ctx.handle, byref(ints), 1, 0, 0.0, 1.0) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "random_normal: unsupported dtype"
        assert L.hmr_random_int(ctx.handle, byref(ints), 1, 0, 5, 0, 3, 0, None) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "random_int: unsupported dtype"
        i64 = capi.make_desc(buf.ptr, capi.I64, [10], [1], 0)
        assert L.hmr_random_int(ctx.handle, byref(i64), 1, 0, 5, 0, 3, 1, None) == capi.HMR_INVALID
        assert L.hmr_last_error().decode() == "random_int: a workspace is needed to reject words"
        # One batch with rejection: the accepted count is left in the workspace's last word.
        blocks, low, rng = 1000, -5, 11
        threshold = ((1 << 64) - rng) % rng
        tiles = (blocks + 255) // 256
        ws = ctx.malloc(8 * (2 * tiles + 1))
        out = ctx.upload(np.zeros(2 * blocks, dtype=np.int64))
        o = capi.make_desc(out.ptr, capi.I64, [2 * blocks], [1], 0)
        capi.check(L.hmr_random_int(ctx.handle, byref(o), 3, 77, blocks, low, rng, threshold, ws.ptr))
        ctx.synchronize()
        words = [w for i in range(blocks) for b in [block(3, 77 + i)] for w in ((b[0] << 32) | b[1], (b[2] << 32) | b[3])]
        kept = [low + w % rng for w in words if w >= threshold]
        assert int(ws.download(np.int64, 2 * tiles + 1)[-1]) == len(kept)
        assert out.download(np.int64, 2 * blocks)[:len(kept)].tolist() == kept
    finally:
        ctx.close()


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(4))
def test_random_sizes_and_ranges_follow_the_cpu(seed):
    """Sizes, ranges and dtypes drawn from a seeded generator (the lists above are fixed): uniform and integer
    samples have the CPU's bits, normal samples stay within their bound, and the generator has advanced by the same
    number of blocks after every call."""
    rng = np.random.default_rng(0x5EED3000 + seed)
    for case in range(40):
        n = int(np.exp(rng.uniform(0.0, np.log(300000.0))))
        shape = [n] if rng.integers(0, 2) else [int(rng.integers(1, 8)), max(1, n // 7)]
        count = int(np.prod(shape))
        s = int(rng.integers(0, 1 << 40))
        kind = int(rng.integers(0, 3))
        if kind == 0:
            dtype = FLOATS[int(rng.integers(0, len(FLOATS)))]
            lo = float(rng.choice([0.0, -1.0, 1.0, -3.5, 1e-3, 100.0])) * float(rng.choice([1.0, 16.0, 1e-2]))
            hi = lo + float(rng.choice([1.0, 0.125, 2.0 ** -6, 37.0, 1000.0]))
            what = f"seed {seed} case {case}: uniform {dtype} {shape} [{lo}, {hi})"
            g, c = both(s, lambda d: h.uniform(shape, lo, hi, dtype, d))
            assert_bitwise(g, c, what)
        elif kind == 1:
            dtype = [DT.I64, DT.I32, DT.I16, DT.U8, DT.F32, DT.F64][int(rng.integers(0, 6))]
            span = int(rng.choice([2, 3, 7, 11, 100, 255]))
            low = 0 if dtype == DT.U8 else int(rng.choice([0, -5, -100, 17]))
            if dtype == DT.I64 and rng.integers(0, 3) == 0:
                low, span = int(rng.choice([I64_MIN, -(1 << 62), 0])), int(rng.choice([(1 << 62) + 12345, (1 << 63) - 1, 1 << 40]))
            high = min(low + span, I64_MAX) if dtype == DT.I64 else min(low + span, 255 if dtype == DT.U8 else low + span)
            what = f"seed {seed} case {case}: randint {dtype} {shape} [{low}, {high})"
            g, c = both(s, lambda d: h.randint(low, high, shape, dtype, d))
            assert_bitwise(g, c, what)
        else:
            dtype = FLOATS[int(rng.integers(0, len(FLOATS)))]
            mean, std = float(rng.choice([0.0, 3.0, -250.0, 1e-2])), float(rng.choice([1.0, 0.5, 10.0, 1e-3]))
            what = f"seed {seed} case {case}: normal {dtype} {shape} ({mean}, {std})"
            g, c = both(s, lambda d: h.normal(shape, mean, std, dtype, d))
            check_within(g.reshape([count]), c.reshape([count]), extra=NORMAL_K * NORMAL_U * normal_sizes(s, count, mean, std), what=what)

        def after(d, kind=kind, dtype=dtype):
            if kind == 0:
                h.uniform(shape, lo, hi, dtype, d)
            elif kind == 1:
                h.randint(low, high, shape, dtype, d)
            else:
                h.normal(shape, mean, std, dtype, d)
            return h.rand([3], DT.F64, "cpu").to(GPU)

        g, c = both(s, after)
        assert_bitwise(g, c.to("cpu"), what + ": the generator afterwards")
