"""Pins the CPU oracle (no GPU): every known answer homura's own tests hold for this path, plus what
the mathematics fixes (exact rational arithmetic, brute force, an independent libm), chosen so that a
dropped term, a wrong sign or index, or a wrong rounding step fails at least one of them.

ref: src/backend/cpu/num.rs:222-246 (erf table), src/dtype.rs:611-665 (element_cast,
     half_casts_round_through_f32), tests/tensor_api.rs:686-701 (scalars stay f32 for half products),
     tests/m0_boundaries.rs:122-154, 380-392, 468-480 (empty reductions, NaN/ties, softmax),
     tests/rocm_reduce.rs:526-653 (exact sums, special values, extreme softmax rows),
     src/backend/cpu/iter.rs:112-121 (iteration order).
"""
import math
from fractions import Fraction

import numpy as np
import pytest

from tests import oracle
from tests.support import DT, FLOATS, NP, array, bits, from_f64, h, tensor, to_f64

h.register_cpu_backend(oracle.backend_address())
L = oracle.lib()
INF = float("inf")
NAN = float("nan")


def f64t(values, shape=None):
    a = np.asarray(values, dtype=np.float64)
    return tensor(a, DT.F64, list(a.shape if shape is None else shape))


def vals(t):
    """Elements of a tensor as exact f64."""
    return to_f64(array(t).reshape(-1), t.dtype)


def ulps64(a, b):
    if a == b:
        return 0
    ia, ib = (np.array([v], dtype=np.float64).view(np.int64)[0] for v in (a, b))
    return abs(int(ia) - int(ib))


def round_to(dtype, q):
    """A rational rounded once to the dtype (halves through f32, as homura rounds them)."""
    v = np.float64(float(q))  # Fraction -> nearest f64, correctly rounded
    return float(to_f64(from_f64([v], dtype), dtype)[0])


# ---- erf -----------------------------------------------------------------------------------------------

ERF_TABLE = [(0.0, 0.0), (1e-10, 1.1283791670955126e-10), (0.5, 0.5204998778130465), (1.0, 0.8427007929497149),
             (2.0, 0.9953222650189527), (2.4999, 0.9995928300996666), (2.5, 0.999593047982555),
             (3.0, 0.9999779095030014), (4.0, 0.9999999845827421), (-1.5, -0.9661051464753108)]


def test_erf_table():
    for x, want in ERF_TABLE:
        assert ulps64(L.orc_erf(x), want) <= 3, (x, L.orc_erf(x), want)
    assert L.orc_erf(INF) == 1.0 and L.orc_erf(-INF) == -1.0
    assert math.isnan(L.orc_erf(NAN))
    assert L.orc_erf(7.0) == 1.0


def test_erf_against_an_independent_libm():
    """glibc's erf is a different algorithm (rational approximations); the series / continued fraction
    must agree with it to a few ulp everywhere, be odd, and switch branches at 1.5 and 6 without a step."""
    xs = np.concatenate([np.linspace(-6.5, 6.5, 5201), [1.4999999, 1.5, 1.5000001, 5.9999999, 6.0, 1e-300, -0.0]])
    worst = 0
    for x in xs:
        got, want = L.orc_erf(float(x)), math.erf(float(x))
        # The series multiplies by exp(-x*x), whose argument carries the rounding of x*x: a few ulp.
        assert abs(got - want) <= 8 * math.ulp(want) + 1e-300, (x, got, want)
        assert L.orc_erf(-float(x)) == -got
        worst = max(worst, ulps64(got, want))
    assert worst <= 8


# ---- integer powers --------------------------------------------------------------------------------------

def wrap(v, nbits):
    v &= (1 << nbits) - 1
    return v - (1 << nbits) if v >> (nbits - 1) else v


def test_int_pow_brute_force():
    for base in range(-128, 128):
        for e in range(0, 12):
            assert L.orc_int_pow_i8(base, e) == wrap(base ** e, 8), (base, e)
    for base in (-7, -2, -1, 0, 1, 2, 3, 10, 46341, 2147483647):
        for e in (0, 1, 2, 3, 5, 31, 32, 33, 63, 64):
            assert L.orc_int_pow_i32(wrap(base, 32), e) == wrap(base ** e, 32), (base, e)
            assert L.orc_int_pow_i64(base, e) == wrap(base ** e, 64), (base, e)
    # Negative exponents (ref: src/backend/cpu/num.rs:162-187): 1 -> 1, -1 -> +-1, else 0.
    for e in (-1, -2, -3, -64):
        assert L.orc_int_pow_i64(1, e) == 1
        assert L.orc_int_pow_i64(-1, e) == (1 if e % 2 == 0 else -1)
        assert L.orc_int_pow_i64(2, e) == 0 and L.orc_int_pow_i64(0, e) == 0 and L.orc_int_pow_i64(-5, e) == 0


# ---- conversions --------------------------------------------------------------------------------------------

def cast(values, src, dst):
    t = tensor(from_f64(values, src) if src != DT.F64 else np.asarray(values, dtype=np.float64), src, [len(values)])
    return array(t.to(dst)).reshape(-1)


def test_element_casts():
    assert cast([-1.7], DT.F32, DT.I32)[0] == -1
    assert tensor(np.array([300], dtype=np.int64), DT.I64, [1]).to(DT.U8).to_bytes() == bytes([44])
    assert cast([300.0], DT.F32, DT.U8)[0] == 44
    assert cast([-1.0], DT.F64, DT.U8)[0] == 255
    assert cast([-129.9], DT.F32, DT.I8)[0] == 127
    assert cast([-2.5], DT.F16, DT.U8)[0] == 254
    assert cast([NAN], DT.F64, DT.I32)[0] == 0
    assert cast([INF], DT.F64, DT.I64)[0] == np.iinfo(np.int64).max
    assert cast([INF], DT.F64, DT.I32)[0] == -1
    assert cast([1e30], DT.F32, DT.I16)[0] == -1
    assert cast([0.1], DT.F64, DT.Bool)[0] == 1
    assert tensor(np.array([1], dtype=np.uint8), DT.Bool, [1]).to(DT.F16).to_bytes() == (0x3C00).to_bytes(2, "little")
    assert cast([2.5], DT.F16, DT.F32)[0] == 2.5


def test_half_casts_round_through_f32():
    p = lambda e: 2.0 ** e
    assert cast([np.float32(1.0 + p(-8) + p(-21))], DT.F32, DT.BF16)[0] == 0x3F81
    assert cast([1.0 + p(-8) + p(-21)], DT.F64, DT.BF16)[0] == 0x3F81
    assert cast([1.0 + p(-8) + p(-40)], DT.F64, DT.BF16)[0] == 0x3F80
    assert cast([1.0 + p(-11) + p(-40)], DT.F64, DT.F16)[0] == 0x3C00

    def from_i64(v, dst):
        return vals(tensor(np.array([v], dtype=np.int64), DT.I64, [1]).to(dst))[0]

    assert from_i64((1 << 24) + 1, DT.BF16) == p(24)
    assert from_i64((1 << 24) + (1 << 16) + 1, DT.BF16) == p(24)
    assert from_i64((1 << 63) - 1, DT.BF16) == p(63)
    assert from_i64(70000, DT.F16) == INF
    assert math.isnan(vals(f64t([NAN]).to(DT.F16))[0])
    neg_nan = np.array([0xFFF8000000000000], dtype=np.uint64).view(np.float64)
    assert int(bits(tensor(neg_nan, DT.F64, [1]).to(DT.BF16))[0]) & 0x8000


def test_every_f32_to_bf16_rounding_against_integer_arithmetic():
    """Round-to-nearest-even on the bit pattern, restated with integers only, over a dense sample of
    f32 patterns including every exponent, ties and the carry into the exponent."""
    rng = np.random.default_rng(11)
    pat = np.concatenate([rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32),
                          (np.arange(0, 1 << 16, dtype=np.uint32) << 16) | np.uint32(0x8000),   # exact ties
                          (np.arange(0, 1 << 16, dtype=np.uint32) << 16) | np.uint32(0x8001),
                          (np.arange(0, 1 << 16, dtype=np.uint32) << 16) | np.uint32(0x7FFF)])
    f = pat.view(np.float32)
    got = array(tensor(f, DT.F32, [len(f)]).to(DT.BF16)).reshape(-1).astype(np.uint32)
    p = pat.astype(np.uint64)
    rounded = ((p + 0x7FFF + ((p >> 16) & 1)) >> 16) & 0xFFFF
    nan = (p & 0x7FFFFFFF) > 0x7F800000
    want = np.where(nan, ((p >> 16) | 0x0040) & 0xFFFF, rounded).astype(np.uint32)
    np.testing.assert_array_equal(got, want)


def test_f16_conversion_matches_numpy_ieee():
    """numpy's float16 is IEEE binary16 with round-to-nearest-even: an independent implementation."""
    rng = np.random.default_rng(12)
    f = rng.integers(0, 1 << 32, 300000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    f = f[~np.isnan(f)]
    got = array(tensor(f, DT.F32, [len(f)]).to(DT.F16)).reshape(-1)
    with np.errstate(all="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got, want)
    allh = np.arange(0, 1 << 16, dtype=np.uint16)
    wide = array(tensor(allh, DT.F16, [1 << 16]).to(DT.F32)).reshape(-1)
    ref = allh.view(np.float16).astype(np.float32)
    ok = (wide == ref) | (np.isnan(wide) & np.isnan(ref))
    assert ok.all()


# ---- elementwise ----------------------------------------------------------------------------------------------

def test_half_products_keep_the_scalar_in_f32():
    s = 1.0 / 3.0
    for dtype, mul, add, sub in [(DT.F16, 2.333984375, 7.33203125, 6.66796875), (DT.BF16, 2.328125, 7.34375, 6.65625)]:
        x = f64t([7.0]).to(dtype)
        assert vals(x.mul(s))[0] == mul
        assert vals(x.rdiv(s))[0] == 0.047607421875
        assert vals(x.add(s))[0] == add
        assert vals(x.sub(s))[0] == sub


def test_ieee_arithmetic_is_correctly_rounded():
    """+ - * / in f32 and the halves equal exact rational arithmetic rounded once to the dtype."""
    rng = np.random.default_rng(13)
    for dtype in (DT.F16, DT.BF16, DT.F32):
        a64 = rng.normal(0, 3, 400)
        b64 = rng.normal(0, 3, 400)
        a, b = tensor(from_f64(a64, dtype), dtype, [400]), tensor(from_f64(b64, dtype), dtype, [400])
        av, bv = vals(a), vals(b)
        for name, fn in (("add", lambda x, y: x + y), ("sub", lambda x, y: x - y), ("mul", lambda x, y: x * y),
                         ("div", lambda x, y: x / y)):
            got = vals(getattr(a, name)(b))
            for i in range(400):
                exact = fn(Fraction(float(av[i])), Fraction(float(bv[i])))
                if dtype == DT.F32:
                    want = float(np.float32(float(exact)))  # may double-round through f64: check below
                    # f64 -> f32 double rounding only matters within 2^-29 relative of an f32 tie; rule it out
                    lo, hi = np.nextafter(np.float32(want), np.float32(-INF)), np.nextafter(np.float32(want), np.float32(INF))
                    assert abs(exact - Fraction(want)) <= min(abs(exact - Fraction(float(lo))), abs(exact - Fraction(float(hi))))
                else:
                    # halves: computed in f32 then rounded to the half: two roundings, by definition of the reference
                    want = float(to_f64(from_f64([np.float64(np.float32(float(exact)))], dtype), dtype)[0])
                assert got[i] == want, (dtype, name, av[i], bv[i], got[i], want)


def test_unary_formulas_against_python_math():
    xs = np.array([-20.0, -3.0, -1.0, -0.5, -0.0, 0.0, 0.25, 1.0, 2.0, 10.0, 30.0])
    x = f64t(xs)
    want = {
        "sigmoid": [1 / (1 + math.exp(-v)) for v in xs],
        "silu": [v / (1 + math.exp(-v)) for v in xs],
        "gelu": [0.5 * v * (1 + math.erf(v * math.sqrt(0.5))) for v in xs],
        "gelu_tanh": [0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v * v * v))) for v in xs],
        "log_sigmoid": [min(v, 0.0) - math.log1p(math.exp(-abs(v))) for v in xs],
        "tanh": [math.tanh(v) for v in xs],
        "exp": [math.exp(v) for v in xs],
        "relu": [max(v, 0.0) for v in xs],
        "sign": [float(v > 0) - float(v < 0) for v in xs],
    }
    for name, w in want.items():
        got = vals(getattr(x, name)())
        for g, e, v in zip(got, w, xs):
            assert abs(g - e) <= 8 * math.ulp(e) + 1e-300, (name, v, g, e)
    # Special values (ref: src/backend/cpu/mod.rs:362-403).
    s = f64t([NAN, -0.0, INF, -INF])
    assert np.array_equal(vals(s.sign()), [0.0, 0.0, 1.0, -1.0])
    r = vals(s.relu())
    assert math.isnan(r[0]) and r[1] == 0 and r[2] == INF and r[3] == 0
    assert np.array_equal(array(s.logical_not()).reshape(-1), [0, 1, 0, 0])


def test_iteration_order_of_a_transposed_view():
    x = tensor(np.arange(6, dtype=np.int64), DT.I64, [3, 2]).transpose(0, 1)      # shape [2,3], strides [1,2]
    assert array(x.contiguous()).reshape(-1).tolist() == [0, 2, 4, 1, 3, 5]
    e = tensor(np.arange(3, dtype=np.int64), DT.I64, [3]).narrow(0, 1, 1).expand([3])
    assert array(e.contiguous()).reshape(-1).tolist() == [1, 1, 1]


# ---- reductions ---------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", FLOATS)
def test_exact_sums_means_variances(dtype):
    v = np.array([((i * 37) % 17) - 8.0 for i in range(256)]).reshape(8, 32)
    x = f64t(v).to(dtype)
    for d in (0, 1):
        n = v.shape[d]
        lines = np.moveaxis(v, d, -1).reshape(-1, n)
        sums = [sum(Fraction(int(e)) for e in line) for line in lines]
        means = [s / n for s in sums]
        var0 = [sum((Fraction(int(e)) - m) ** 2 for e in line) / n for line, m in zip(lines, means)]
        var1 = [sum((Fraction(int(e)) - m) ** 2 for e in line) / (n - 1) for line, m in zip(lines, means)]
        assert vals(x.sum_dim(d, False)).tolist() == [round_to(dtype, s) for s in sums]
        assert vals(x.mean_dim(d, False)).tolist() == [round_to(dtype, m) for m in means]
        assert vals(x.var_dim(d, 0, False)).tolist() == [round_to(dtype, q) for q in var0]
        got = vals(x.std_dim(d, 1, False))
        for g, q in zip(got, var1):
            want = float(to_f64(from_f64([math.sqrt(float(q))], dtype), dtype)[0])
            assert g == want
    # The mean divides the f64 sum, not its rounding to the dtype.
    m = {DT.F16: [1401.0, 1401.0, 1400.0], DT.F32: [16777215.0, 16777215.0, 16777213.0]}.get(dtype, [1.0, 2.0, 2.0])
    got = vals(f64t([m]).to(dtype).mean_dim(1, False))[0]
    assert got == round_to(dtype, Fraction(int(sum(m))) / 3)
    if dtype == DT.F16:
        assert got == 1401.0
    if dtype == DT.F32:
        assert got == 16777214.0
    assert vals(f64t([2.0, -0.5, 4.0, 0.25, -1.0, 8.0]).to(dtype).prod())[0] == 8.0
    # Too few elements for the correction: x / 0.
    w = f64t([[1.0, 3.0], [2.0, 2.0]]).to(dtype)
    for c in (2, 3):
        r = vals(w.var_dim(1, c, False))
        assert r[0] == INF and math.isnan(r[1])


@pytest.mark.parametrize("dtype", FLOATS)
def test_empty_and_special_reductions(dtype):
    e = tensor(np.zeros(0, dtype=NP[dtype]), dtype, [3, 0])
    assert vals(e.sum_dim(1, False)).tolist() == [0.0] * 3
    assert vals(e.prod_dim(1, False)).tolist() == [1.0] * 3
    assert np.isnan(vals(e.mean_dim(1, False))).all()
    assert np.isnan(vals(e.var_dim(1, 0, False))).all()
    assert array(e.all_dim(1, False)).reshape(-1).tolist() == [1, 1, 1]
    assert array(e.any_dim(1, False)).reshape(-1).tolist() == [0, 0, 0]
    with pytest.raises(Exception):
        e.max()
    with pytest.raises(Exception):
        e.min_dim(1, False)
    with pytest.raises(Exception):
        e.argmax()
    rows = [[1.0, NAN, 2.0, 3.0], [1.0, INF, 2.0, 3.0], [1.0, -INF, 2.0, 3.0], [INF, 1.0, -INF, 3.0], [0.0, INF, 2.0, 3.0]]
    x = f64t(rows).to(dtype)
    s = vals(x.sum_dim(1, False))
    assert math.isnan(s[0]) and s[1] == INF and s[2] == -INF and math.isnan(s[3]) and s[4] == INF
    p = vals(x.prod_dim(1, False))
    assert math.isnan(p[0]) and p[1] == INF and p[2] == -INF and p[3] == -INF and math.isnan(p[4])
    assert np.isnan(vals(x.var_dim(1, 1, False))).all()


def test_nan_ties_and_integer_reductions():
    x = f64t([[1.0, NAN, NAN], [4.0, 4.0, 2.0]])
    assert array(x.argmax_dim(1, False)).reshape(-1).tolist() == [1, 0]
    assert array(x.argmin_dim(1, False)).reshape(-1).tolist() == [1, 2]
    assert math.isnan(vals(x.max())[0])
    z = f64t([[0.0, -0.0], [-0.0, 0.0]])
    assert array(z.argmax_dim(1, False)).reshape(-1).tolist() == [0, 0]      # +0 / -0 tie: the first
    assert bits(z.max_dim(1, False)[0]).tolist() == [0, 1 << 63]
    u = tensor(np.array([0, 2], dtype=np.uint8), DT.U8, [2])
    assert u.any().dtype == DT.U8 and array(u.any()).item() == 1 and array(u.all()).item() == 0
    b = tensor(np.array([1, 0, 1], dtype=np.uint8), DT.Bool, [3])
    assert b.prod().dtype == DT.I64 and array(b.prod()).item() == 0
    big = tensor(np.array([2**63 - 1, 1], dtype=np.int64), DT.I64, [2])
    assert array(big.sum()).item() == -2**63


def test_sum_is_a_sequential_f64_fold():
    """Order matters in floating point: 1e16 + 1 + 1 + ... folded left to right in f64 loses every 1,
    while any pairwise or compensated order would not; the oracle must reproduce the sequential result."""
    v = np.array([1e16] + [1.0] * 64)
    assert vals(f64t(v).sum())[0] == 1e16
    assert vals(f64t(v[::-1].copy()).sum())[0] == 1e16 + 64
    # f32 input accumulates in f64, not f32: 2^24 + 1 + 1 ... is exact in f64.
    w = f64t([16777216.0] + [1.0] * 3).to(DT.F32)
    assert vals(w.sum())[0] == float(np.float32(16777219.0))


# ---- softmax ----------------------------------------------------------------------------------------------------------

def test_softmax_known_answers():
    x = f64t([[10000.0, 10001.0, 10002.0], [NAN, 1.0, 2.0]])
    p = vals(x.softmax(-1).to(DT.F32))
    assert abs(p[0] - 0.09003057) < 1e-6 and abs(p[1] - 0.24472848) < 1e-6 and abs(p[2] - 0.66524094) < 1e-6
    assert np.isnan(p[3:]).all()
    y = f64t([0.0, -INF])
    assert vals(y.softmax(0)).tolist() == [1.0, 0.0]
    assert vals(y.log_softmax(0)).tolist() == [0.0, -INF]
    t = f64t(3.0, [])
    assert vals(t.softmax(0))[0] == 1.0 and vals(t.log_softmax(-1))[0] == 0.0


@pytest.mark.parametrize("dtype", FLOATS)
def test_softmax_extreme_rows(dtype):
    big = {DT.F16: 6e4, DT.BF16: 3e38, DT.F32: 3e38, DT.F64: 1e300}[dtype]
    rows = [[-INF, -INF, -INF, -INF], [1.0, NAN, 2.0, 3.0], [1.0, INF, 2.0, 3.0], [big, -big, big, 0.0],
            [-big, -big, 1.0, -INF], [0.0, -0.0, 0.0, -0.0]]
    x = f64t(rows).to(dtype)
    s = vals(x.softmax(1)).reshape(6, 4)
    l = vals(x.log_softmax(1)).reshape(6, 4)
    assert np.isnan(s[:3]).all() and np.isnan(l[:3]).all()
    assert s[3].tolist() == [0.5, 0.0, 0.5, 0.0]
    assert l[3][1] <= -big and l[3][0] == round_to(dtype, Fraction(math.log(0.5)))
    assert s[4].tolist() == [0.0, 0.0, 1.0, 0.0] and l[4][2] == 0.0 and l[4][3] == -INF
    assert s[5].tolist() == [0.25] * 4
    one = f64t([[3.0], [-INF], [NAN]]).to(dtype)
    o = vals(one.softmax(1))
    assert o[0] == 1.0 and math.isnan(o[1]) and math.isnan(o[2])


def test_softmax_against_exact_arithmetic():
    """exp(x - max) from libm, then the sum and the quotient in exact rational arithmetic: the oracle's
    sequential f64 sum of 257 terms may differ from that by a few ulp (far below one dropped term, 1/257),
    and each row must sum to one."""
    rng = np.random.default_rng(21)
    x = rng.normal(0, 3, (16, 257))
    got = vals(f64t(x).softmax(-1)).reshape(16, 257)
    glog = vals(f64t(x).log_softmax(-1)).reshape(16, 257)
    for r in range(16):
        m = max(x[r])
        e = [Fraction(math.exp(v - m)) for v in x[r]]
        tot = sum(e)
        for c in range(257):
            want = float(e[c] / tot)
            assert abs(got[r, c] - want) <= 16 * math.ulp(want)
            wl = (x[r, c] - m) - math.log(float(tot))
            assert abs(glog[r, c] - wl) <= 16 * math.ulp(wl)
        assert abs(sum(Fraction(float(g)) for g in got[r]) - 1) < Fraction(1, 10**13)


# ---- fused optimizer steps: exact rational arithmetic with the roundings where the reference has them ------

def nearest_even(frac, dtype):
    """`frac` (a Fraction) rounded to nearest-even in F32 or F64, as a Fraction; finite normal results only."""
    if frac == 0:
        return Fraction(0)
    p = 24 if dtype == DT.F32 else 53
    sign, mag = (-1 if frac < 0 else 1), abs(frac)
    e = mag.numerator.bit_length() - mag.denominator.bit_length()
    if Fraction(2) ** e > mag:
        e -= 1
    scaled = mag / Fraction(2) ** (e - p + 1)  # in [2^(p-1), 2^p)
    q, r = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * r
    if twice > scaled.denominator or (twice == scaled.denominator and q % 2 == 1):
        q += 1
    return sign * q * Fraction(2) ** (e - p + 1)


@pytest.mark.parametrize("dtype", [DT.F32, DT.F64])
def test_fused_steps_round_once_where_the_reference_does(dtype):
    """ref: src/backend/cpu/mod.rs:540-567. ScaledAdd = R(a + alpha*b); Lerp = R(w*R(b-a) + a) or
    R((w-1)*R(b-a) + b); Addcmul = R(R(v*b)*c + a); Addcdiv = R(a + R(R(v*b)/c)), R = one rounding to the
    computation type. A product rounded before its sum (no FMA), or an FMA where the reference has none,
    differs from these on some of the 300 samples."""
    rng = np.random.default_rng(17)
    n = 300
    npdt = NP[dtype]
    a, b, c = ((rng.standard_normal(n) * 2.0 ** rng.integers(-3, 4, n)).astype(npdt) for _ in range(3))
    c = np.where(np.abs(c) < 0.01, npdt(0.5), c).astype(npdt)
    R = lambda f: nearest_even(f, dtype)
    F = lambda arr: [Fraction(float(v)) for v in arr]
    fa, fb, fc = F(a), F(b), F(c)
    ta, tb, tc = (tensor(v, dtype) for v in (a, b, c))

    def check(got, want, what):
        got = [Fraction(float(v)) for v in array(got)]
        bad = [i for i in range(n) if got[i] != want[i]]
        assert not bad, f"{what}: element {bad[0]}: {float(got[bad[0]])!r} != {float(want[bad[0]])!r} ({len(bad)} differ)"

    differs_without_fma = 0
    for v in (0.1, -0.3, 0.7, 1.0 / 3.0):
        s = Fraction(float(npdt(v)))  # the coefficient in the computation type
        check(h.scaled_add(ta, tb, v), [R(x + s * y) for x, y in zip(fa, fb)], f"scaled_add {v}")
        differs_without_fma += sum(R(x + s * y) != R(x + R(s * y)) for x, y in zip(fa, fb))
        if abs(v) < 0.5:
            want = [R(s * R(y - x) + x) for x, y in zip(fa, fb)]
        else:
            w1 = R(s - 1)
            want = [R(w1 * R(y - x) + y) for x, y in zip(fa, fb)]
        check(h.lerp_step(ta, tb, v), want, f"lerp {v}")
        check(h.addcmul_step(ta, tb, tc, v), [R(R(s * y) * z + x) for x, y, z in zip(fa, fb, fc)], f"addcmul {v}")
        check(h.addcdiv_step(ta, tb, tc, v), [R(x + R(R(s * y) / z)) for x, y, z in zip(fa, fb, fc)], f"addcdiv {v}")
    assert differs_without_fma > 20  # the samples do tell an FMA from a rounded product


def test_scaled_add_rounds_alpha_to_the_dtype_first():
    """ref: src/backend/cpu/mod.rs:543: alpha = down(of(alpha)).up(); the other steps keep their coefficient in
    the computation type (f32 for BF16)."""
    bf = lambda *v: tensor(from_f64(np.array(v, dtype=np.float64), DT.BF16), DT.BF16)
    # 0.1 in BF16 is 0.10009765625; a + that, rounded to BF16's 8 bits.
    assert list(vals(h.scaled_add(bf(1.0, 2.0, -3.0), bf(1.0, 1.0, 1.0), 0.1))) == [1.1015625, 2.09375, -2.90625]
    # 1 + 2^-9 is an f32 but rounds to 1 in BF16. As an f32 value: 512 * (1 + 2^-9) * 1 + 1.5 = 514.5, which is
    # 516 in BF16 (spacing 4); as a BF16 alpha: 512 + 1.5 = 513.5, which is 512.
    assert list(vals(h.addcmul_step(bf(1.5), bf(512.0), bf(1.0), 1.0 + 2.0 ** -9))) == [516.0]
    assert list(vals(h.scaled_add(bf(1.5), bf(512.0), 1.0 + 2.0 ** -9))) == [512.0]


# ---- addr: one kernel with the bits of the composition of pinned elementwise ops ------------------------------

def addr_values(dtype, n, seed):
    """Special values first, then random ones (ref: tests/gemm_writeback.rs:266-299)."""
    rng = np.random.default_rng(seed)
    if dtype == DT.Bool:
        return tensor((rng.standard_normal(n) > 0).astype(np.uint8), DT.Bool)
    if dtype not in FLOATS:
        special = np.array([0, 1, -1, 2 ** 63 - 1, -2 ** 63, 255, -128], dtype=np.int64)
        v = np.concatenate([special, (rng.standard_normal(n) * 1e6).astype(np.int64)])[:n]
        return tensor(v, DT.I64).to(dtype)
    special = np.array([NAN, -NAN, INF, -INF, 0.0, -0.0, 1e-40, -5.96e-8, 65504.0, 3.0e38, -1.0e300])
    v = np.concatenate([special, rng.standard_normal(n) * 8.0])[:n]
    return tensor(v, DT.F64).to(dtype)


def addr_composite(inp, v1, v2, beta, alpha, dtype):
    """ref: tests/gemm_writeback.rs:250-264: alpha scales vec1 (floats) or the outer product (integers, bools),
    then beta * input is added unless beta is zero; a coefficient of one is skipped."""
    scale = lambda t, s: t if float(s) == 1.0 else t.mul(s)
    outer = lambda a, b: a.unsqueeze(1).mul(b.unsqueeze(0))
    product = outer(scale(v1, alpha), v2) if dtype in FLOATS else scale(outer(v1, v2), alpha)
    if float(beta) == 0.0:
        return product
    return scale(inp, beta).add(product)


def addr_cases(dtype, device="cpu", n=13, m=12):
    """(what, input, v1, v2, beta, alpha) over coefficients of the dtype and input layouts
    (ref: tests/gemm_writeback.rs:301-375)."""
    if dtype == DT.Bool:
        coefficients = [False, True]
    elif dtype in FLOATS:
        raw = [0.0, 1.0, -1.0, 0.5, 2.0, -1.5, 0.1, 1e-30, INF, NAN]
        coefficients = [float(v) for v in vals(tensor(np.array(raw), DT.F64).to(dtype))]  # rounded to the dtype first
    else:
        coefficients = [0, 1, -1, 2, 3, 127]
    v1 = addr_values(dtype, 2 * n, 1).to(device).reshape([n, 2]).select(1, 1)  # every other element
    v2 = addr_values(dtype, m, 2).to(device)
    full = addr_values(dtype, n * m, 3).to(device)
    inputs = [full.reshape([n, m]), full.reshape([m, n]).transpose(0, 1), full.narrow(0, 0, m),
              full.narrow(0, 0, n).reshape([n, 1]), full.narrow(0, 0, 1), full.narrow(0, 0, 1).reshape([])]
    for k, inp in enumerate(inputs):
        for alpha in coefficients:
            for beta in coefficients:
                yield f"{dtype} input {k} alpha {alpha} beta {beta}", inp, v1, v2, beta, alpha


@pytest.mark.parametrize("dtype", [DT.F16, DT.BF16, DT.F32, DT.F64, DT.U8, DT.I8, DT.I16, DT.I32, DT.I64, DT.Bool])
def test_addr_gives_the_composites_bits(dtype):
    checked = 0
    for what, inp, v1, v2, beta, alpha in addr_cases(dtype):
        got, want = inp.addr(v1, v2, beta, alpha), addr_composite(inp, v1, v2, beta, alpha, dtype)
        assert got.shape == [13, 12] and got.dtype == dtype, what
        g, w = bits(got), bits(want)
        if dtype in FLOATS:
            nan = {DT.F16: lambda b: (b & 0x7FFF) > 0x7C00, DT.BF16: lambda b: (b & 0x7FFF) > 0x7F80,
                   DT.F32: lambda b: (b & 0x7FFFFFFF) > 0x7F800000,
                   DT.F64: lambda b: (b & np.uint64(0x7FFFFFFFFFFFFFFF)) > np.uint64(0x7FF0000000000000)}[dtype]
            same = (g == w) | (nan(g) & nan(w))
        else:
            same = g == w
        assert same.all(), f"{what}: element {np.nonzero(~same)[0][0]}"
        checked += 1
    assert checked >= (4 * 6 if dtype == DT.Bool else 100)


def test_addr_known_answers_and_coefficient_rules():
    """ref: tests/m0_followup.rs:150-222, tests/m0_m1_readiness.rs:66."""
    m = h.full([1, 1], 1, DT.I32, "cpu")
    v = h.full([1], 1, DT.I32, "cpu")
    assert array(m.addr(v, v, 2, 3)).tolist() == [[5]]
    b = tensor(np.array([1], dtype=np.uint8), DT.Bool)
    assert array(b.unsqueeze(0).addr(b, b, True, 2)).tolist() == [[1]]
    with pytest.raises(Exception, match="Boolean alpha only supported for Boolean results"):
        m.addr(v, v, 1, True)
    for beta, alpha in ((1.0, 1), (1, 2.0), (0.5, 0.5)):
        with pytest.raises(Exception, match="must not be a floating point number"):
            m.addr(v, v, beta, alpha)
    hh = h.full([1, 1], 1.0, DT.F16, "cpu")
    with pytest.raises(Exception, match="alpha=100000 cannot be converted to f16 without overflow"):
        hh.addr(hh.flatten(0, -1), hh.flatten(0, -1), 1, 1e5)
    with pytest.raises(Exception, match="vec1 must be a 1-D tensor, got 2-D tensor"):
        hh.addr(hh, hh.flatten(0, -1), 1, 1)
    # All three inputs take part in the promotion, a zero-dimensional self included.
    out = h.full([], 1.5, DT.F64, "cpu").addr(h.full([2], 2, DT.I32, "cpu"), h.full([3], 3.0, DT.F16, "cpu"), 1, 1)
    assert out.dtype == DT.F64 and array(out).tolist() == [[7.5] * 3] * 2
    # A zero or tiny alpha never meets the other factor's infinity: alpha scales vec1 first.
    big, two = tensor(np.array([3.0e38], dtype=np.float32), DT.F32), tensor(np.array([2.0], dtype=np.float32), DT.F32)
    got = array(h.full([1, 1], 0.0, DT.F32, "cpu").addr(big, two, 1, 1e-30))
    assert got.tolist() == [[np.float32(1e-30) * np.float32(3.0e38) * np.float32(2.0)]] and np.isfinite(got).all()


def test_in_place_operations_check_the_target_and_write_through_views():
    """add_ / mul_ / sub_ / clamp_ / masked_fill_ / copy_ / fill_ compute out of place and copy into the target
    (ref: src/ops/mod.rs:308-392, src/ops/binary.rs:225-242, 504-515, 594-692): known answers through views, the
    messages for a shape that would grow, a dtype that cannot be cast and a target whose elements share memory,
    and a copy onto an overlapping part of itself (ref: tests/rocm_copy.rs:180-183)."""
    base = tensor(np.arange(12, dtype=np.float32), DT.F32, [3, 4])
    col = base.narrow(1, 1, 2)                    # a strided view: the write lands in the base
    col.add_(tensor(np.array([10.0, 20.0], dtype=np.float32), DT.F32, [2])).mul_(2.0)
    assert array(base).tolist() == [[0, 22, 44, 3], [4, 30, 52, 7], [8, 38, 60, 11]]
    base.transpose(0, 1).sub_(1)
    assert array(base).tolist() == [[-1, 21, 43, 2], [3, 29, 51, 6], [7, 37, 59, 10]]
    base.clamp_(0, 40)
    assert array(base).tolist() == [[0, 21, 40, 2], [3, 29, 40, 6], [7, 37, 40, 10]]
    mask = tensor(np.array([1, 0, 0, 1], dtype=np.uint8), DT.Bool, [4])
    base.masked_fill_(mask, -5.0)
    assert array(base).tolist() == [[-5, 21, 40, -5], [-5, 29, 40, -5], [-5, 37, 40, -5]]
    # An integer target takes an integer result, and refuses a float one.
    ints = tensor(np.arange(6, dtype=np.int32), DT.I32, [6])
    ints.add_(tensor(np.ones(6, dtype=np.int64), DT.I64, [6])).mul_(3)
    assert array(ints).tolist() == [3, 6, 9, 12, 15, 18]
    for call, message in (
            (lambda: ints.mul_(0.5), "result type f32 can't be cast to the desired output type i32"),
            (lambda: ints.div_(2), "result type f32 can't be cast to the desired output type i32"),
            (lambda: tensor(np.zeros(4, dtype=np.float32), DT.F32, [4]).add_(base),
             "output with shape [4] doesn't match the broadcast shape [3, 4]"),
            (lambda: tensor(np.zeros(3, dtype=np.float32), DT.F32, [3]).expand([2, 3]).add_(1.0),
             "unsupported operation: more than one element of the written-to tensor may refer to a single memory "
             "location. Please deep_clone() the tensor before performing the operation."),
            (lambda: tensor(np.zeros(3, dtype=np.float32), DT.F32, [3]).expand([2, 3]).fill_(1.0),
             "unsupported operation: more than one element of the written-to tensor may refer to a single memory "
             "location. Please deep_clone() the tensor before performing the operation.")):
        with pytest.raises(Exception) as e:
            call()
        assert message in str(e.value), str(e.value)
    assert array(ints).tolist() == [3, 6, 9, 12, 15, 18]  # a refused operation wrote nothing
    # copy_: a transposed target, a broadcast source of another dtype (ref: tests/rocm_copy.rs:160-170).
    target = tensor(np.zeros(15, dtype=np.int8), DT.I8, [5, 3]).transpose(0, 1)
    target.copy_(tensor(np.array([1.9, -2.9, 300.0, 0.0, -0.5], dtype=np.float32), DT.F32, [1, 5]))
    assert array(target).tolist() == [[1, -2, 44, 0, 0]] * 3
    with pytest.raises(Exception):
        target.copy_(tensor(np.zeros(4, dtype=np.float32), DT.F32, [4]))
    x = tensor(np.arange(6, dtype=np.int64), DT.I64, [6])
    x.narrow(0, 1, 5).copy_(x.narrow(0, 0, 5))
    assert array(x).tolist() == [0, 0, 1, 2, 3, 4]
    x.fill_(7).narrow(0, 2, 2).zero_()
    assert array(x).tolist() == [7, 7, 0, 0, 7, 7]
    with pytest.raises(Exception):
        tensor(np.zeros(2, dtype=np.uint8), DT.U8, [2]).fill_(300)
    # The composites' in-place forms (ref: src/ops/composite.rs, addcmul_ / addcdiv_ / lerp_).
    f = lambda v: tensor(np.array(v, dtype=np.float32), DT.F32, [len(v)])
    y = f([1.0, 2.0, 3.0])
    y.addcmul_(f([2.0, 2.0, 2.0]), f([1.0, 0.5, 4.0]), 0.5).addcdiv_(f([1.0, 1.0, 1.0]), f([4.0, 2.0, 1.0]), 2.0)
    assert array(y).tolist() == [2.5, 3.5, 9.0]
    y.lerp_(f([4.5, 3.5, 1.0]), 0.5)
    assert array(y).tolist() == [3.5, 3.5, 5.0]


def test_the_references_known_answers_for_in_place_operations_and_overlapping_copies():
    in_place_known_answers("cpu")


def in_place_known_answers(device):
    """ref: tests/m0_boundaries.rs (as_strided_offset_bounds_and_independent_copy, overlap_copy_transpose_and_broadcast,
    rejected_writes_leave_destination_unchanged, composite_in_place_operations_preserve_aliases_and_values) and
    tests/tensor_api.rs (in_place_on_itself_and_overlapping_copy, in_place_casts_and_broadcasts and the four
    should_panic cases after them). Also run on the GPU (tests/test_rocm_elementwise.py)."""
    i64 = lambda v, shape=None: tensor(np.array(v, dtype=np.int64), DT.I64, shape if shape is not None else [len(v)], device)
    f32 = lambda v, shape=None: tensor(np.array(v, dtype=np.float32), DT.F32, shape if shape is not None else [len(v)], device)
    x = i64(np.arange(10))
    y = x.as_strided([2, 3], [4, 1], 1)
    assert array(y).reshape(-1).tolist() == [1, 2, 3, 5, 6, 7]
    y.copy_(i64([20, 30, 40]))
    assert array(x).tolist() == [0, 20, 30, 40, 4, 20, 30, 40, 8, 9]
    for bad in (lambda: x.as_strided([2, 3], [4, 1], 5), lambda: x.as_strided([2, 3], [1], 0)):
        with pytest.raises(h.HomuraError):
            bad()
    x = i64(np.arange(9)).view([3, 3])
    x.copy_(x.transpose(0, 1))
    assert array(x).reshape(-1).tolist() == [0, 3, 6, 1, 4, 7, 2, 5, 8]
    x.copy_(x.narrow(0, 0, 1))
    assert array(x).reshape(-1).tolist() == [0, 3, 6, 0, 3, 6, 0, 3, 6]
    y = i64(np.arange(6))
    y.narrow(0, 0, 5).copy_(y.narrow(0, 1, 5))
    assert array(y).tolist() == [1, 2, 3, 4, 5, 5]
    x = i64([1, 2, 3])
    for bad in (lambda: x.add_(f32(np.zeros(6), [2, 3])), lambda: x.copy_(i64([1, 2])), lambda: x.add_(0.5)):
        with pytest.raises(h.HomuraError):
            bad()
    assert array(x).tolist() == [1, 2, 3]
    assert array(i64([2, 3]).mul(4)).tolist() == [8, 12]
    # tensor_api.rs
    x = f32([1.0, 2.0, 3.0])
    x.add_(x)
    assert array(x).tolist() == [2.0, 4.0, 6.0]
    x.mul_(x.narrow(0, 0, 1))
    assert array(x).tolist() == [4.0, 8.0, 12.0]
    y = i64(np.arange(6))
    y.narrow(0, 1, 5).copy_(y.narrow(0, 0, 5))
    assert array(y).tolist() == [0, 0, 1, 2, 3, 4]
    half = tensor(np.zeros(6, dtype=np.uint16), DT.F16, [2, 3], device)
    half.add_(f32([1.0, 2.0, 3.0]))
    assert half.dtype == DT.F16 and to_f64(array(half), DT.F16).reshape(-1).tolist() == [1.0, 2.0, 3.0, 1.0, 2.0, 3.0]
    i = i64([1, 2, 3])
    i.mul_(2)
    assert array(i).tolist() == [2, 4, 6]
    i.copy_(f32([1.9, -1.9, 0.5]))
    assert array(i).tolist() == [1, -1, 0]
    for bad, message in ((lambda: i64([1, 2]).add_(1.5), "result type f32 can't be cast to the desired output type i64"),
                         (lambda: i64([1, 2]).div_(2), "result type f32 can't be cast to the desired output type i64"),
                         (lambda: f32(np.zeros(3)).add_(f32(np.zeros(6), [2, 3])),
                          "output with shape [3] doesn't match the broadcast shape [2, 3]"),
                         (lambda: f32(np.zeros(3), [1, 3]).expand([4, 3]).fill_(1.0),
                          "more than one element of the written-to tensor")):
        with pytest.raises(h.HomuraError) as e:
            bad()
        assert message in str(e.value), str(e.value)
    # m0_boundaries.rs: the composites, through an alias of the same storage.
    x = f32([2.0, 4.0])
    alias = x.view([2])
    a, b = f32([3.0, 6.0]), f32([2.0, 2.0])
    x.addcmul_(a, b, 1).addcdiv_(a, b, 2)
    assert array(alias).tolist() == [11.0, 22.0]
    x.lerp_(f32([0.0, 0.0]), 0.5).pow_(2).sub_(0.25).mul_(2).div_(4)
    assert array(alias).tolist() == [15.0, 60.375]
    x.clamp_(0, 20).masked_fill_(tensor(np.array([1, 0], dtype=np.uint8), DT.Bool, [2], device), -1)
    assert array(alias).tolist() == [-1.0, 20.0]


def test_more_known_answers_of_the_references_boundary_tests():
    boundary_known_answers("cpu")


def boundary_known_answers(device):
    """ref: tests/m0_boundaries.rs (noncontiguous_offset_kernels, scalar_reductions_views_and_softmax,
    view_strides_and_contiguous_alias_contract, the triangles of shape_operators_on_noncontiguous_inputs, the view and
    elementwise parts of empty_creation_views_and_broadcasting); what needs matmul, concat or stack is out of scope.
    Also run on the GPU (tests/test_rocm_elementwise.py)."""
    i64 = lambda v, shape=None: tensor(np.array(v, dtype=np.int64), DT.I64, shape if shape is not None else [len(v)], device)
    flat = lambda t: array(t).reshape(-1).tolist()
    x = i64(np.arange(24)).view([2, 3, 4]).narrow(2, 1, 2).permute([1, 0, 2])
    assert flat(x) == [1, 2, 13, 14, 5, 6, 17, 18, 9, 10, 21, 22]
    assert flat(x.sum_dim([0, 2], False)) == [33, 105]
    assert flat(x.max_dim(2, False)[0]) == [2, 14, 6, 18, 10, 22]
    assert flat(x.pow(2)) == [1, 4, 169, 196, 25, 36, 289, 324, 81, 100, 441, 484]
    assert x.to(DT.F16).is_contiguous()
    t = tensor(np.array([3.0], dtype=np.float32), DT.F32, [], device)
    for dim in (0, -1):
        assert t.sum_dim([dim], True).shape == []
        v, i = t.max_dim(dim, True)
        assert array(v).item() == 3.0 and array(i).item() == 0
        assert array(t.softmax(dim)).item() == 1.0 and array(t.log_softmax(dim)).item() == 0.0
        assert t.transpose(dim, dim).shape == []
    assert t.unsqueeze(-1).squeeze().shape == []
    assert array(t.var(0)).item() == 0.0 and math.isnan(array(t.var(1)).item())
    assert t.flatten(0, -1).shape == [1]
    source = i64(np.arange(12)).view([3, 4])
    strided = source.slice(1, 0, 4, 2)
    assert strided.strides == [4, 2] and strided.view([6]).strides == [2]
    strided.view([6]).fill_(9)
    assert flat(source) == [9, 1, 9, 3, 9, 5, 9, 7, 9, 9, 9, 11]
    copied = source.transpose(0, 1).contiguous()
    copied.fill_(-1)
    assert array(source.select(0, 0).select(0, 0)).item() == 9
    expanded = i64([7]).expand([3, 4])
    assert flat(expanded) == [7] * 12
    with pytest.raises(h.HomuraError):
        expanded.copy_(i64(np.ones(12), [3, 4]))
    tt = i64(np.arange(6)).view([2, 3]).transpose(0, 1)
    assert flat(tt.triu(1)) == [0, 3, 0, 0, 0, 0] and flat(tt.tril(-1)) == [0, 0, 1, 0, 2, 5]
    with pytest.raises(h.HomuraError):
        tt.flip([0, -2])
    for dtype in (DT.Bool, DT.U8, DT.I64, DT.F16, DT.BF16, DT.F32, DT.F64):
        e = tensor(np.zeros(0, dtype=NP[dtype]), dtype, [2, 0, 3], device)
        assert e.num_elements() == 0 and e.is_contiguous()
        assert e.to(dtype).shape == [2, 0, 3] and e.transpose(0, 2).reshape([0, 6]).shape == [0, 6]
        assert e.add(tensor(np.ones(3, dtype=NP[dtype]), dtype, [1, 3], device)).shape == [2, 0, 3]
        assert e.flip([0, 2]).shape == [2, 0, 3]
    assert tensor(np.zeros(0, dtype=np.float32), DT.F32, [0], device).view([-1, 3]).shape == [0, 3]
