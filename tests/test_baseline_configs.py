"""The five BASELINE configurations at their full sizes on the GPU.

Every result is compared with the single-threaded CPU oracle as a whole (bit-exact for IEEE arithmetic,
integers, comparisons and where; within 1 ulp of the output dtype for transcendentals, reductions and
softmax) - the bf16 unary ops of configs[3] through the oracle's results for all 65 536 patterns - and held
to size-independent properties besides: agreement between the strided and the contiguous kernel variants,
numpy's exact integer arithmetic, rows summing to one, masked entries exactly 0 / -inf.
"""
import numpy as np
import pytest

from tests import oracle
from tests.support import DT, GPU, array, assert_bitwise, assert_same, check_within, from_f64, h, normal, tensor, to_f64, uniform, words

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())


def test_config_0_contiguous_f32_add_is_bit_exact():
    n = 4096 * 4096
    a = uniform(0x5EED0100, n, -1.0, 1.0).astype(np.float32)
    b = uniform(0x5EED0101, n, -1.0, 1.0).astype(np.float32)
    ca, cb = tensor(a, DT.F32, [4096, 4096]), tensor(b, DT.F32, [4096, 4096])
    gpu = ca.to(GPU).add(cb.to(GPU))
    assert_same(gpu, ca.add(cb), "cfg0 add")
    np.testing.assert_array_equal(array(gpu).reshape(-1), a + b)          # numpy's IEEE add, a second opinion


def test_config_1_broadcast_chain_with_promotion_is_bit_exact():
    B, S, H = 8, 2048, 4096
    N = B * S * H
    x = tensor(from_f64(normal(0x5EED0001, N), DT.BF16), DT.BF16, [B, S, H])
    bias = tensor(from_f64(normal(0x5EED0002, H, 0.0, 0.02), DT.BF16), DT.BF16, [H])
    scale = tensor(from_f64(uniform(0x5EED0003, B * S, 0.5, 1.5), DT.BF16), DT.BF16, [B, S, 1])
    res = tensor(normal(0x5EED0004, N).astype(np.float32), DT.F32, [B, S, H])
    cpu = x.add(bias).mul(scale).add(res)
    gx, gb, gs, gr = (t.to(GPU) for t in (x, bias, scale, res))
    gpu = gx.add(gb).mul(gs).add(gr)
    assert gpu.dtype == DT.F32 and gpu.shape == [B, S, H]
    assert_same(gpu, cpu, "cfg1 chain (fused promotion)")
    h.set_fused_promotion(False)
    try:
        assert_same(gx.add(gb).mul(gs).add(gr), cpu, "cfg1 chain (cast kernel + add)")
    finally:
        h.set_fused_promotion(True)
    # Each intermediate too: two bf16 roundings.
    assert_same(gx.add(gb), x.add(bias), "cfg1 step 1")
    assert_same(gx.add(gb).mul(gs), x.add(bias).mul(scale), "cfg1 step 2")
    # The broadcast operand first (another form of the kernel: which inputs go through the caches is chosen per
    # launch), and both operands broadcast (an outer sum of the bias and the scale).
    assert_same(gb.add(gx), x.add(bias), "cfg1 step 1, bias first")
    assert_same(gs.mul(gx.add(gb)), x.add(bias).mul(scale), "cfg1 step 2, scale first")
    assert_same(gs.add(gb), scale.add(bias), "bias + scale, both broadcast")


def test_config_2_reductions_stay_within_one_ulp():
    R, C = 16384, 4096
    v = normal(0x5EED0004, R * C).astype(np.float32)
    x = tensor(v, DT.F32, [R, C])
    g = x.to(GPU)
    for dim in (-1, 0):
        check_within(g.sum_dim(dim, False), x.sum_dim(dim, False), what=f"cfg2 sum dim={dim}")
        check_within(g.mean_dim(dim, False), x.mean_dim(dim, False), what=f"cfg2 mean dim={dim}")
        check_within(g.var_dim(dim, 1, False), x.var_dim(dim, 1, False), what=f"cfg2 var dim={dim}")
        gv, gi = g.max_dim(dim, False)
        cv, ci = x.max_dim(dim, False)
        assert_same(gv, cv, f"cfg2 amax dim={dim}")
        assert_same(gi, ci, f"cfg2 argmax dim={dim}")
    check_within(g.sum(), x.sum(), what="cfg2 full sum")
    # The f64 accumulation is what keeps the full sum within an ulp: the exact sum of the f32 inputs
    # (integer arithmetic on scaled mantissas is overkill here; math.fsum is exact) rounds to the same f32
    # or its neighbour.
    import math
    exact = math.fsum(v.astype(np.float64))
    assert abs(float(array(g.sum()).item()) - exact) <= float(np.spacing(np.float32(abs(exact))))
    xb = x.to(DT.BF16)
    gb = g.to(DT.BF16)
    assert_same(gb, xb, "cfg2 bf16 copy")
    check_within(gb.sum_dim(-1, False), xb.sum_dim(-1, False), what="cfg2 bf16 sum dim=-1")
    # Reproducible from run to run.
    assert_same(g.sum_dim(0, False), g.sum_dim(0, False), "cfg2 sum dim=0 repeats")
    assert_same(g.sum(), g.sum(), "cfg2 full sum repeats")


def test_config_3_permuted_unary_and_int64_ops():
    N = 8 * 2048 * 32 * 128
    raw = from_f64(normal(0x5EED0400, N, 0.0, 2.0), DT.BF16)
    base = tensor(raw, DT.BF16, [8, 2048, 32, 128])
    gbase = base.to(GPU)
    p, gp = base.permute([0, 2, 1, 3]), gbase.permute([0, 2, 1, 3])
    for name in ("silu", "gelu"):
        full = getattr(gp, name)()
        assert full.is_contiguous() and full.shape == [8, 32, 2048, 128]
        # Strided variant == contiguous variant of the same data, everywhere.
        assert_same(full, getattr(gp.contiguous(), name)(), f"cfg3 {name}: permuted vs contiguous input")
        # The WHOLE result against the oracle, to 1 ulp of bf16: a unary op on bf16 is a function of 65 536 patterns,
        # so the oracle's results for all of them, indexed by the input's patterns, are its result for the tensor.
        every = tensor(np.arange(65536, dtype=np.uint16), DT.BF16)
        by_pattern = array(getattr(every, name)()).reshape(-1)
        want = by_pattern[raw.reshape(8, 2048, 32, 128).transpose(0, 2, 1, 3)]
        check_within(full, tensor(want, DT.BF16, [8, 32, 2048, 128]), what=f"cfg3 {name}, all 67 108 864 elements")
        del want
        # The oracle run directly on one batch entry agrees with its table (the oracle's own strided walk).
        check_within(getattr(gp.narrow(0, 3, 1), name)(), getattr(p.narrow(0, 3, 1), name)(), what=f"cfg3 {name} batch 3")
        assert_same(full.narrow(0, 3, 1).contiguous(), getattr(gp.narrow(0, 3, 1), name)(), f"cfg3 {name}: slice of full")
    del raw, base, gbase, p, gp
    a = (words(0x5EED0401, N) % np.uint64(2001)).astype(np.int64) - 1000
    b = (words(0x5EED0402, N) % np.uint64(2001)).astype(np.int64) - 1000
    assert a.min() == -1000 and a.max() == 1000
    ga, gb = tensor(a, DT.I64, [8, 2048, 4096], GPU), tensor(b, DT.I64, [8, 2048, 4096], GPU)
    band = ga.bitwise_and(gb)
    assert band.dtype == DT.I64
    np.testing.assert_array_equal(array(band).reshape(-1), a & b)
    mask = ga.greater(gb)
    assert mask.dtype == DT.Bool
    np.testing.assert_array_equal(array(mask).reshape(-1), (a > b).astype(np.uint8))
    sel = h.where_(mask, ga, gb)
    assert sel.dtype == DT.I64
    np.testing.assert_array_equal(array(sel).reshape(-1), np.maximum(a, b))
    # And the oracle agrees with numpy on a slice (pins the oracle's integer path at these values).
    ca, cb = tensor(a[:1 << 20], DT.I64, [1 << 20]), tensor(b[:1 << 20], DT.I64, [1 << 20])
    np.testing.assert_array_equal(array(ca.bitwise_and(cb)), a[:1 << 20] & b[:1 << 20])
    np.testing.assert_array_equal(array(h.where_(ca.greater(cb), ca, cb)), np.maximum(a[:1 << 20], b[:1 << 20]))


def row_sums(t):
    return to_f64(array(t), t.dtype).sum(axis=-1)


def test_config_4a_bf16_logits():
    R, C = 4096, 32000
    raw = from_f64(normal(0x5EED0500, R * C, 0.0, 3.0), DT.BF16)
    x = tensor(raw, DT.BF16, [R, C])
    g = x.to(GPU)
    sm, lsm = g.softmax(-1), g.log_softmax(-1)
    # Every one of the 4096 rows against the oracle (a few seconds of f64 exponentials on one core), to 1 ulp of bf16.
    check_within(sm, x.softmax(-1), what="cfg4a softmax, all rows")
    check_within(lsm, x.log_softmax(-1), what="cfg4a log_softmax, all rows")
    # Every row: probabilities in [0, 1] summing to one within bf16 rounding of C terms; log-probabilities <= 0.
    p = to_f64(array(sm), DT.BF16)
    assert p.min() >= 0.0 and p.max() <= 1.0
    # Each term carries at most half a bf16 ulp (2^-9 relative): the sum is within 2^-9 of one.
    assert np.abs(p.sum(axis=-1) - 1.0).max() <= 2.0 ** -9
    lp = to_f64(array(lsm), DT.BF16)
    assert lp.max() <= 0.0
    # The largest logit of a row gets the largest probability.
    top = to_f64(raw, DT.BF16).reshape(R, C).argmax(axis=-1)
    np.testing.assert_array_equal(p[np.arange(R), top], p.max(axis=-1))


def test_config_4b_causal_f32_scores():
    Bh, T = 32, 2048
    s = normal(0x5EED0501, Bh * T * T).astype(np.float32).reshape(Bh, T, T)
    iu = np.triu_indices(T, 1)
    s[:, iu[0], iu[1]] = -np.inf
    x = tensor(s, DT.F32, [Bh, T, T])
    g = x.to(GPU)
    sm, lsm = g.softmax(-1), g.log_softmax(-1)
    # All 32 heads against the oracle, to 1 ulp of f32.
    check_within(sm, x.softmax(-1), what="cfg4b softmax, all heads")
    check_within(lsm, x.log_softmax(-1), what="cfg4b log_softmax, all heads")
    p = array(sm)
    lp = array(lsm)
    assert (p[:, iu[0], iu[1]] == 0.0).all(), "masked entries are exactly zero"
    assert np.isneginf(lp[:, iu[0], iu[1]]).all(), "masked entries are exactly -inf"
    assert not np.isnan(p).any() and not np.isnan(lp).any()
    assert (p[:, 0, 0] == 1.0).all() and (lp[:, 0, 0] == 0.0).all()        # the first row has one live entry
    sums = p.astype(np.float64).sum(axis=-1)
    # Each of up to T terms carries at most half an f32 ulp of itself: |sum - 1| <= 2^-24 (+ the f64 fold).
    assert np.abs(sums - 1.0).max() <= 2.0 ** -23
    live = np.tril(np.ones((T, T), dtype=bool))
    with np.errstate(all="ignore"):
        back = np.exp(lp.astype(np.float64))
    assert np.abs(back[:, live] - p[:, live]).max() <= 1e-6
