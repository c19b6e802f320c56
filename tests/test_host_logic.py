"""Host-side logic of the path (no GPU): promotion, casting rules, broadcasting, view strides and
dimension merging, checked against the known answers that homura's own unit tests hold.

ref: src/dtype.rs:541-609 (promotion_table, result_type_priorities, casting_rules),
     src/shape.rs:779-815 (broadcasting, view_strides, contiguity),
     src/backend/rocm/tests.rs:545-568 (kernel_dimensions_merge_like_the_cpu_plan),
     src/backend/cpu/iter.rs:112-129 (contiguous_and_transposed, extreme strides).
"""
import numpy as np
import pytest

from tests.support import DT, DTYPES, h


def test_promotion_table():
    p = h.promote_types
    assert p(DT.U8, DT.I8) == DT.I16
    assert p(DT.U8, DT.I32) == DT.I32
    assert p(DT.I16, DT.I32) == DT.I32
    assert p(DT.F16, DT.BF16) == DT.F32
    assert p(DT.BF16, DT.F64) == DT.F64
    assert p(DT.I64, DT.F16) == DT.F16
    assert p(DT.Bool, DT.U8) == DT.U8
    for d in DTYPES:
        assert p(d, d) == d
        assert p(DT.Bool, d) == d


def test_promotion_is_commutative_and_matches_the_lattice():
    """Independent of the implementation's table: a promoted type can hold both operands' categories
    (bool < integer < float), is never narrower than either operand within a category, and the
    operation is commutative and idempotent."""
    cat = {DT.Bool: 0, DT.U8: 1, DT.I8: 1, DT.I16: 1, DT.I32: 1, DT.I64: 1, DT.F16: 2, DT.BF16: 2, DT.F32: 2, DT.F64: 2}
    width = {DT.Bool: 1, DT.U8: 1, DT.I8: 1, DT.I16: 2, DT.I32: 4, DT.I64: 8, DT.F16: 2, DT.BF16: 2, DT.F32: 4, DT.F64: 8}
    for a in DTYPES:
        for b in DTYPES:
            r = h.promote_types(a, b)
            assert r == h.promote_types(b, a)
            assert cat[r] == max(cat[a], cat[b])
            assert h.promote_types(r, a) == r and h.promote_types(r, b) == r
            for x in (a, b):
                if cat[x] == cat[r]:
                    assert width[r] >= width[x]
            # Integers never promote to a float here, and a float beats any integer without widening.
            if cat[a] == 2 and cat[b] < 2:
                assert r == a


def test_result_type_priorities():
    rt = h.result_type
    assert rt([(DT.F16, 1)], [2.0]) == DT.F16          # f16 tensor * float scalar stays f16
    assert rt([(DT.I32, 1)], [2.5]) == DT.F32          # integer tensor * float scalar -> default dtype
    assert rt([(DT.I64, 2), (DT.F64, 0)], []) == DT.F64  # 0-dim tensor of a higher category wins
    assert rt([(DT.F32, 2), (DT.F64, 0)], []) == DT.F32  # ... but not within a category
    assert rt([(DT.U8, 1)], [-1]) == DT.U8
    assert rt([(DT.Bool, 1)], [1]) == DT.I64
    # The promotion of BASELINE configs[1]: bf16 tensor + f32 tensor.
    assert rt([(DT.BF16, 3), (DT.F32, 3)], []) == DT.F32


def test_casting_rules():
    assert h.can_cast(DT.I64, DT.F16)
    assert not h.can_cast(DT.F32, DT.I64)
    assert not h.can_cast(DT.I32, DT.Bool)
    assert h.can_cast(DT.Bool, DT.Bool)
    assert h.can_cast(DT.F64, DT.F16)


def test_broadcasting():
    assert h.broadcast_shapes([3, 1, 5], [4, 1]) == [3, 4, 5]
    assert h.broadcast_shapes([], [2]) == [2]
    assert h.broadcast_shapes([8, 2048, 4096], [4096]) == [8, 2048, 4096]
    assert h.broadcast_shapes([8, 2048, 1], [8, 2048, 4096]) == [8, 2048, 4096]
    with pytest.raises(Exception, match="must match the size"):
        h.broadcast_shapes([3], [4])


def test_view_strides_and_contiguity():
    assert h.compute_view_strides([2, 3, 4], [12, 4, 1], [6, 4]) == [4, 1]
    assert h.compute_view_strides([3, 2], [1, 3], [6]) is None          # a transposed matrix can't be flattened
    assert h.compute_view_strides([3, 2], [1, 3], [3, 1, 2]) == [1, 6, 3]  # size-1 dims go anywhere
    assert h.is_contiguous([2, 1, 3], [3, 100, 1])
    assert not h.is_contiguous([2, 3], [1, 2])
    assert h.contiguous_strides([2, 0, 3]) == [3, 3, 1]


def test_merge_dims_known_answers():
    m = h.merge_dims
    assert m([2, 1, 3, 4], [[12, 12, 4, 1]]) == [(24, [1])]
    assert m([2, 3], [[3, 1], [1, 2]]) == [(2, [3, 1]), (3, [1, 2])]
    assert m([4, 3, 5], [[0, 0, 0]]) == [(60, [0])]
    assert m([0, 3], [[3, 1]]) is None
    assert m([], [[]]) == []
    # stride * size overflows the index type: not merged.
    half = (1 << 62)
    assert len(m([2, 2], [[0, half * 2 - 1]])) == 2


def test_merge_dims_of_the_baseline_configs():
    """The merged dimensions decide the kernel variant; these are the forms the BASELINE shapes take."""
    m = h.merge_dims
    # cfg1: contiguous -> one dimension.
    assert m([4096, 4096], [[4096, 1]] * 3) == [(4096 * 4096, [1, 1, 1])]
    # cfg2 step 1: out, x contiguous, bias [4096] expanded (strides 0,0,1) -> rows x columns.
    assert m([8, 2048, 4096], [[8388608, 4096, 1], [8388608, 4096, 1], [0, 0, 1]]) == [
        (16384, [4096, 4096, 0]), (4096, [1, 1, 1])]
    # cfg2 step 2: scale [8,2048,1] expanded (strides 2048,1,0).
    assert m([8, 2048, 4096], [[8388608, 4096, 1], [8388608, 4096, 1], [2048, 1, 0]]) == [
        (16384, [4096, 4096, 1]), (4096, [1, 1, 0])]
    # cfg4: [8,2048,32,128].permute(0,2,1,3) read into a contiguous output: four dimensions remain.
    assert m([8, 32, 2048, 128], [[8388608, 262144, 128, 1], [8388608, 128, 4096, 1]]) == [
        (8, [8388608, 8388608]), (32, [262144, 128]), (2048, [128, 4096]), (128, [1, 1])]


def test_merge_dims_preserves_every_offset():
    """Brute force on small shapes: walking the merged dimensions visits the same operand offsets, in
    the same order, as walking the original ones."""
    rng = np.random.default_rng(7)

    def walk(shape, strides):
        offs = np.zeros((1, len(strides)), dtype=np.int64)
        for d, n in enumerate(shape):
            step = np.array([s[d] for s in strides], dtype=np.int64)
            offs = (offs[:, None, :] + np.arange(n)[None, :, None] * step[None, None, :]).reshape(-1, len(strides))
        return offs

    for _ in range(200):
        nd = int(rng.integers(1, 5))
        shape = [int(rng.integers(1, 5)) for _ in range(nd)]
        ops = []
        for _ in range(int(rng.integers(1, 4))):
            kind = int(rng.integers(0, 3))
            st = h.contiguous_strides(shape)
            if kind == 1:  # broadcast some dims
                st = [0 if rng.integers(0, 2) else s for s in st]
            elif kind == 2:  # permuted storage
                perm = rng.permutation(nd)
                base = h.contiguous_strides([shape[i] for i in perm])
                st = [0] * nd
                for k, i in enumerate(perm):
                    st[i] = base[k]
            ops.append(st)
        merged = h.merge_dims(shape, ops)
        assert merged is not None
        mshape = [s for s, _ in merged]
        mstrides = [[st[k] for _, st in merged] for k in range(len(ops))]
        assert all(s != 1 for s in mshape) or int(np.prod(shape)) == 1
        np.testing.assert_array_equal(walk(shape, ops), walk(mshape, mstrides))


def test_dims_mask():
    assert h.dims_mask([], 3) == [True, True, True]            # no dims = all dims
    assert h.dims_mask([-1], 3) == [False, False, True]
    assert h.dims_mask([0, 2], 3) == [True, False, True]
    with pytest.raises(Exception, match="multiple times"):
        h.dims_mask([0, -3], 3)
    with pytest.raises(Exception):
        h.dims_mask([3], 3)


def test_scalar_bits():
    """Scalars cross the C ABI as the bit pattern of the compute dtype, zero-extended to 64 bits
    (ref: src/backend/rocm/copy.rs:255-270)."""
    sb = h.scalar_bits
    assert sb(1.0, DT.F32) == 0x3F800000
    assert sb(1.0, DT.F64) == 0x3FF0000000000000
    assert sb(1.0, DT.F16) == 0x3C00
    assert sb(1.0, DT.BF16) == 0x3F80
    assert sb(-1, DT.I8) == 0xFF
    assert sb(-1, DT.I64) == 0xFFFFFFFFFFFFFFFF
    assert sb(300, DT.U8) == 44
    assert sb(2, DT.Bool) == 1
    assert sb(1.0 / 3.0, DT.BF16) == 0x3EAB
    assert sb(-2.5, DT.I32) == 0xFFFFFFFE                      # truncation toward zero, then wrap


def test_the_remaining_views_follow_numpy_and_keep_the_references_messages():
    """view, expand_as, squeeze, squeeze_dim, unfold, as_strided (ref: src/tensor/view.rs): shapes, strides and offsets
    against numpy's views of the same buffer (sliding_window_view for unfold, as_strided itself), and the messages
    for a view that would need a copy, a window longer than the dimension and a view outside its storage."""
    from numpy.lib.stride_tricks import as_strided, sliding_window_view
    from tests import oracle
    from tests.support import array, tensor
    h.register_cpu_backend(oracle.backend_address())
    a = np.arange(2 * 1 * 3 * 1 * 4, dtype=np.int32).reshape(2, 1, 3, 1, 4)
    t = tensor(a, DT.I32, list(a.shape))

    def same(view, expected):
        assert view.shape == list(expected.shape), (view.shape, expected.shape)
        assert np.array_equal(array(view), expected)

    same(t.squeeze(), a.squeeze())
    same(t.squeeze_dim([1]), a.squeeze(1))
    same(t.squeeze_dim([0]), a)                      # not of size 1: left alone
    same(t.squeeze_dim([1, -2]), a.squeeze((1, 3)))
    same(t.squeeze_dim([]), a)                       # an empty list removes none
    same(t.squeeze().transpose(0, 1).squeeze(), a.squeeze().transpose(1, 0, 2))
    same(t.view([2, 3, 4]), a.reshape(2, 3, 4))
    same(t.view([-1, 4]), a.reshape(-1, 4))
    same(t.squeeze().transpose(1, 2).view([2, 4, 3, 1]), a.squeeze().transpose(0, 2, 1).reshape(2, 4, 3, 1))
    with pytest.raises(h.HomuraError) as e:
        t.squeeze().transpose(1, 2).view([2, 12])
    assert "view size is not compatible with input tensor's size and stride" in str(e.value)
    row = tensor(np.arange(4, dtype=np.int32), DT.I32, [4])
    same(row.expand_as(t), np.broadcast_to(np.arange(4, dtype=np.int32), a.shape))
    # unfold: every window of `size` elements, `step` apart, as a new last dimension.
    m = np.arange(30, dtype=np.int32).reshape(5, 6)
    tm = tensor(m, DT.I32, [5, 6])
    for dim, size, step in ((1, 3, 1), (1, 2, 2), (0, 2, 3), (-1, 6, 1), (0, 5, 7), (1, 0, 2)):
        windows = sliding_window_view(m, size, axis=dim % 2)[(slice(None, None, step),) if dim % 2 == 0 else (slice(None), slice(None, None, step))]
        same(tm.unfold(dim, size, step), windows)
    same(tensor(np.array([7], dtype=np.int32), DT.I32, []).unfold(0, 1, 1), np.array([7], dtype=np.int32))
    for call, message in ((lambda: tm.unfold(1, 7, 1), "maximum size for tensor at dimension 1 is 6 but size is 7"),
                          (lambda: tm.unfold(0, 2, 0), "step is 0 but must be > 0")):
        with pytest.raises(h.HomuraError) as e:
            call()
        assert message in str(e.value)
    # as_strided: overlapping windows and a diagonal; outside the storage it is refused with PyTorch's message.
    same(tm.as_strided([4, 3], [6, 1], 2), as_strided(m.reshape(-1)[2:], (4, 3), (24, 4)))
    same(tm.as_strided([5], [7], 0), m.diagonal())
    same(tm.as_strided([3, 3], [1, 1], 4), as_strided(m.reshape(-1)[4:], (3, 3), (4, 4)))
    same(tm.as_strided([0, 9], [100, 100], 1000), np.zeros((0, 9), dtype=np.int32))
    with pytest.raises(h.HomuraError) as e:
        tm.as_strided([4, 3], [8, 1], 5)
    assert str(e.value) == ("setStorage: sizes [4, 3], strides [8, 1], storage offset 5, and itemsize 4 requiring a storage "
                            "size of 128 are out of bounds for storage of size 120")
    with pytest.raises(h.HomuraError) as e:
        tm.as_strided([4, 3], [8], 0)
    assert "mismatch in length of strides and shape" in str(e.value)
    # Writing through a view whose elements overlap is refused; reading it is not.
    overlapping = tm.as_strided([3, 3], [1, 1], 4)
    with pytest.raises(h.HomuraError):
        overlapping.add_(1)
    assert array(overlapping.add(1)).tolist() == (as_strided(m.reshape(-1)[4:], (3, 3), (4, 4)) + 1).tolist()
