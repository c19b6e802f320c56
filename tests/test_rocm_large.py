"""Tensors of more than 2^31 elements: offsets, element counts and reduction lengths that need 64 bits.

2 147 487 747 u8 elements (2^31 + 4099: odd, so the last 16-byte tile is ragged) go through a contiguous
binary op, a copy out of a transposed view, a comparison, a full sum and a row sum; every result is compared
element for element with numpy, which is exact for these integer ops.
"""
import numpy as np
import pytest

from tests.support import DT, GPU, array, tensor

pytestmark = pytest.mark.gpu

N = (1 << 31) + 4099


def pattern(n, mul):
    """n bytes with a period of 1 000 003 (prime): cheap to build and different in every 16-byte tile."""
    base = ((np.arange(1_000_003, dtype=np.uint64) * np.uint64(mul)) >> np.uint64(7)).astype(np.uint8)
    return np.resize(base, n)


def test_more_than_two_to_the_31_elements():
    a, b = pattern(N, 2654435761), pattern(N, 40503)
    x, y = tensor(a, DT.U8, [N], GPU), tensor(b, DT.U8, [N], GPU)
    # Contiguous binary op, wrapping in u8.
    got = array(x.add(y))
    assert got.shape == (N,) and np.array_equal(got, a + b)
    del got
    # A conversion (one input; the output is large enough for the streaming stores).
    got = array(x.to(DT.I8))
    assert np.array_equal(got, a.astype(np.int8))
    del got
    # A comparison into bool.
    got = array(x.greater(y))
    assert np.array_equal(got, (a > b).astype(np.uint8))
    del got
    # The full sum and the sums of two rows of 2^30 + 2049 elements (I64 results).
    assert int(array(x.sum()).reshape(-1)[0]) == int(a.sum(dtype=np.int64))
    half = (N - 1) // 2
    rows = x.narrow(0, 1, N - 1).reshape([2, half])
    assert array(rows.sum_dim(1, False)).tolist() == a[1:].reshape(2, half).sum(axis=1, dtype=np.int64).tolist()
    # Column sums of the same view: 2^30 + 2049 outputs of two elements each.
    got = array(rows.sum_dim(0, False))
    assert np.array_equal(got, a[1:].reshape(2, half).sum(axis=0, dtype=np.int64))
    del got
    # A copy out of the transposed view (strides 1 and 2^30 + 2049, an offset of 1).
    got = array(rows.transpose(0, 1).contiguous())
    assert got.shape == (half, 2) and np.array_equal(got, a[1:].reshape(2, half).T)
