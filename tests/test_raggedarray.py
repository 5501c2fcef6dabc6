"""Host ragged array: layout, views, alignment (cases of the reference's
tests/test_clraggedarray.py :33-117 that concern the host class)."""

import numpy as np
import pytest

from helpers import RA
from nengo_ocl_amd import raggedarray as ra
from nengo_ocl_amd.raggedarray import RaggedArray


def test_shape_zeros():
    A = RA([[]])
    assert A[0].shape == (0, 1)


def test_layout_fields_and_roundtrip(rng):
    vals = [rng.normal(size=s).astype(np.float32) for s in [(3,), (4, 5), (), (1, 7)]]
    A = RA(vals)
    assert list(A.starts) == [0, 3, 23, 24]
    assert list(A.shape0s) == [3, 4, 1, 1] and list(A.shape1s) == [1, 5, 1, 7]
    assert list(A.stride0s) == [1, 5, 1, 7] and list(A.stride1s) == [1, 1, 1, 1]
    assert A.buf.dtype == np.float32 and A.buf.size == 31 and A.nbytes == 31 * 4
    for v, item in zip(vals, A):
        assert np.array_equal(np.atleast_1d(v).reshape(item.shape), item)
    assert all(a.dtype == np.int32 for a in (A.starts, A.shape0s, A.shape1s, A.stride0s, A.stride1s))


def test_alignment_policies():
    sizes = [3, 20, 9, 1, 17]
    arrays = [np.ones(s) for s in sizes]
    packed = RA(arrays)
    assert list(packed.starts) == [0, 3, 23, 32, 33]
    aligned = RA(arrays, align=True)
    assert all(s % 16 == 0 for s, n in zip(aligned.starts, sizes) if n >= 4)
    ref = RA(arrays, align="reference")  # 16 for >= 16 elements, 4 for >= 8, else packed
    assert list(ref.starts) == [0, 16, 36, 45, 48]
    for A in (packed, aligned, ref):
        for i, n in enumerate(sizes):
            assert A[i].shape == (n, 1) and np.all(A[i] == 1)
        assert A.buf.sum() == sum(sizes)  # padding is zero


def test_getitems_share_the_buffer(rng):
    A = RA([rng.normal(size=(n, 3)) for n in range(2, 12)])
    sub = A[[1, 3, 7, 8]]
    assert len(sub) == 4 and sub.buf is A.buf
    assert np.array_equal(sub[2], A[7])
    sub[0] = 5.0
    assert np.all(A[1] == 5.0)
    assert len(A[2:5]) == 3


def test_setitem_and_discontiguous_view(rng):
    A = RA([rng.normal(size=(9, 8)), rng.normal(size=(5,))])
    A0 = np.array(A[0])
    a = A0[::3, ::2]
    A.add_views([A.starts[0]], [a.shape[0]], [a.shape[1]], [a.strides[0] // 4], [a.strides[1] // 4])
    v = rng.uniform(-1, 1, size=a.shape).astype(np.float32)
    a[...] = v
    A[-1] = v
    assert np.allclose(A[0], A0) and np.allclose(A[-1], v)
    with pytest.raises(NotImplementedError):
        A[[0, 1]] = 1.0


def test_add_views_rejects_overrun():
    A = RA([np.zeros(10)])
    with pytest.raises(ValueError):
        A.add_views([5], [10], [1], [1], [1])


def test_allclose_and_type_checks():
    A = RA([[1.0, 2.0], [3.0]])
    B = RA([[1.0, 2.0], [3.0 + 1e-6]])
    assert ra.allclose(A, B)
    assert not ra.allclose(A, RA([[1.0, 2.0, 3.0]]))
    with pytest.raises(TypeError):
        RaggedArray([np.zeros(3, dtype=np.float64)])
    I = RA([[1, 2], [3]], dtype=np.int32)
    assert I.ctype == "int" and A.ctype == "float"


def test_offsets_beyond_int32_are_refused():
    """Offsets are int32 element counts (reference raggedarray.py:107-111): metadata that
    does not fit is refused instead of wrapping around."""
    buf = np.zeros(8, dtype=np.float32)
    with pytest.raises(ValueError, match="2\\^31"):
        RaggedArray.from_buffer(buf, [0, 2 ** 31], [1, 1], [1, 1], [1, 1], [1, 1])
    with pytest.raises(ValueError, match="2\\^31"):
        RaggedArray.from_buffer(buf, np.array([0, 2 ** 31 + 5], dtype=np.int64), [1, 1], [1, 1],
                                [1, 1], [1, 1])


def test_small_helpers_under_the_reference_names():
    """nengo_ocl/utils.py:16-57: `as_ascii`, `equal_strides`, `nonelist`,
    `round_up_power_of_2`; `HostSparseMatrix` is reachable from `utils` as there."""
    from nengo_ocl_amd import utils

    assert utils.as_ascii(b"abc") == "abc" and utils.as_ascii("x") == "x" and utils.as_ascii(3) == "3"
    assert utils.equal_strides((8, 4), (8, 4), (3, 2))
    assert utils.equal_strides((99, 4), (8, 4), (1, 2))      # an axis of length one may differ
    assert not utils.equal_strides((16, 4), (8, 4), (3, 2))
    assert not utils.equal_strides((8,), (8, 4), (3, 2))
    assert utils.nonelist(1, None, "a", None) == [1, "a"]
    assert [utils.round_up_power_of_2(v) for v in (0, 0.5, 1, 3, 4, 5, 1000, -3)] == [
        1, 1, 1, 4, 4, 8, 1024, -4]
    from nengo_ocl_amd.hipra_spmv import HostSparseMatrix

    assert utils.HostSparseMatrix is HostSparseMatrix
