"""The device mirror of the ragged array (upload, item reads, list indexing, item writes,
writes through strided views), following the cases of the reference's
nengo_ocl/tests/test_clraggedarray.py:33-110."""

import numpy as np
import pytest

from helpers import RA, to_dev
from nengo_ocl_amd import raggedarray as ra

pytestmark = pytest.mark.gpu


def random_ra(rng, n, d, low=20, high=40):
    shapes = [tuple(rng.randint(low=low, high=high, size=d)) for _ in range(n)]
    return RA([rng.normal(size=s) for s in shapes])


def test_unit_and_small(queue, rng):
    val = np.float32(rng.randn())
    assert np.allclose(val, to_dev(queue, RA([val]))[0])
    A = RA([rng.normal(size=3) for _ in range(3)])
    assert ra.allclose(A, to_dev(queue, A).to_host())


@pytest.mark.parametrize("d, low, high", [(1, 3000, 4000), (2, 20, 40)])
def test_random_roundtrip(queue, rng, d, low, high):
    A = random_ra(rng, int(rng.randint(5, 10)), d, low, high)
    dA = to_dev(queue, A)
    back = dA.to_host()
    assert ra.allclose(A, back) and np.array_equal(back.buf, A.buf)
    for name in ("starts", "shape0s", "shape1s", "stride0s", "stride1s"):
        assert np.array_equal(getattr(dA, name), getattr(A, name))
        assert np.array_equal(getattr(dA, "cl_" + name).get(), getattr(A, name))


def test_getitem_and_getitems(queue, rng):
    A = random_ra(rng, 10, 2)
    dA = to_dev(queue, A)
    assert np.allclose(A[3], dA[3])
    sel = [1, 3, 7, 8]
    sub = dA[sel]
    assert ra.allclose(A[sel], sub.to_host())
    assert sub.dev_buf is dA.dev_buf  # a view: same device memory


def test_to_host_helper_and_reference_class_name(queue, rng):
    """The module-level `to_host` (clraggedarray.py:36-62): a strided section of the device
    buffer, bit for bit; `CLRaggedArray` is the device class under the reference's name."""
    from nengo_ocl_amd import hipraggedarray as hra

    A = random_ra(rng, 6, 2)
    dA = to_dev(queue, A)
    assert hra.CLRaggedArray is type(dA)
    for i in range(len(A)):
        got = hra.to_host(queue, dA.dev_buf, A.dtype, A.starts[i], (A.shape0s[i], A.shape1s[i]),
                          (A.stride0s[i], A.stride1s[i]))
        assert np.array_equal(got, A[i])
    # every second column of an item
    m, n = int(A.shape0s[2]), int(A.shape1s[2])
    got = hra.to_host(queue, dA.dev_buf, A.dtype, A.starts[2], (m, (n + 1) // 2),
                      (A.stride0s[2], 2 * A.stride1s[2]))
    assert np.array_equal(got, A[2][:, ::2])
    assert hra.to_host(queue, dA.dev_buf, A.dtype, 0, (0, 3), (3, 1)).shape == (0, 3)


def test_setitem(queue, rng):
    A = random_ra(rng, 3, 2)
    dA = to_dev(queue, A)
    v = rng.uniform(0, 1, size=A[0].shape)
    A[0] = v.astype(A.dtype)
    dA[0] = v.astype(dA.dtype)
    A[1] = 3
    dA[1] = 3
    assert ra.allclose(A, dA.to_host())


def test_discontiguous_setitem(queue, rng):
    A = random_ra(rng, 3, 2)
    A0 = np.array(A[0])
    a = A0[::3, ::2]
    v = rng.uniform(-1, 1, size=a.shape).astype(np.float32)
    assert a.size > 0
    A.add_views([A.starts[0]], [a.shape[0]], [a.shape[1]], [a.strides[0] // a.itemsize],
                [a.strides[1] // a.itemsize])
    dA = to_dev(queue, A)
    a[...] = v
    dA[-1] = v
    assert np.allclose(dA[0], A0)      # only the strided elements of item 0 changed
    assert np.allclose(dA[-1], v)
    assert np.allclose(dA[1], A[1])    # and nothing else


def test_bounds_are_checked_on_the_host(queue, rng):
    A = random_ra(rng, 2, 2)
    dA = to_dev(queue, A)
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray

    bad = HIPRaggedArray.from_buffer(queue, dA.dev_buf, [A.buf.size - 4], [3], [3], [3], [1])
    with pytest.raises(ValueError):
        bad.check_bounds("bad")
