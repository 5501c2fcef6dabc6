"""Shared helpers for the parity tests."""

import numpy as np

from nengo_ocl_amd.raggedarray import RaggedArray


def RA(arrays, dtype=np.float32, **kw):
    return RaggedArray(arrays, dtype=dtype, **kw)


def clone(ra):
    """An independent host copy (same metadata, own buffer)."""
    return RaggedArray.from_buffer(
        np.array(ra.buf), ra.starts, ra.shape0s, ra.shape1s, ra.stride0s, ra.stride1s, names=ra.names
    )


def to_dev(queue, ra):
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray

    return HIPRaggedArray(queue, ra)


def run_plans(plans):
    for p in plans:
        p()
