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


PHILOX_KNOWN_ANSWERS = [
    # counter, key -> output: the generator's published test vectors (Random123 kat_vectors,
    # philox4x32 with 10 rounds)
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]
