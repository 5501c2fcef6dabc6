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


def buffer_differences(sim_a, sim_b, limit=12):
    """Where the signal buffers of two simulators of one model differ: a list of
    ``(signal name, number of differing elements, largest difference, first index)``,
    empty when every float has the same value (NaNs in the same places count as equal)."""
    # (the buffer as the host is shown it: currents that are not stored brought up to date,
    # signals that device memory holds a step ahead taken from their copy)
    a, b = sim_a.signal_buffer(), sim_b.signal_buffer()
    if a.shape != b.shape:
        return [("buffer sizes", a.size, b.size, -1)]
    bad = ~((a == b) | (np.isnan(a) & np.isnan(b)))
    if not bad.any():
        return []
    ra = sim_b.all_data
    out = []
    for i, base in enumerate(sim_b.all_bases):
        start = int(ra.starts[i])
        n = int(ra.shape0s[i]) * int(ra.shape1s[i])
        where = np.flatnonzero(bad[start:start + n])
        if len(where):
            diff = np.abs(a[start:start + n][where].astype(np.float64) - b[start:start + n][where])
            out.append((str(getattr(base, "name", i)), len(where), float(np.nanmax(diff)),
                        int(where[0])))
            if len(out) >= limit:
                break
    return out or [("outside every base", int(bad.sum()), 0.0, int(np.flatnonzero(bad)[0]))]


def assert_same_signals(sim_a, sim_b):
    """Every signal of the two simulators holds the same values; a failure names the
    signals that differ instead of printing two buffers."""
    diffs = buffer_differences(sim_a, sim_b)
    assert not diffs, "signals differ (name, elements, largest difference, first index): %s" % diffs
