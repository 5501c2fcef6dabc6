"""Small host-side helpers shared by the planner and the plan builders.

Counterparts of the helpers in the reference's ``nengo_ocl/utils.py`` that the
timestep path needs (``round_up`` :48, ``split`` :56, ``stable_unique`` :69,
``get_closures`` :40, and the one-liners ``as_ascii`` :16, ``equal_strides`` :25,
``nonelist`` :48, ``round_up_power_of_2`` :56 under their names; ``HostSparseMatrix``
lives with the sparse products and is reachable from here as in the reference).  The
benchmark ``SimRunner`` registry of that file is not part of the timestep path and is
not provided.
"""

import numpy as np


def is_iterable(obj):
    """True for lists, tuples, ranges and ndarrays with ndim > 0."""
    if isinstance(obj, np.ndarray):
        return obj.ndim > 0
    if isinstance(obj, (str, bytes)):
        return False
    try:
        iter(obj)
    except TypeError:
        return False
    return True


def is_number(obj):
    return isinstance(obj, (int, float, np.integer, np.floating)) and not isinstance(
        obj, bool
    )


def round_up(x, n):
    """Smallest multiple of ``n`` that is >= ``x`` (integers)."""
    x, n = int(x), int(n)
    return -(-x // n) * n


def next_pow2(x):
    x = int(x)
    return 1 if x <= 1 else 1 << (x - 1).bit_length()


def split(items, criterion):
    """Partition ``items`` into (matching, not matching), order kept."""
    yes, no = [], []
    for item in items:
        (yes if criterion(item) else no).append(item)
    return yes, no


def stable_unique(seq):
    """Unique elements of ``seq`` in first-appearance order."""
    return list(dict.fromkeys(seq))


def groupby(objects, key):
    """Group ``objects`` by ``key(obj)`` keeping first-appearance order of keys.

    Keys are compared with ``==`` (not identity), like ``nengo.utils.stdlib.groupby``
    as the reference uses it (simulator.py:913-915).
    """
    keys, groups = [], []
    for obj in objects:
        k = key(obj)
        for i, k2 in enumerate(keys):
            if k2 is k or k2 == k:
                groups[i].append(obj)
                break
        else:
            keys.append(k)
            groups.append([obj])
    return list(zip(keys, groups))


def get_closures(f):
    """Map free-variable name -> value for a Python closure."""
    return dict(zip(f.__code__.co_freevars, (c.cell_contents for c in f.__closure__)))


def indent(text, n):
    pad = " " * n
    return "\n".join(pad + line for line in text.split("\n"))


def f32_bits(value):
    """The int32 bit pattern of ``value`` rounded to float32.

    Kernel work lists are int32 tables; float scalars (alpha, tau, ...) ride in
    them as raw bits and are re-read on the device with ``__int_as_float``.
    """
    return int(np.asarray(value, dtype=np.float32).view(np.int32))


def as_ascii(text):
    """``text`` as a str: bytes are decoded as ASCII, other objects go through ``str``."""
    if isinstance(text, bytes):
        return text.decode("ascii")
    return text if isinstance(text, str) else str(text)


def equal_strides(strides_a, strides_b, shape):
    """Whether two stride tuples address an array of ``shape`` the same way: axes of
    length one may differ, all others must agree, and the ranks must match."""
    if not (len(strides_a) == len(strides_b) == len(shape)):
        return False
    return all(n == 1 or a == b for n, a, b in zip(shape, strides_a, strides_b))


def nonelist(*args):
    """The arguments that are not None, in order."""
    return [a for a in args if a is not None]


def round_up_power_of_2(x):
    """The power of two at or above ``|x|`` with the sign of ``x`` (1 for ``|x| < 1``)."""
    if abs(x) < 1:
        return 1
    magnitude = 2 ** int(np.ceil(np.log2(abs(x))))
    return magnitude if x > 0 else -magnitude


def __getattr__(name):
    # (imported on demand: the sparse module imports this one)
    if name == "HostSparseMatrix":
        from .hipra_spmv import HostSparseMatrix

        return HostSparseMatrix
    raise AttributeError(name)
