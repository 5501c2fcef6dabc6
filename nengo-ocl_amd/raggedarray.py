"""Host ragged array: many small 2-D arrays inside one flat buffer.

This layout *is* the kernel ABI of the timestep path: every kernel receives
one flat float32 (or int32) buffer plus int32 element offsets / shapes /
strides, so it is kept field-for-field compatible with the reference's
``nengo_ocl/raggedarray.py`` (class ``RaggedArray`` :31-236): ``buf``,
``starts``, ``shape0s``, ``shape1s``, ``stride0s``, ``stride1s``, ``names``;
items may alias each other (views added with ``add_views``).

Differences from the reference, all deliberate:

* ``align=True`` pads every item start to a multiple of ``align_elems``
  (default 16 floats = 64 B) so that rows of matrices whose row stride is a
  multiple of 4 can be read with 16-byte vector loads on the GPU; items of 1024
  elements or more start on a multiple of 64 elements (256 B), and matrices of
  65536 elements or more are skewed against each other inside 16 KiB windows (HBM
  channel spreading, see ``SKEW_ITEM_ELEMS``).  The
  reference's policy (16 for size >= 16, 4 for size >= 8, raggedarray.py:46-55)
  is available as ``align="reference"``.
* the five metadata vectors live in one ``(5, n)`` int32 table, exposed through
  read-only properties with the reference's names.
"""

from io import StringIO

import numpy as np

from .utils import is_iterable, round_up

# items this large start on a 256-byte boundary, so that a wave's 1 KiB load
# instruction covers whole 128-byte memory lines of the matrix
BIG_ITEM_ELEMS = 1024
BIG_ITEM_ALIGN = 64
# Matrices of this size or more are additionally skewed against each other: the
# k-th one starts (9 k mod 64) * 256 bytes past a 16 KiB boundary.  Many waves
# stream rows of many such matrices at the same column offset at the same time; when
# all rows are congruent modulo the memory channel interleave (row strides of 4 KiB
# multiples, bases 512 B or 4 KiB apart) the traffic piles up on a few HBM channels.
# Measured on MI355X, 256 matrices of 64 x 4096: 78 us per pass with bases 1 MiB +
# 4 KiB apart, 66 us at + 512 B, 51 us with this skew.
SKEW_ITEM_ELEMS = 65536
SKEW_WINDOW = 4096     # elements: 16 KiB
SKEW_STEP = 9 * 64     # elements: 2304 bytes

_FIELDS = ("starts", "shape0s", "shape1s", "stride0s", "stride1s")


def allclose(a, b, atol=1e-3, rtol=1e-3):
    """Same layout and numerically close buffers (raggedarray.py:16-29)."""
    for f in _FIELDS:
        if not np.array_equal(getattr(a, f), getattr(b, f)):
            return False
    return bool(np.allclose(a.buf, b.buf, atol=atol, rtol=rtol))


def _as_int32_row(values):
    """Offsets, shapes and strides are int32 element counts, as in the reference
    (raggedarray.py:107-111): a buffer of 2^31 elements or more cannot be described."""
    wide = np.asarray(values, dtype=np.int64).reshape(-1)
    if wide.size and (wide.max() > np.iinfo(np.int32).max or wide.min() < np.iinfo(np.int32).min):
        raise ValueError("a ragged array is limited to 2^31 - 1 elements (int32 offsets); "
                         "got an offset, shape or stride of %d" % int(np.abs(wide).max()))
    row = wide.astype(np.int32)
    row.setflags(write=False)
    return row


class RaggedArray:
    """A linear buffer partitioned into (possibly overlapping) 2-D sections."""

    def __init__(self, arrays, names=None, dtype=None, align=False, align_elems=16):
        arrays = [np.asarray(a) for a in arrays]
        if len(arrays) == 0:
            raise ValueError("RaggedArray needs at least one item")
        if any(a.ndim > 2 for a in arrays):
            raise ValueError("RaggedArray items are at most 2-D")

        dtype = np.dtype(arrays[0].dtype if dtype is None else dtype)
        if dtype not in (np.dtype(np.float32), np.dtype(np.int32)):
            raise TypeError("RaggedArray holds float32 or int32, got %s" % dtype)

        sizes = [a.size for a in arrays]
        starts = []
        cursor = 0
        n_skewed = 0
        for size in sizes:
            if align == "reference":
                unit = 16 if size >= 16 else 4 if size >= 8 else 1
            elif align:
                unit = BIG_ITEM_ALIGN if size >= BIG_ITEM_ELEMS else align_elems if size >= 4 else 1
            else:
                unit = 1
            if align is True and size >= SKEW_ITEM_ELEMS:
                cursor = round_up(cursor, SKEW_WINDOW) + (n_skewed * SKEW_STEP) % SKEW_WINDOW
                n_skewed += 1
            cursor = round_up(cursor, unit)
            starts.append(cursor)
            cursor += size
        if cursor > np.iinfo(np.int32).max:
            raise ValueError("a ragged array is limited to 2^31 - 1 elements (int32 offsets); "
                             "these items need %d" % cursor)

        self._set_meta(
            starts,
            [a.shape[0] if a.ndim > 0 else 1 for a in arrays],
            [a.shape[1] if a.ndim > 1 else 1 for a in arrays],
            [a.shape[1] if a.ndim == 2 else 1 for a in arrays],
            [1] * len(arrays),
        )

        buf = np.zeros(cursor, dtype=dtype)
        for a, s in zip(arrays, starts):
            buf[s : s + a.size] = a.ravel()
        self.buf = buf
        self.names = names

    # ------------------------------------------------------------------ meta
    def _set_meta(self, starts, shape0s, shape1s, stride0s, stride1s):
        rows = [_as_int32_row(v) for v in (starts, shape0s, shape1s, stride0s, stride1s)]
        n = rows[0].size
        if any(r.size != n for r in rows):
            raise ValueError("ragged metadata vectors differ in length")
        if np.any(rows[0] < 0) or np.any(rows[1] < 0) or np.any(rows[2] <= 0):
            raise ValueError("negative start/shape0 or non-positive shape1")
        if np.any(rows[3] == 0) or np.any(rows[4] == 0):
            raise ValueError("zero stride")
        self._meta = rows
        self._sizes = None

    @classmethod
    def from_buffer(cls, buf, starts, shape0s, shape1s, stride0s, stride1s, names=None):
        """Wrap an existing buffer without copying (raggedarray.py:74-84)."""
        self = cls.__new__(cls)
        self._set_meta(starts, shape0s, shape1s, stride0s, stride1s)
        self.buf = buf
        self.names = names
        return self

    starts = property(lambda self: self._meta[0])
    shape0s = property(lambda self: self._meta[1])
    shape1s = property(lambda self: self._meta[2])
    stride0s = property(lambda self: self._meta[3])
    stride1s = property(lambda self: self._meta[4])

    @property
    def sizes(self):
        if self._sizes is None:
            self._sizes = self.shape0s * self.shape1s
        return self._sizes

    @property
    def dtype(self):
        return self._buf.dtype

    @property
    def ctype(self):
        return "float" if self.dtype == np.float32 else "int"

    @property
    def nbytes(self):
        return int(self.sizes.sum()) * self.dtype.itemsize

    @property
    def buf(self):
        return self._buf

    @buf.setter
    def buf(self, buf):
        buf = np.asarray(buf)
        if buf.dtype not in (np.dtype(np.float32), np.dtype(np.int32)):
            raise TypeError("RaggedArray buffer must be float32 or int32")
        self._buf = buf

    @property
    def names(self):
        return self._names

    @names.setter
    def names(self, names):
        n = len(self)
        self._names = tuple([""] * n if names is None else names)
        if len(self._names) != n:
            raise ValueError("need one name per item")

    # ------------------------------------------------------------ containers
    def __len__(self):
        return int(self._meta[0].size)

    def _select(self, idx):
        return [[int(row[i]) for i in idx] for row in self._meta]

    def __getitem__(self, item):
        """One index -> strided ndarray view; several -> sub-RaggedArray (no copy)."""
        if isinstance(item, slice):
            item = range(len(self))[item]
        if is_iterable(item):
            idx = [int(i) for i in item]
            return type(self).from_buffer(
                self.buf, *self._select(idx), names=[self.names[i] for i in idx]
            )

        i = int(np.asarray(item).reshape(()))
        isz = self.dtype.itemsize
        return np.ndarray(
            shape=(int(self.shape0s[i]), int(self.shape1s[i])),
            dtype=self.dtype,
            buffer=self.buf.data,
            offset=isz * int(self.starts[i]),
            strides=(isz * int(self.stride0s[i]), isz * int(self.stride1s[i])),
        )

    def __setitem__(self, item, value):
        try:
            item = int(item)
        except TypeError as e:
            raise NotImplementedError("`item` must be castable to int") from e
        self[item][...] = value

    def __iter__(self):
        return (self[i] for i in range(len(self)))

    def add_views(self, starts, shape0s, shape1s, stride0s, stride1s, names=None):
        """Append items that alias existing memory (raggedarray.py:224-236)."""
        starts = [int(s) for s in starts]
        for s, m, n in zip(starts, shape0s, shape1s):
            if s + int(m) * int(n) > self.buf.size:
                raise ValueError("view runs past the end of the buffer")
        old_names = self.names
        merged = [
            list(old) + [int(v) for v in new]
            for old, new in zip(
                self._meta, (starts, shape0s, shape1s, stride0s, stride1s)
            )
        ]
        self._set_meta(*merged)
        self._names = old_names + tuple(names if names else [""] * len(starts))

    def __str__(self):
        sio = StringIO()
        width = max(len(n) for n in self.names)
        for i, name in enumerate(self.names):
            print(name.rjust(width), self[i], file=sio)
        return sio.getvalue()
