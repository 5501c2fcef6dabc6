"""Device side of the ragged signal layout: one flat HBM buffer + int32 metadata.

Counterpart of the reference's ``nengo_ocl/clraggedarray.py`` (``CLRaggedArray``
:65-311, ``to_host`` :36-62) over HIP device memory.  Device memory and the
stream come from PyTorch-ROCm (``torch.empty(..., device="cuda")``,
``torch.cuda.Stream``); kernels never see torch types, only raw pointers.

``Queue`` stands where the reference passes a ``pyopencl.CommandQueue``: every
``plan_*`` function takes one as its first argument.
"""

import ctypes
from io import StringIO

import numpy as np

from . import _lib
from .raggedarray import RaggedArray
from .utils import is_iterable

_TORCH = None


def _torch():
    global _TORCH
    if _TORCH is None:
        import torch

        if not torch.cuda.is_available():
            raise RuntimeError(
                "no HIP device visible: the MI355X backend has no CPU fallback"
            )
        _TORCH = torch
    return _TORCH


class Queue:
    """An in-order HIP stream on one device (default priority)."""

    def __init__(self, device=0):
        torch = _torch()
        self.device = torch.device("cuda", device)
        self.stream = torch.cuda.Stream(device=self.device)
        self.handle = ctypes.c_void_p(self.stream.cuda_stream)
        self.lib = _lib.lib()
        n_cu, wave, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        name = ctypes.create_string_buffer(64)
        with torch.cuda.device(self.device):
            _lib.check(self.lib.nhip_device_info(ctypes.byref(n_cu), ctypes.byref(wave),
                                                 ctypes.byref(lds), name, 64), "device info")
        self.n_compute_units = max(1, n_cu.value)
        self.arch = name.value.decode()
        self.global_mem_size = int(torch.cuda.get_device_properties(self.device).total_memory)

    def finish(self):
        _lib.check(self.lib.nhip_stream_sync(self.handle), "stream sync")

    def context(self):
        """Context manager making this stream torch's current stream."""
        return _torch().cuda.stream(self.stream)


class DeviceArray:
    """A flat device array (float32 or int32) with the few methods plans need."""

    def __init__(self, queue, tensor, dtype):
        self.queue = queue
        self.tensor = tensor
        self.dtype = np.dtype(dtype)
        addr = tensor.data_ptr()
        self.ptr = ctypes.c_void_p(addr if addr else None)

    @property
    def shape(self):
        return tuple(self.tensor.shape)

    @property
    def size(self):
        return int(self.tensor.numel())

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def ctype(self):
        return "float" if self.dtype == np.float32 else "int"

    @property
    def data(self):
        return self.ptr

    def get(self):
        with self.queue.context():
            return self.tensor.cpu().numpy()

    def get_span(self, start, length):
        with self.queue.context():
            return self.tensor.view(-1)[start : start + length].cpu().numpy()

    def set(self, array, start=0):
        torch = _torch()
        array = np.ascontiguousarray(array, dtype=self.dtype).reshape(-1)
        with self.queue.context():
            self.tensor.view(-1)[start : start + array.size].copy_(torch.from_numpy(array))
            self.queue.stream.synchronize()  # the pageable source may go away

    def fill(self, value):
        with self.queue.context():
            self.tensor.fill_(value)


def to_device(queue, array, dtype=None):
    """Upload a host array; returns a `DeviceArray` of the same shape."""
    torch = _torch()
    array = np.ascontiguousarray(array, dtype=dtype)
    if not array.flags.writeable:  # read-only views (metadata rows): torch wants its own copy
        array = array.copy()
    if array.dtype not in (np.dtype(np.float32), np.dtype(np.int32)):
        raise TypeError("device arrays are float32 or int32, got %s" % array.dtype)
    with queue.context():
        t = torch.empty(array.shape, dtype=getattr(torch, array.dtype.name), device=queue.device)
        if array.size:
            t.copy_(torch.from_numpy(array))
        queue.stream.synchronize()
    return DeviceArray(queue, t, array.dtype)


class HIPRaggedArray:
    """A linear device buffer partitioned into (possibly aliasing) 2-D sections."""

    def __init__(self, queue, np_raggedarray):
        self.queue = queue
        self._set_meta(np_raggedarray)
        self.dev_buf = to_device(queue, np_raggedarray.buf)
        self.names = np_raggedarray.names

    def _set_meta(self, src):
        self.starts = src.starts
        self.shape0s = src.shape0s
        self.shape1s = src.shape1s
        self.stride0s = src.stride0s
        self.stride1s = src.stride1s
        self._dev_meta = {}

    @classmethod
    def from_arrays(cls, queue, arrays, names=None, dtype=None, align=False):
        return cls(queue, RaggedArray(arrays, names=names, dtype=dtype, align=align))

    @classmethod
    def from_buffer(cls, queue, dev_buf, starts, shape0s, shape1s, stride0s, stride1s, names=None):
        """A view onto an existing device buffer (no allocation, no copy)."""
        host_view = RaggedArray.from_buffer(
            np.zeros(0, dtype=dev_buf.dtype), starts, shape0s, shape1s, stride0s, stride1s
        )
        self = cls.__new__(cls)
        self.queue = queue
        self._set_meta(host_view)
        self.dev_buf = dev_buf
        self.names = names
        return self

    # -- the five int32 metadata vectors also exist on the device, uploaded on
    #    first use (clraggedarray.py:123-184 uploads them eagerly)
    def _dev(self, field):
        if field not in self._dev_meta:
            self._dev_meta[field] = to_device(self.queue, getattr(self, field))
        return self._dev_meta[field]

    dev_starts = property(lambda self: self._dev("starts"))
    dev_shape0s = property(lambda self: self._dev("shape0s"))
    dev_shape1s = property(lambda self: self._dev("shape1s"))
    dev_stride0s = property(lambda self: self._dev("stride0s"))
    dev_stride1s = property(lambda self: self._dev("stride1s"))
    # names the reference's call sites use
    cl_buf = property(lambda self: self.dev_buf)
    cl_starts = dev_starts
    cl_shape0s = dev_shape0s
    cl_shape1s = dev_shape1s
    cl_stride0s = dev_stride0s
    cl_stride1s = dev_stride1s

    @property
    def ctype(self):
        return self.dev_buf.ctype

    @property
    def dtype(self):
        return self.dev_buf.dtype

    @property
    def ptr(self):
        return self.dev_buf.ptr

    @property
    def names(self):
        return self._names

    @names.setter
    def names(self, names):
        self._names = tuple([""] * len(self.starts) if names is None else names)

    @property
    def sizes(self):
        return self.shape0s * self.shape1s

    @property
    def nbytes(self):
        return int(self.sizes.sum()) * self.dtype.itemsize

    @property
    def buf(self):
        buf = self.dev_buf.get().reshape(-1)
        buf.setflags(write=False)
        return buf

    def __len__(self):
        return int(self.starts.size)

    def check_bounds(self, what="ragged array"):
        """Raise if any item reaches outside the device buffer.

        Kernels trust the int32 offsets they are given; every plan builder calls
        this on its operands so that a bad view fails on the host, at plan time,
        instead of as a memory fault on the device."""
        if len(self) == 0:
            return
        m = self.shape0s.astype(np.int64)
        n = self.shape1s.astype(np.int64)
        last = (self.starts.astype(np.int64) + np.maximum(m - 1, 0) * self.stride0s
                + np.maximum(n - 1, 0) * self.stride1s)
        used = (m * n) > 0
        if np.any(self.starts < 0) or np.any(self.stride0s < 0) or np.any(self.stride1s < 0):
            raise ValueError("%s: negative start or stride" % what)
        if used.any() and int(last[used].max()) >= self.dev_buf.size:
            bad = int(np.nonzero(used & (last >= self.dev_buf.size))[0][0])
            raise ValueError("%s: item %d (start %d, shape %dx%d, strides %d,%d) runs past the "
                             "end of its %d-element buffer" % (
                                 what, bad, self.starts[bad], m[bad], n[bad], self.stride0s[bad],
                                 self.stride1s[bad], self.dev_buf.size))

    # ------------------------------------------------------------- host access
    def _span(self, i):
        m, n = int(self.shape0s[i]), int(self.shape1s[i])
        sm, sn = int(self.stride0s[i]), int(self.stride1s[i])
        if min(sm, sn) < 0:
            raise NotImplementedError("negative strides")
        return m, n, sm, sn, (m - 1) * sm + (n - 1) * sn + 1

    def _read_item(self, i):
        """Copy the smallest contiguous span holding item ``i``; view it strided."""
        m, n, sm, sn, length = self._span(i)
        if m * n == 0:
            return np.zeros((m, n), dtype=self.dtype)
        span = self.dev_buf.get_span(int(self.starts[i]), length)
        isz = self.dtype.itemsize
        return np.lib.stride_tricks.as_strided(span, shape=(m, n), strides=(sm * isz, sn * isz))

    def __getitem__(self, item):
        """One index -> host ndarray (read-only copy); several -> device sub-view."""
        if isinstance(item, slice) or is_iterable(item):
            return self.getitem_device(item)
        out = self._read_item(int(item))
        out.setflags(write=False)
        return out

    def getitem_device(self, item):
        if isinstance(item, slice):
            item = range(len(self))[item]
        idx = [int(i) for i in item]
        return HIPRaggedArray.from_buffer(
            self.queue,
            self.dev_buf,
            self.starts[idx],
            self.shape0s[idx],
            self.shape1s[idx],
            self.stride0s[idx],
            self.stride1s[idx],
            names=[self.names[i] for i in idx],
        )

    def __setitem__(self, item, new_value):
        if isinstance(item, slice) or is_iterable(item):
            raise NotImplementedError("setting several items at once")
        i = int(item)
        m, n, sm, sn, length = self._span(i)
        if m * n == 0:
            return
        start = int(self.starts[i])
        value = np.asarray(new_value)
        if value.size == m * n:
            value = value.reshape(m, n)
        row_major = (sn == 1 or n == 1) and (sm == n or m == 1)
        if row_major:
            block = np.empty((m, n), dtype=self.dtype)
            block[...] = value
            self.dev_buf.set(block.ravel(), start=start)
        else:
            # discontiguous: read the surrounding span, patch it, write it back
            span = self.dev_buf.get_span(start, length).copy()
            isz = self.dtype.itemsize
            view = np.lib.stride_tricks.as_strided(
                span, shape=(m, n), strides=(sm * isz, sn * isz))
            view[...] = value
            self.dev_buf.set(span, start=start)

    def to_host(self):
        """Download the whole object into a host `RaggedArray`."""
        return RaggedArray.from_buffer(
            np.array(self.buf),
            self.starts,
            self.shape0s,
            self.shape1s,
            self.stride0s,
            self.stride1s,
            names=self.names,
        )

    def __str__(self):
        sio = StringIO()
        width = max([0] + [len(n) for n in self.names])
        for i, name in enumerate(self.names):
            print(name.rjust(width), self[i], file=sio)
        return sio.getvalue()


def to_host(queue, data, dtype, start, shape, elemstrides, is_blocking=True):
    """One strided 2-D section of the device array `data` as a host array: the smallest
    contiguous span that holds it is copied and viewed with the element strides (the
    reference's helper of this name, clraggedarray.py:36-62; copies here always wait)."""
    m, n = (int(v) for v in shape)
    sm, sn = (int(v) for v in elemstrides)
    if min(sm, sn) < 0:
        raise NotImplementedError("negative strides")
    dtype = np.dtype(dtype)
    if m * n == 0:
        return np.zeros((m, n), dtype=dtype)
    span = data.get_span(int(start), (m - 1) * sm + (n - 1) * sn + 1)
    isz = dtype.itemsize
    return np.lib.stride_tricks.as_strided(span.view(dtype), shape=(m, n), strides=(sm * isz, sn * isz))


# The reference's name for this class, so that code written against it reads the same.
CLRaggedArray = HIPRaggedArray
