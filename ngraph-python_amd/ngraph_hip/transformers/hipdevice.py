"""Device memory of the `hipgpu` transformer: one allocation per base tensor, views as pointer +
element strides, host reads and writes (gputransform.py:525-909: GPUDeviceBufferStorage,
GPUDeviceTensor).  Strided views go through the device copy kernel and one context-owned scratch
buffer; large copies through the context's pinned staging buffers.
"""
from __future__ import division

import numpy as np

from ngraph_hip.transformers.base import DeviceBufferStorage, DeviceTensor


def _td(op):
    """The tensor description of `op` in this backend's conventions: strides and offset in
    elements, one stride per axis.  The graph front of this repository describes tensors that
    way itself (`_adapt_td` is the identity); the plug-in for the real package, whose
    descriptions hold byte strides and nested strides for flattened axes
    (ngraph/op_graph/axes.py:1174-1232), replaces `_adapt_td`."""
    return _adapt_td(op.tensor_description())


def _adapt_td(td):
    return td


class HipDeviceBufferStorage(DeviceBufferStorage):
    """One device allocation per base tensor (gputransform.py:642-676); allocated on first use."""

    def __init__(self, transformer, bytes, dtype, **kwargs):
        super(HipDeviceBufferStorage, self).__init__(transformer, bytes, dtype, **kwargs)
        self._ptr = None

    @property
    def ptr(self):
        if self._ptr is None:
            self._ptr = self.transformer.runtime.malloc(max(int(self.bytes), 4))
        return self._ptr

    def create_device_tensor(self, tensor_description):
        return HipDeviceTensor(self.transformer, self, tensor_description,
                               name="v_" + tensor_description.name)

    def free(self):
        if self._ptr is not None:
            self.transformer.runtime.free(self._ptr)
            self._ptr = None


class HipDeviceTensor(DeviceTensor):
    """A strided view of a device buffer with host I/O (gputransform.py:679-909)."""

    storage_np_dtype = None   # None: the logical dtype

    def transform_allocate(self):
        pass

    @property
    def view(self):
        """The view's description with strides and offset in elements (see _td)."""
        return _adapt_td(self.tensor_description)

    @property
    def np_dtype(self):
        d = self.tensor_description.dtype
        return d if isinstance(d, np.dtype) else np.dtype(np.int16)

    @property
    def ngh_dtype(self):
        return self.transformer.ngh_dtype(self.tensor_description.dtype)

    @property
    def itemsize(self):
        return self.np_dtype.itemsize

    @property
    def ptr(self):
        return self.device_buffer.ptr + self.view.offset * self.itemsize

    @property
    def shape(self):
        return self.view.shape

    @property
    def element_strides(self):
        return self.view.full_strides

    def _read_raw(self):
        """The view's elements as a C-contiguous host array of the storage dtype."""
        td, rt = self.view, self.transformer.runtime
        out = np.empty(td.shape, dtype=self.np_dtype)
        if out.size == 0:
            return out
        if td.c_contiguous:
            rt.memcpy_d2h(out, self.ptr)
            return out
        # strided or broadcast view: gather on the device (into the context's scratch), then one
        # contiguous copy out
        tmp = rt.io_scratch(out.nbytes)
        contiguous = [int(s) // out.itemsize for s in out.strides]
        rt.copy_strided(tmp, self.ptr, td.shape, contiguous, td.full_strides, out.itemsize)
        rt.memcpy_d2h(out, tmp)
        return out

    def _write_window(self, host, offset, shape, strides):
        """host (broadcast to `shape`) into the window of the buffer that starts `offset` elements
        into this view and has the given element strides."""
        rt = self.transformer.runtime
        host = np.ascontiguousarray(np.broadcast_to(host, shape), dtype=self.np_dtype)
        if host.size == 0:
            return
        ptr = self.ptr + offset * self.itemsize
        dense, run = True, 1
        for n, s in zip(reversed(shape), reversed(strides)):
            dense = dense and (n == 1 or s == run)
            run *= n
        if dense:
            rt.memcpy_h2d(ptr, host)
            return
        if any(s == 0 and n > 1 for s, n in zip(strides, shape)):
            raise ValueError("cannot write through a broadcast view")
        # one contiguous copy in (the host copy returns when the data has arrived), then a
        # scatter on the device, which later kernels on the stream are ordered behind
        tmp = rt.io_scratch(host.nbytes)
        rt.memcpy_h2d(tmp, host)
        contiguous = [int(s) // host.itemsize for s in host.strides]
        rt.copy_strided(ptr, tmp, shape, strides, contiguous, host.itemsize)

    def _write_raw(self, host):
        td = self.view
        self._write_window(host, 0, td.shape, td.full_strides)

    def get(self, tensor):
        value = self._read_raw()
        if tensor is None:
            return value
        tensor[...] = value
        return tensor

    def __getitem__(self, key):
        return self.get(None)[key]

    def _window_of(self, key):
        """(offset, shape, strides) in elements of view[key] for a key made of integers and
        slices (what NumPy calls basic indexing); None for anything else."""
        td = self.view
        key = key if isinstance(key, tuple) else (key,)
        if any(k is Ellipsis for k in key):
            i = [k is Ellipsis for k in key].index(True)
            if any(k is Ellipsis for k in key[i + 1:]):
                return None
            key = key[:i] + (slice(None),) * (len(td.shape) - (len(key) - 1)) + key[i + 1:]
        if len(key) > len(td.shape):
            return None
        key = key + (slice(None),) * (len(td.shape) - len(key))
        offset, shape, strides = 0, [], []
        for k, n, s in zip(key, td.shape, td.full_strides):
            if isinstance(k, (int, np.integer)):
                k = int(k)
                if not -n <= k < n:
                    raise IndexError("index %d is out of bounds for an axis of length %d" % (k, n))
                offset += (k % n) * s
            elif isinstance(k, slice):
                lo, hi, step = k.indices(n)
                count = len(range(lo, hi, step))
                offset += lo * s if count else 0
                shape.append(count)
                strides.append(s * step)
            else:
                return None
        return offset, shape, strides

    def __setitem__(self, key, value):
        value = np.asarray(value)
        if key is Ellipsis or key == () or (isinstance(key, slice) and key == slice(None, None, None)):
            self._write_raw(value.astype(self.np_dtype, copy=False))
            return
        window = self._window_of(key)
        if window is not None and all(s >= 0 for s in window[2]):
            # only the addressed window travels: a contiguous copy in and a strided copy on the device
            self._write_window(value.astype(self.np_dtype, copy=False), *window)
            return
        whole = self._read_raw()
        whole[key] = value
        self._write_raw(whole)
