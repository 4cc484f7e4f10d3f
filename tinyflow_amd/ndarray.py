"""NDArray: the array container handed across the C-ABI.

Same public surface as the reference ``pycode/tinyflow/ndarray.py`` (DLContext,
DLArray, cpu()/gpu(), NDArray with shape/ctx/asnumpy/copyto/free_gpu, array(),
empty(), random initialisers).  As in the reference, ``array`` and ``empty``
return an ``int`` (the byte count that could not be allocated) instead of an
NDArray when the device is out of memory (reference ndarray.py:232-260).
"""
import ctypes

import numpy as np

from ._base import _LIB, check_call, c_array


class DLContext(ctypes.Structure):
    """{device_id, device_type}; device_type 1 = cpu, 2 = gpu."""
    _fields_ = [("device_id", ctypes.c_int), ("device_type", ctypes.c_int)]
    _NAMES = {1: "cpu", 2: "gpu"}

    def __init__(self, device_id=0, device_type=1):
        super().__init__()
        self.device_id = device_id
        self.device_type = device_type

    def __repr__(self):
        return "%s(%d)" % (self._NAMES.get(self.device_type, "?"), self.device_id)

    def __eq__(self, other):
        return (isinstance(other, DLContext) and self.device_id == other.device_id
                and self.device_type == other.device_type)

    def __hash__(self):
        return hash((self.device_id, self.device_type))


class DLArray(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("ctx", DLContext), ("ndim", ctypes.c_int),
                ("shape", ctypes.POINTER(ctypes.c_int64))]


DLArrayHandle = ctypes.POINTER(DLArray)


def cpu(dev_id=0):
    return DLContext(dev_id, 1)


def gpu(dev_id=0):
    return DLContext(dev_id, 2)


def is_gpu_ctx(ctx):
    return bool(ctx) and ctx.device_type == 2


class NDArray(object):
    """Owner of one DLArray allocated by the library."""
    __slots__ = ["handle", "is_freed", "_shape"]

    def __init__(self, handle):
        self.handle = handle
        self.is_freed = False
        self._shape = None

    def __del__(self):
        if self.is_freed:
            return
        self.is_freed = True
        try:
            _LIB.DLArrayFree(self.handle)
        except Exception:  # interpreter teardown
            pass

    def free_gpu(self):
        """Release the storage now (the swap path frees device copies eagerly)."""
        if self.is_freed:
            return
        self.is_freed = True
        check_call(_LIB.DLArrayFree(self.handle))

    @property
    def shape(self):
        if self._shape is None:
            c = self.handle.contents
            self._shape = tuple(c.shape[i] for i in range(c.ndim))
        return self._shape

    @property
    def ctx(self):
        return self.handle.contents.ctx

    def __setitem__(self, in_slice, value):
        if (not isinstance(in_slice, slice) or in_slice.start is not None
                or in_slice.stop is not None):
            raise ValueError("Array only support set from numpy array")
        if isinstance(value, NDArray):
            if value.handle is not self.handle:
                value.copyto(self, None)
        elif isinstance(value, (np.ndarray, np.generic)):
            self._sync_copyfrom(value)
        else:
            raise TypeError("type %s not supported" % str(type(value)))

    def _sync_copyfrom(self, source_array):
        """Synchronous host -> this array copy of an fp32-convertible array."""
        if not isinstance(source_array, np.ndarray):
            try:
                source_array = np.array(source_array, dtype=np.float32)
            except Exception:
                raise TypeError("array must be an array_like data, type %s is not supported"
                                % str(type(source_array)))
        source_array = np.ascontiguousarray(source_array, dtype=np.float32)
        if source_array.shape != self.shape:
            raise ValueError("array shape do not match the shape of NDArray")
        borrowed, keep = NDArray._numpyasarray(source_array)
        check_call(_LIB.DLArrayCopyFromTo(ctypes.byref(borrowed), self.handle, None))
        del keep

    @staticmethod
    def _numpyasarray(np_data):
        """Borrowed DLArray view (ctx cpu(0)) of a C-contiguous fp32 numpy array."""
        assert np_data.flags["C_CONTIGUOUS"] and np_data.dtype == np.float32
        arr = DLArray()
        shape = c_array(ctypes.c_int64, np_data.shape)
        arr.data = np_data.ctypes.data_as(ctypes.c_void_p)
        arr.shape = shape
        arr.ndim = np_data.ndim
        arr.ctx = cpu(0)
        return arr, shape

    def asnumpy(self):
        np_arr = np.empty(self.shape, dtype=np.float32)
        borrowed, keep = NDArray._numpyasarray(np_arr)
        check_call(_LIB.DLArrayCopyFromTo(self.handle, ctypes.byref(borrowed), None))
        del keep
        return np_arr

    def copyto(self, target, cudaStream=None):
        """Copy into ``target`` (an NDArray, or a DLContext to allocate on)."""
        if isinstance(target, DLContext):
            target = empty(self.shape, target)
            if isinstance(target, int):
                return target
        if not isinstance(target, NDArray):
            raise ValueError("Unsupported target type %s" % str(type(target)))
        check_call(_LIB.DLArrayCopyFromTo(self.handle, target.handle, cudaStream))
        return target

    def prepare_fresh(self):
        """Call right after allocating a device array that ``copy_into_fresh`` will fill
        later: the copy then waits for nothing enqueued after this call."""
        check_call(_LIB.DLArrayPrepareFresh(self.handle))
        return self

    def copy_into_fresh(self, target, cudaStream):
        """Host -> device copy into ``target``, a device array that was just allocated and
        has not been used yet: waits only for the previous life of its storage, not
        for everything enqueued (the prefetch of the swap path)."""
        check_call(_LIB.DLArrayCopyIntoFresh(self.handle, target.handle, cudaStream))
        return target


def empty(shape, ctx=cpu(0)):
    """Uninitialised array; returns the wanted byte count (int) when out of memory."""
    shape = tuple(int(s) for s in shape)
    c_shape = c_array(ctypes.c_int64, shape)
    handle = DLArrayHandle()
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLArrayAlloc(c_shape, ctypes.c_int(len(shape)), ctx, ctypes.byref(handle),
                                 ctypes.byref(wanted)))
    if wanted.value != 0 or not handle:
        return wanted.value if wanted.value != 0 else -1
    arr = NDArray(handle)
    arr._shape = shape
    return arr


def array(arr, ctx=cpu(0)):
    """Array on ``ctx`` initialised from ``arr`` (converted to fp32)."""
    if not isinstance(arr, np.ndarray):
        arr = np.array(arr)
    ret = empty(arr.shape, ctx)
    if isinstance(ret, int):
        return ret
    ret._sync_copyfrom(arr)
    return ret


def _from_numpy(values, ctx):
    return array(np.asarray(values), ctx)


def Normal(loc=0, scale=1, size=None, ctx=cpu(0)):
    return _from_numpy(np.random.normal(loc, scale, size), ctx)


def Uniform(low=0, high=1, size=None, ctx=cpu(0)):
    return _from_numpy(np.random.uniform(low, high, size), ctx)


def xavier_Normal(loc=0, size=None, ctx=cpu(0)):
    scale = np.sqrt(2.0 / (size[0] + size[1]))
    return _from_numpy(np.random.normal(loc, scale, size), ctx)


def xavier_Uniform(size=None, ctx=cpu(0)):
    a = np.sqrt(6.0 / (size[0] + size[1]))
    return _from_numpy(np.random.uniform(-a, a, size), ctx)
