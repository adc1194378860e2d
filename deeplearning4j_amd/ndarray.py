"""Host-side array handle: the stand-in for INDArray + OpaqueNDArray + OpaqueDataBuffer on the Java side.

An `NDArray` owns (or shares) a native data buffer (host + device storage with coherence stamps), a
shapeInfo descriptor buffer and the native array handle built from them with `createOpaqueNDArray`
(nd4j-api `org.nd4j.nativeblas.OpaqueNDArray.fromINDArray`, OpaqueNDArray.java:78-107).
Views (permute / reshape / slices) share the data buffer and carry their own descriptor and offset.
"""
import ctypes

import numpy as np

from . import nativeops as N

BOOL, HALF, FLOAT32, DOUBLE, INT32, INT64, BFLOAT16 = 1, 3, 5, 6, 9, 10, 17
INT8, INT16, UINT8, UINT16, UINT32, UINT64 = 7, 8, 11, 12, 13, 14          # array/DataType.h:27-50
DT_SIZE = {BOOL: 1, HALF: 2, FLOAT32: 4, DOUBLE: 8, INT32: 4, INT64: 8, BFLOAT16: 2, INT8: 1, INT16: 2, UINT8: 1, UINT16: 2, UINT32: 4, UINT64: 8}
_UNSIGNED = 8388608                                                            # array/ArrayOptions.h: ARRAY_UNSIGNED
DT_FLAG = {HALF: 4096, BFLOAT16: 2048, FLOAT32: 8192, DOUBLE: 16384, INT32: 131072, INT64: 262144, BOOL: 524288, INT8: 32768, INT16: 65536,
           UINT8: 32768 | _UNSIGNED, UINT16: 65536 | _UNSIGNED, UINT32: 131072 | _UNSIGNED, UINT64: 262144 | _UNSIGNED}
DT_NP = {BOOL: np.bool_, HALF: np.float16, FLOAT32: np.float32, DOUBLE: np.float64, INT32: np.int32, INT64: np.int64,
         BFLOAT16: np.uint16, INT8: np.int8, INT16: np.int16, UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32, UINT64: np.uint64}
# (a numpy uint16 array is taken as bf16 bit patterns only when BFLOAT16 is asked for; by itself it is UINT16)
NP_DT = {np.dtype(np.bool_): BOOL, np.dtype(np.float16): HALF, np.dtype(np.float32): FLOAT32,
         np.dtype(np.float64): DOUBLE, np.dtype(np.int32): INT32, np.dtype(np.int64): INT64, np.dtype(np.int8): INT8,
         np.dtype(np.int16): INT16, np.dtype(np.uint8): UINT8, np.dtype(np.uint16): UINT16, np.dtype(np.uint32): UINT32,
         np.dtype(np.uint64): UINT64}


def dtype_of_extra(extra):
    """The data type a shape descriptor's extra word names (array/ArrayOptions.hXX, dataType(): the sign bit picks the
    unsigned twin of an integer type)."""
    type_bits = 0
    for v in DT_FLAG.values():
        type_bits |= v
    for k, v in DT_FLAG.items():
        if extra & type_bits == v:
            return k
    raise ValueError("shape descriptor names no data type: extra = %d" % extra)


def f32_to_bf16_bits(a):
    """float32 -> bf16 bit patterns, round-to-nearest-even, NaN -> 0x7FC0."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[np.isnan(a)] = 0x7FC0
    return r.reshape(a.shape)


def bf16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    return (h.astype(np.uint32) << 16).view(np.float32).reshape(h.shape)


def dense_strides(shape, order="c"):
    st = [0] * len(shape)
    s = 1
    rng = range(len(shape) - 1, -1, -1) if order == "c" else range(len(shape))
    for i in rng:
        st[i] = s
        s *= max(int(shape[i]), 1)
    return st


def make_shape_info(shape, strides, dtype, order="c", empty=False):
    """Reference descriptor int64[2*rank+4] (libnd4j/include/helpers/shape.h:76-104)."""
    r = len(shape)
    flags = DT_FLAG[dtype] | (8 if empty else 0)
    if r == 0:
        return np.array([0, 0, 1, flags, 1, ord(order)], dtype=np.int64)
    ews = 1 if list(strides) == dense_strides(shape, order) else 0
    return np.array([r, *shape, *strides, flags, ews, ord(order)], dtype=np.int64)


class DataBuffer:
    """Owner of a native OpaqueDataBuffer."""

    def __init__(self, n_elements, dtype, allocate_both=True):
        L = N.load()
        self.dtype = dtype
        self.n = int(n_elements)
        self.ptr = L.dbAllocateDataBuffer(self.n, dtype, allocate_both)
        N.check("dbAllocateDataBuffer")
        if not self.ptr:
            raise N.NativeOpsError("dbAllocateDataBuffer returned null")

    def host_view(self):
        """numpy view of the host (primary) storage; does not synchronise."""
        L = N.load()
        p = L.dbPrimaryBuffer(self.ptr)
        n = max(self.n, 1)
        buf = (ctypes.c_char * (n * DT_SIZE[self.dtype])).from_address(p)
        return np.frombuffer(buf, dtype=DT_NP[self.dtype], count=n)

    def __del__(self):
        try:
            if getattr(self, "ptr", None):
                N.load().deleteDataBuffer(self.ptr)
                self.ptr = None
        except Exception:
            pass


class NDArray:
    def __init__(self, buffer, shape, strides=None, dtype=None, offset=0, order="c"):
        L = N.load()
        self.buffer = buffer
        self.dtype = dtype if dtype is not None else buffer.dtype
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(int(s) for s in (strides if strides is not None else dense_strides(self.shape, order)))
        self.offset = int(offset)
        self.order = order
        empty = any(s == 0 for s in self.shape)
        self.shape_info = make_shape_info(self.shape, self.strides, self.dtype, order, empty)
        # the descriptor travels in a small INT64 data buffer, as on the Java side
        self._si_buf = DataBuffer(len(self.shape_info), INT64, allocate_both=False)
        self._si_buf.host_view()[: len(self.shape_info)] = self.shape_info
        self.handle = L.createOpaqueNDArray(self._si_buf.ptr, None if empty else buffer.ptr, None if empty else buffer.ptr,
                                            self.offset)
        N.check("createOpaqueNDArray")

    # ---- construction ----
    @staticmethod
    def from_numpy(a, dtype=None, order="c"):
        """Dense copy of `a` into a fresh buffer.  dtype=BFLOAT16 rounds float input to bf16 (RNE)."""
        a = np.asarray(a)
        if dtype == BFLOAT16 and a.dtype != np.uint16:
            a = f32_to_bf16_bits(a.astype(np.float32))
        dt = dtype if dtype is not None else NP_DT[a.dtype]
        a = a.astype(DT_NP[dt], copy=False)
        buf = DataBuffer(max(a.size, 1), dt)
        arr = NDArray(buf, a.shape, None, dt, 0, order)
        if a.size:
            flat = np.asfortranarray(a).ravel(order="F") if order == "f" else np.ascontiguousarray(a).ravel()
            buf.host_view()[: a.size] = flat
        N.load().dbTickHostWrite(buf.ptr)
        return arr

    @staticmethod
    def empty(shape, dtype, order="c"):
        n = int(np.prod(shape)) if len(shape) else 1
        buf = DataBuffer(max(n, 1), dtype)
        return NDArray(buf, shape, None, dtype, 0, order)

    @staticmethod
    def scalar(value, dtype):
        return NDArray.from_numpy(np.array(value, dtype=DT_NP[dtype] if dtype != BFLOAT16 else np.float32), dtype)

    # ---- views ----
    def view(self, shape, strides, offset=None):
        return NDArray(self.buffer, shape, strides, self.dtype, self.offset if offset is None else offset, self.order)

    def permute(self, *axes):
        return self.view([self.shape[a] for a in axes], [self.strides[a] for a in axes])

    def reshape(self, *shape):
        assert list(self.strides) == dense_strides(self.shape, "c"), "reshape needs a dense c-order array"
        shape = list(shape)
        if -1 in shape:
            known = int(np.prod([s for s in shape if s != -1]))
            shape[shape.index(-1)] = self.length() // known
        return self.view(shape, dense_strides(shape, "c"))

    def slice(self, dim, start, stop):
        shape = list(self.shape)
        shape[dim] = stop - start
        return self.view(shape, self.strides, self.offset + start * self.strides[dim])

    def length(self):
        return int(np.prod(self.shape)) if len(self.shape) else 1

    # ---- data movement ----
    def sync_to_device(self):
        N.load().dbSyncToSpecial(self.buffer.ptr)
        N.check("dbSyncToSpecial")

    def to_numpy(self):
        """Synchronise device -> host and return a copy of the view (bf16 comes back as uint16 bit patterns)."""
        L = N.load()
        L.dbSyncToPrimary(self.buffer.ptr)
        N.check("dbSyncToPrimary")
        L.dbTickHostRead(self.buffer.ptr)
        host = self.buffer.host_view()
        if len(self.shape) == 0:
            return host[self.offset].copy()
        if self.length() == 0:
            return np.zeros(self.shape, dtype=DT_NP[self.dtype])
        item = host.itemsize
        v = np.lib.stride_tricks.as_strided(host[self.offset:], shape=self.shape, strides=[s * item for s in self.strides])
        return np.array(v)

    def to_float(self):
        a = self.to_numpy()
        if self.dtype == BFLOAT16:
            return bf16_bits_to_f32(a)
        return a.astype(np.float32) if self.dtype == HALF else a

    def assign_numpy(self, a):
        """Overwrite the view's elements on the host and mark the host side as written."""
        L = N.load()
        L.dbSyncToPrimary(self.buffer.ptr)
        host = self.buffer.host_view()
        a = np.asarray(a)
        if self.dtype == BFLOAT16 and a.dtype != np.uint16:
            a = f32_to_bf16_bits(a.astype(np.float32))
        item = host.itemsize
        v = np.lib.stride_tricks.as_strided(host[self.offset:], shape=self.shape, strides=[s * item for s in self.strides])
        v[...] = a.astype(host.dtype, copy=False).reshape(self.shape)
        L.dbTickHostWrite(self.buffer.ptr)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                N.load().deleteNDArray(self.handle)
                self.handle = None
        except Exception:
            pass
