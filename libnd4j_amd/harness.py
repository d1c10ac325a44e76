"""Host-side plumbing a caller of NativeOps needs: device buffers, shapeInfo buffers, TAD tables and the
``extraPointers`` array of the reference's CUDA calling convention.  This is what nd4j's Java executioner
does around every call; tests, ``bench.py`` and the smoke test use it to drive the library through its
C ABI.  Nothing here computes op results.
"""
import ctypes

import numpy as np

from .native import NativeOps

DTYPES = {"Float": np.float32, "Half": np.float16, "Double": np.float64}
SUFFIX_OF = {np.dtype(np.float32): "Float", np.dtype(np.float16): "Half", np.dtype(np.float64): "Double"}


def _is_vector(shape):
    r = len(shape)
    if r == 0:
        return False
    if r == 1:
        return True
    if r > 2:
        return False
    return shape[0] == 1 or shape[1] == 1


def compute_ews(shape, strides, f_order=False):
    """shape::computeElementWiseStride (reference: include/helpers/shape.h:1461-1608)."""
    rank = len(shape)
    if rank == 0:
        return 1
    if _is_vector(shape):
        return int(strides[rank - 1])
    dims = [(s, t) for s, t in zip(shape, strides) if s != 1]
    n = 1
    for s in shape:
        n *= s
    if n == 0:
        return -1
    if not dims:
        return int(strides[rank - 1])
    for k in range(len(dims) - 1):
        if f_order:
            if dims[k + 1][1] != dims[k][0] * dims[k][1]:
                return -1
        elif dims[k][1] != dims[k + 1][0] * dims[k + 1][1]:
            return -1
    if f_order:
        return int(dims[0][1] * n)
    return int(dims[-1][1])


def dense_strides(shape, order):
    """shape::calcStrides / calcStridesFortran (shape.h:1270-1400): vectors get all-ones strides."""
    rank = len(shape)
    if _is_vector(shape):
        return [1] * rank
    st = [0] * rank
    acc = 1
    rng = range(rank) if order == "f" else range(rank - 1, -1, -1)
    for i in rng:
        st[i] = acc
        acc *= shape[i]
    return st


def shape_info(shape, order="c", strides=None, ews=None, offset=0):
    """Builds a shapeInfo buffer [rank, shape, stride, offset, ews, order] as shape::shapeBuffer /
    shapeBufferFortran do (shape.h:1617-1710): EWS is computed in C mode, so a dense f-order matrix gets -1."""
    shape = [int(s) for s in shape]
    if strides is None:
        strides = dense_strides(shape, order)
    strides = [int(s) for s in strides]
    if ews is None:
        ews = compute_ews(shape, strides, False)
    rank = len(shape)
    return np.array([rank] + shape + strides + [offset, ews, ord(order)], dtype=np.int64)


def info_shape(info):
    r = int(info[0])
    return [int(v) for v in info[1:1 + r]]


def info_strides(info):
    r = int(info[0])
    return [int(v) for v in info[1 + r:1 + 2 * r]]


def info_numel(info):
    n = 1
    for s in info_shape(info):
        n *= s
    return n


def element_offsets(info):
    """Memory offset of every element, in C-order logical enumeration."""
    shape, strides = info_shape(info), info_strides(info)
    if not shape:
        return np.zeros(1, dtype=np.int64)
    idx = np.indices(shape).reshape(len(shape), -1)
    return (idx * np.array(strides, dtype=np.int64)[:, None]).sum(axis=0)


def span_of(info):
    """Number of elements a buffer must hold for the view described by info."""
    shape, strides = info_shape(info), info_strides(info)
    span = 1
    for s, t in zip(shape, strides):
        if s > 0:
            span += (s - 1) * abs(t)
    return span


class DeviceArray(object):
    def __init__(self, dev, ptr, nbytes):
        self.dev = dev
        self.ptr = ptr
        self.nbytes = nbytes

    def download(self, dtype, count=None):
        dtype = np.dtype(dtype)
        if count is None:
            count = self.nbytes // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        if count:
            self.dev.ops.streamSynchronize(self.dev.stream)
            self.dev.ops.memcpy(out.ctypes.data, self.ptr, count * dtype.itemsize, 2, None)
        return out

    def free(self):
        if self.ptr:
            self.dev.ops.freeDevice(self.ptr, None)
            self.ptr = None


class Device(object):
    """One GPU, one stream, and the buffers a caller keeps resident."""

    def __init__(self):
        self.ops = NativeOps()
        self.ops.initializeDevicesAndFunctions()
        if self.ops.getAvailableDevices() < 1:
            raise RuntimeError("no GPU visible")
        self.stream = self.ops.createStream()
        self._keep = []

    def empty(self, nbytes):
        ptr = self.ops.mallocDevice(max(int(nbytes), 16), None, 0)
        if not ptr:
            raise MemoryError("mallocDevice(%d) failed" % nbytes)
        return DeviceArray(self, ptr, int(nbytes))

    def upload(self, array):
        array = np.ascontiguousarray(array)
        d = self.empty(array.nbytes)
        if array.nbytes:
            self.ops.memcpy(d.ptr, array.ctypes.data, array.nbytes, 1, None)
        return d

    def sync(self):
        self.ops.streamSynchronize(self.stream)

    # ---- TAD tables -------------------------------------------------------------------------
    def tad(self, x_info, dims):
        """(tadShapeInfo, offsets) from the library's tadOnlyShapeInfo (host side)."""
        x_info = np.ascontiguousarray(x_info, dtype=np.int64)
        dims_np = np.array(list(dims), dtype=np.int32)
        rank = int(x_info[0])
        tad_len = 1
        for d in dims:
            tad_len *= int(x_info[1 + (d % rank)])
        n = info_numel(x_info)
        num = n // tad_len if tad_len else 0
        target = np.zeros(2 * max(rank, 2) + 4, dtype=np.int64)
        offsets = np.zeros(max(num, 1), dtype=np.int64)
        self.ops.tadOnlyShapeInfo(x_info.ctypes.data, dims_np.ctypes.data, len(dims), target.ctypes.data,
                                  offsets.ctypes.data)
        r = int(target[0])
        return target[:2 * r + 4].copy(), offsets[:num].copy()

    # ---- extraPointers ----------------------------------------------------------------------
    def extra(self, x_info=None, y_info=None, z_info=None, tad=None, tad_z=None, host_buffer=None):
        """extraPointers of the CUDA convention (reference: blas/cuda/NativeOps.cu:1813-1823): [0] host
        xShapeInfo (or the host u64 buffer for initRandom), [1] stream, [7]/[8] host y/z shapeInfo, [9] host TAD
        shapeInfo, [10]/[11] device TAD shapeInfo/offsets, [12]/[13] the same for the result.  ``tad`` and
        ``tad_z`` are (tadShapeInfo, offsets) numpy pairs; their device copies are kept alive by this object."""
        arr = (ctypes.c_void_p * 20)()
        keep = []

        def host(a):
            a = np.ascontiguousarray(a, dtype=np.int64)
            keep.append(a)
            return a.ctypes.data

        if host_buffer is not None:
            arr[0] = host_buffer
        elif x_info is not None:
            arr[0] = host(x_info)
        arr[1] = self.stream
        arr[2] = 0
        if y_info is not None:
            arr[7] = host(y_info)
        if z_info is not None:
            arr[8] = host(z_info)
        if tad is not None:
            arr[9] = host(tad[0])
            d_info = self.upload(np.ascontiguousarray(tad[0], dtype=np.int64))
            d_off = self.upload(np.ascontiguousarray(tad[1], dtype=np.int64))
            keep += [d_info, d_off]
            arr[10] = d_info.ptr
            arr[11] = d_off.ptr
        if tad_z is not None:
            d_info = self.upload(np.ascontiguousarray(tad_z[0], dtype=np.int64))
            d_off = self.upload(np.ascontiguousarray(tad_z[1], dtype=np.int64))
            keep += [d_info, d_off]
            arr[12] = d_info.ptr
            arr[13] = d_off.ptr
        self._keep.append(keep)
        arr._keep = keep
        return arr

    def release(self):
        """Frees the device copies created by extra()."""
        self.sync()
        for keep in self._keep:
            for k in keep:
                if isinstance(k, DeviceArray):
                    k.free()
        self._keep = []


class Operand(object):
    """A device-resident array with its shapeInfo on host and device."""

    def __init__(self, dev, data, info):
        self.dev = dev
        self.info = np.ascontiguousarray(info, dtype=np.int64)
        self.dtype = np.dtype(data.dtype)
        self.buf = dev.upload(data)
        self.dinfo = dev.upload(self.info)
        self.count = int(data.size)

    @property
    def ptr(self):
        return self.buf.ptr

    @property
    def info_ptr(self):
        return self.dinfo.ptr

    def get(self):
        return self.buf.download(self.dtype, self.count)

    def free(self):
        self.buf.free()
        self.dinfo.free()
