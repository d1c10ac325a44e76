"""ctypes binding of libnd4j_amd.so and a thin host-side mirror of the reference's ``NativeOps`` class.

The method names, argument order and argument meaning are those of the reference's ``blas/NativeOps.h``
(hot-path members only).  Where the C++ class overloads a member, the Python method of the same name picks
the overload from the arguments (an ``int`` stride selects the strided overload, index buffers the indexed
one), and the explicit C names (``...Strided``, ``...Full``, ``...XZ``, ``...XYZ``) are available too.

All pointers are plain integers (device or host addresses).  Nothing here computes anything: the library
must be built (``libnd4j_amd/csrc/build.sh``) or loading fails loudly.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libnd4j_amd.so")

c_void_p = ctypes.c_void_p
c_ll = ctypes.c_longlong
c_int = ctypes.c_int

_SUFFIX_RET = {"Float": ctypes.c_float, "Half": ctypes.c_float, "Double": ctypes.c_double}

# (C name template, argument ctypes, returns-scalar)
_P = c_void_p
_EXEC_SIGNATURES = {
    "nd4j_execIndexReduceScalar{S}": ([_P, c_int, _P, _P, _P], True),
    "nd4j_execIndexReduce{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, c_int], False),
    "nd4j_execBroadcast{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P, c_int], False),
    "nd4j_execPairwiseTransform{S}Strided": ([_P, c_int, _P, c_ll, _P, c_ll, _P, c_ll, _P, c_ll], False),
    "nd4j_execPairwiseTransform{S}Indexed": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P], False),
    "nd4j_execPairwiseTransform{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P], False),
    "nd4j_execReduce{S}Full": ([_P, c_int, _P, _P, _P, _P, _P], False),
    "nd4j_execReduce{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, c_int], False),
    "nd4j_execReduceScalar{S}": ([_P, c_int, _P, _P, _P], True),
    "nd4j_execSummaryStatsScalar{S}": ([_P, c_int, _P, _P, _P, c_int], True),
    "nd4j_execSummaryStats{S}Full": ([_P, c_int, _P, _P, _P, _P, _P, c_int], False),
    "nd4j_execSummaryStats{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, c_int, c_int], False),
    "nd4j_execTransform{S}Strided": ([_P, c_int, _P, c_ll, _P, c_ll, _P, c_ll], False),
    "nd4j_execTransform{S}": ([_P, c_int, _P, _P, _P, _P, _P], False),
    "nd4j_execTransform{S}Indexed": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P], False),
    "nd4j_execRandom{S}": ([_P, c_int, _P, _P, _P, _P], False),
    "nd4j_execRandom{S}XYZ": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P], False),
    "nd4j_execRandom{S}XZ": ([_P, c_int, _P, _P, _P, _P, _P, _P], False),
    "nd4j_execReduce3{S}Full": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P], False),
    "nd4j_execReduce3Scalar{S}": ([_P, c_int, _P, _P, _P, _P, _P], True),
    "nd4j_execReduce3{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, c_int], False),
    "nd4j_execReduce3All{S}": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, c_int, _P, _P, _P, _P], False),
    # _SCALAR stands for the by-value scalar: float for Float and Half, double for Double
    "nd4j_execScalar{S}Strided": ([_P, c_int, _P, c_ll, _P, c_ll, "_SCALAR", _P, c_ll], False),
    "nd4j_execScalar{S}": ([_P, c_int, _P, _P, _P, _P, "_SCALAR", _P], False),
    "nd4j_execScalar{S}Indexed": ([_P, c_int, _P, _P, _P, _P, "_SCALAR", _P, _P, _P], False),
    "nd4j_execScalar{S}AlongDimension": ([_P, c_int, _P, _P, _P, _P, _P, _P, _P, c_int], False),
    # data-movement specials
    "nd4j_flatten{S}": ([_P, c_int, ctypes.c_char, _P, _P, _P, _P], False),
    "nd4j_concat{S}": ([_P, c_int, c_int, _P, _P, _P, _P, _P, _P], False),
    "nd4j_pullRows{S}": ([_P, _P, _P, _P, _P, c_ll, _P, _P, _P, _P, _P], False),
    "nd4j_tear{S}": ([_P, _P, _P, _P, _P, _P, _P], False),
    "nd4j_shuffle{S}": ([_P, _P, _P, _P, _P, c_int, _P, _P, _P], False),
    "nd4j_average{S}": ([_P, _P, _P, c_int, c_ll, c_int], False),
    "nd4j_accumulate{S}": ([_P, _P, _P, c_int, c_ll], False),
}

_PLAIN_SIGNATURES = {
    "nd4j_lastError": ([], ctypes.c_char_p),
    "nd4j_initRandom": ([_P, ctypes.c_long, ctypes.c_long, _P], _P),
    "nd4j_refreshBuffer": ([_P, ctypes.c_long, _P], None),
    "nd4j_reSeedBuffer": ([_P, ctypes.c_long, _P], None),
    "nd4j_destroyRandom": ([_P], None),
    "nd4j_tadOnlyShapeInfo": ([_P, _P, c_int, _P, _P], None),
    "nd4j_convertTypes": ([_P, c_int, _P, c_ll, c_int, _P], None),
    "nd4j_initializeDevicesAndFunctions": ([], None),
    "nd4j_mallocHost": ([c_ll, c_int], _P),
    "nd4j_mallocDevice": ([c_ll, _P, c_int], _P),
    "nd4j_freeHost": ([_P], c_int),
    "nd4j_freeDevice": ([_P, _P], c_int),
    "nd4j_ompGetMaxThreads": ([], c_int),
    "nd4j_ompGetNumThreads": ([], c_int),
    "nd4j_setOmpNumThreads": ([c_int], None),
    "nd4j_setOmpMinThreads": ([c_int], None),
    "nd4j_createContext": ([], _P),
    "nd4j_createStream": ([], _P),
    "nd4j_createEvent": ([], _P),
    "nd4j_registerEvent": ([_P, _P], c_int),
    "nd4j_destroyEvent": ([_P], c_int),
    "nd4j_setDevice": ([_P], c_int),
    "nd4j_getDevice": ([], c_int),
    "nd4j_streamSynchronize": ([_P], c_int),
    "nd4j_eventSynchronize": ([_P], c_int),
    "nd4j_getDeviceFreeMemory": ([_P], c_ll),
    "nd4j_getDeviceTotalMemory": ([_P], c_ll),
    "nd4j_getDeviceMajor": ([_P], c_int),
    "nd4j_getDeviceMinor": ([_P], c_int),
    "nd4j_getDeviceName": ([_P], ctypes.c_char_p),
    "nd4j_memcpy": ([_P, _P, c_ll, c_int, _P], c_int),
    "nd4j_memcpyAsync": ([_P, _P, c_ll, c_int, _P], c_int),
    "nd4j_memset": ([_P, c_int, c_ll, c_int, _P], c_int),
    "nd4j_memsetAsync": ([_P, c_int, c_ll, c_int, _P], c_int),
    "nd4j_memcpyConstantAsync": ([c_ll, _P, c_ll, c_int, _P], c_int),
    "nd4j_getConstantSpace": ([], _P),
    "nd4j_getAvailableDevices": ([], c_int),
    "nd4j_enableDebugMode": ([c_int], None),
    "nd4j_enableVerboseMode": ([c_int], None),
    "nd4j_setGridLimit": ([c_int], None),
    "nd4j_setElementThreshold": ([c_int], None),
    "nd4j_setTADThreshold": ([c_int], None),
    "nd4j_amd_rngDump": ([_P, _P, c_ll, c_ll, _P], None),
    "nd4j_amd_rngState": ([_P, _P], None),
    "nd4j_amd_timerCreate": ([], _P),
    "nd4j_amd_timerRecord": ([_P, _P], c_int),
    "nd4j_amd_timerElapsedMs": ([_P, _P], ctypes.c_float),
    "nd4j_amd_timerDestroy": ([_P], c_int),
    "nd4j_amd_copyKernel": ([_P, _P, _P, c_ll], None),
    "nd4j_amd_hostFetchCount": ([], c_ll),
    "nd4j_amd_setCooperativeWaitLimit": ([c_int], None),
    "nd4j_amd_forderTileCopy": ([_P, _P, _P, c_ll, c_ll], None),
    "nd4j_amd_releaseStream": ([_P], None),
    "nd4j_amd_setSlotTicket": ([_P, ctypes.c_uint], None),
    "nd4j_amd_execReduceFloatNoAlloc": ([_P, c_int, _P, _P, _P, _P], None),
}


def exported_symbol_names():
    """Every symbol include/nd4j_native_c.h declares."""
    names = list(_PLAIN_SIGNATURES)
    for template in _EXEC_SIGNATURES:
        for suffix in _SUFFIX_RET:
            names.append(template.format(S=suffix))
    return names


class Nd4jError(RuntimeError):
    """A device failure reported by the library (std::runtime_error on the reference)."""


_lib = None


def load_library(path=None):
    """Loads libnd4j_amd.so (once).  Raises if the library has not been built: there is no fallback."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIBRARY_PATH
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with libnd4j_amd/csrc/build.sh (hipcc, gfx950); "
            "there is no CPU fallback for the op path" % path)
    lib = ctypes.CDLL(path)
    for name, (args, ret) in _PLAIN_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = ret
    for template, (args, scalar) in _EXEC_SIGNATURES.items():
        for suffix, ret in _SUFFIX_RET.items():
            fn = getattr(lib, template.format(S=suffix))
            fn.argtypes = [ret if a == "_SCALAR" else a for a in args]
            fn.restype = ret if scalar else None
    _lib = lib
    return lib


class NativeOps(object):
    """Python mirror of the reference's ``class NativeOps`` (blas/NativeOps.h), hot-path members."""

    def __init__(self, path=None):
        self._lib = load_library(path)

    # -- plumbing --------------------------------------------------------------------------------
    def _check(self):
        msg = self._lib.nd4j_lastError()
        if msg:
            raise Nd4jError(msg.decode("utf-8", "replace"))

    def _call(self, name, *args):
        r = getattr(self._lib, name)(*args)
        self._check()
        return r

    def __getattr__(self, name):
        # plain members: initRandom, mallocDevice, createStream, ...
        lib = object.__getattribute__(self, "_lib")
        cname = "nd4j_" + name
        if cname in _PLAIN_SIGNATURES:
            def plain(*args):
                return self._call(cname, *args)
            plain.__name__ = name
            return plain
        for suffix in _SUFFIX_RET:
            for template in _EXEC_SIGNATURES:
                if template.format(S=suffix) == cname:
                    def explicit(*args, _c=cname):
                        return self._call(_c, *args)
                    explicit.__name__ = name
                    return explicit
        raise AttributeError(name)

    # -- overloaded members, resolved like the C++ overload set -------------------------------------
    def _transform(self, S, extra, opNum, dx, a, result, b, extraParams, *rest):
        # 8 arguments: strided (a, b are strides, rest = n); 7: shaped; 9: indexed
        if len(rest) == 1:
            return self._call("nd4j_execTransform%sStrided" % S, extra, opNum, dx, a, result, b, extraParams, rest[0])
        if len(rest) == 2:
            return self._call("nd4j_execTransform%sIndexed" % S, extra, opNum, dx, a, result, b, extraParams, *rest)
        return self._call("nd4j_execTransform%s" % S, extra, opNum, dx, a, result, b, extraParams)

    def _pairwise(self, S, extra, opNum, dx, a, y, b, result, c, extraParams, *rest):
        if len(rest) == 1:
            return self._call("nd4j_execPairwiseTransform%sStrided" % S, extra, opNum, dx, a, y, b, result, c,
                              extraParams, rest[0])
        if len(rest) == 3:
            return self._call("nd4j_execPairwiseTransform%sIndexed" % S, extra, opNum, dx, a, y, b, result, c,
                              extraParams, *rest)
        return self._call("nd4j_execPairwiseTransform%s" % S, extra, opNum, dx, a, y, b, result, c, extraParams)

    def _reduce(self, S, extra, opNum, x, xShapeInfo, extraParams, result, resultShapeInfo, *rest):
        if len(rest) == 2:
            return self._call("nd4j_execReduce%s" % S, extra, opNum, x, xShapeInfo, extraParams, result,
                              resultShapeInfo, rest[0], rest[1])
        return self._call("nd4j_execReduce%sFull" % S, extra, opNum, x, xShapeInfo, extraParams, result,
                          resultShapeInfo)

    def _stats(self, S, extra, opNum, x, xShapeInfo, extraParams, result, resultShapeInfo, *rest):
        if len(rest) == 3:
            return self._call("nd4j_execSummaryStats%s" % S, extra, opNum, x, xShapeInfo, extraParams, result,
                              resultShapeInfo, rest[0], rest[1], int(bool(rest[2])))
        return self._call("nd4j_execSummaryStats%sFull" % S, extra, opNum, x, xShapeInfo, extraParams, result,
                          resultShapeInfo, int(bool(rest[0])))

    def _scalar(self, S, extra, opNum, x, a, result, b, c, d, *rest):
        # strided: (x, xStride, result, resultStride, scalar, extraParams, n); shaped: (x, xInfo, result, resultInfo,
        # scalar, extraParams); indexed: shaped + two index buffers; along a dimension: (x, xInfo, z, zInfo, scalars,
        # extraParams, dimension, dimensionLength)
        if len(rest) == 1:
            return self._call("nd4j_execScalar%sStrided" % S, extra, opNum, x, a, result, b, c, d, rest[0])
        if len(rest) == 0:
            return self._call("nd4j_execScalar%s" % S, extra, opNum, x, a, result, b, c, d)
        if isinstance(rest[1], int) and not isinstance(c, float):
            return self._call("nd4j_execScalar%sAlongDimension" % S, extra, opNum, x, a, result, b, c, d, rest[0], rest[1])
        return self._call("nd4j_execScalar%sIndexed" % S, extra, opNum, x, a, result, b, c, d, rest[0], rest[1])

    def _reduce3(self, S, extra, opNum, x, xInfo, params, y, yInfo, result, resultInfo, *rest):
        if len(rest) == 2:
            return self._call("nd4j_execReduce3%s" % S, extra, opNum, x, xInfo, params, y, yInfo, result, resultInfo, *rest)
        return self._call("nd4j_execReduce3%sFull" % S, extra, opNum, x, xInfo, params, y, yInfo, result, resultInfo)

    def _random(self, S, extra, opNum, state, *rest):
        if len(rest) == 3:
            return self._call("nd4j_execRandom%s" % S, extra, opNum, state, *rest)
        if len(rest) == 5:
            return self._call("nd4j_execRandom%sXZ" % S, extra, opNum, state, *rest)
        return self._call("nd4j_execRandom%sXYZ" % S, extra, opNum, state, *rest)


def _install_overloads():
    for S in _SUFFIX_RET:
        def mk(kind, S=S):
            def method(self, *args):
                return getattr(self, kind)(S, *args)
            return method
        setattr(NativeOps, "execTransform" + S, mk("_transform"))
        setattr(NativeOps, "execPairwiseTransform" + S, mk("_pairwise"))
        setattr(NativeOps, "execReduce" + S, mk("_reduce"))
        setattr(NativeOps, "execSummaryStats" + S, mk("_stats"))
        setattr(NativeOps, "execRandom" + S, mk("_random"))
        setattr(NativeOps, "execScalar" + S, mk("_scalar"))
        setattr(NativeOps, "execReduce3" + S, mk("_reduce3"))


_install_overloads()
