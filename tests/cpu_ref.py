"""ctypes wrapper over the CPU checkers (TEST INFRASTRUCTURE).

Two libraries export the same ``nd4j_cpu_*`` C interface:
  * ``oracle/libnd4j_oracle.so``  - this repository's CPU restatement of the reference loops ("port");
  * ``oracle/_ref/libnd4j_ref.so`` - the reference's own loop sources compiled as they are ("reference"),
    present when it was built in a container that has the reference tree.
Arrays are numpy arrays in host memory; shapeInfo buffers are int64 numpy arrays.
"""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "libnd4j_oracle.so")
REF_PATH = os.path.join(ROOT, "oracle", "_ref", "libnd4j_ref.so")

SUF = {np.dtype(np.float32): "f32", np.dtype(np.float16): "f16", np.dtype(np.float64): "f64"}


def _p(a):
    if a is None:
        return None
    return a.ctypes.data


def _ints(v):
    return np.ascontiguousarray(v, dtype=np.int32)


def _info(v):
    return np.ascontiguousarray(v, dtype=np.int64)


class CpuLib(object):
    def __init__(self, path):
        self.path = path
        self.lib = ctypes.CDLL(path)
        L = self.lib
        L.nd4j_cpu_kind.restype = ctypes.c_char_p
        L.nd4j_cpu_rng_init.restype = ctypes.c_void_p
        L.nd4j_cpu_rng_init.argtypes = [ctypes.c_longlong, ctypes.c_longlong, ctypes.c_void_p]
        for name in ("refresh", "reseed", "rewind", "set_offset"):
            getattr(L, "nd4j_cpu_rng_" + name).argtypes = [ctypes.c_void_p, ctypes.c_longlong]
        L.nd4j_cpu_rng_destroy.argtypes = [ctypes.c_void_p]
        L.nd4j_cpu_rng_state.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.nd4j_cpu_rng_elements.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_longlong, ctypes.c_void_p]
        L.nd4j_cpu_rng_uniform_f32.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_longlong, ctypes.c_void_p]
        L.nd4j_cpu_tad_only_shape_info.restype = ctypes.c_longlong
        L.nd4j_cpu_tad_only_shape_info.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                                   ctypes.c_void_p]
        L.nd4j_cpu_tad_count.restype = ctypes.c_longlong
        L.nd4j_cpu_tad_count.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.nd4j_cpu_shape_buffer.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        L.nd4j_cpu_compute_ews.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.nd4j_cpu_get_order.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.nd4j_cpu_set_thresholds.argtypes = [ctypes.c_int, ctypes.c_int]
        L.nd4j_cpu_set_threads.argtypes = [ctypes.c_int]
        V, I, LL = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
        sigs = {
            "transform": [I, V, V, V, V, V],
            "transform_strided": [I, V, LL, V, LL, V, LL],
            "reduce3_scalar": [I, V, V, V, V, V, V],
            "reduce3": [I, V, V, V, V, V, V, V, V, I],
            "reduce3_tad": [I, V, V, V, V, V, V, V, V, I],
            "reduce3_all": [I, V, V, V, V, V, V, V, V, I],
            "scalar": [I, V, V, V, V, ctypes.c_double, V],
            "scalar_strided": [I, V, LL, V, LL, ctypes.c_double, V, LL],
            "scalar_tad": [I, V, V, V, V, V, V, V, I],
            "pairwise": [I, V, V, V, V, V, V, V],
            "pairwise_strided": [I, V, LL, V, LL, V, LL, V, LL],
            "broadcast": [I, V, V, V, V, V, V, V, I],
            "reduce": [I, V, V, V, V, V, V, I],
            "reduce_scalar": [I, V, V, V, V],
            "indexreduce": [I, V, V, V, V, V, V, I],
            "indexreduce_scalar": [I, V, V, V, V],
            "summarystats": [I, I, V, V, V, V, V, V, I],
            "summarystats_scalar": [I, I, V, V, V, V],
            "random_z": [I, V, V, V, V],
            "random_xz": [I, V, V, V, V, V, V],
            "random_xyz": [I, V, V, V, V, V, V, V, V],
            "flatten": [I, I, V, V, V, V],
            "concat": [I, I, V, V, V, V],
            "pullrows": [V, V, V, V, LL, V, V, V, V, V],
            "tear": [V, V, V, V, V, V],
            "shuffle": [V, V, I, V, V, V],
            "average": [V, V, I, LL, I],
            "accumulate": [V, V, I, LL],
        }
        L.nd4j_cpu_convert.restype = I
        L.nd4j_cpu_convert.argtypes = [I, V, LL, I, V]
        for fam, sig in sigs.items():
            for suf in SUF.values():
                fn = getattr(L, "nd4j_cpu_%s_%s" % (fam, suf))
                fn.argtypes = sig
                fn.restype = None

    @property
    def kind(self):
        return self.lib.nd4j_cpu_kind().decode()

    def _fn(self, fam, arr):
        return getattr(self.lib, "nd4j_cpu_%s_%s" % (fam, SUF[np.dtype(arr.dtype)]))

    # -- data movement ---------------------------------------------------------------------------------
    @staticmethod
    def _table(arrays):
        return (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])

    def flatten(self, offset, order, z, z_info, x, x_info):
        self._fn("flatten", x)(offset, ord(order), _p(z), _p(_info(z_info)), _p(x), _p(_info(x_info)))

    def concat(self, dim, arrays, infos, z, z_info):
        infos = [_info(i) for i in infos]
        self._fn("concat", z)(dim, len(arrays), self._table(arrays), self._table(infos), _p(z), _p(_info(z_info)))

    def pullrows(self, x, x_info, z, z_info, indexes, tad, z_tad):
        idx = np.ascontiguousarray(indexes, dtype=np.int64)
        ti, to, zi, zo = [_info(v) for v in (tad[0], tad[1], z_tad[0], z_tad[1])]
        self._fn("pullrows", x)(_p(x), _p(_info(x_info)), _p(z), _p(_info(z_info)), len(idx), _p(idx), _p(ti), _p(to), _p(zi),
                                _p(zo))

    def tear(self, x, x_info, targets, z_info, tad):
        ti, to = _info(tad[0]), _info(tad[1])
        self._fn("tear", x)(_p(x), _p(_info(x_info)), self._table(targets), _p(_info(z_info)), _p(ti), _p(to))

    def shuffle(self, arrays, infos, shuffle_map, tads):
        infos = [_info(i) for i in infos]
        tis = [_info(t[0]) for t in tads]
        tos = [_info(t[1]) for t in tads]
        m = _ints(shuffle_map)
        self._fn("shuffle", arrays[0])(self._table(arrays), self._table(infos), len(arrays), _p(m), self._table(tis),
                                       self._table(tos))

    def average(self, arrays, z, propagate):
        self._fn("average", arrays[0])(self._table(arrays), _p(z), len(arrays), arrays[0].size, int(propagate))

    def accumulate(self, arrays, z):
        self._fn("accumulate", arrays[0])(self._table(arrays), _p(z), len(arrays), arrays[0].size)

    def convert(self, src_type, x, dst_type, z):
        return self.lib.nd4j_cpu_convert(src_type, _p(x), x.size, dst_type, _p(z))

    # -- families -----------------------------------------------------------------------------------
    def transform(self, op, x, x_info, z, z_info, extra=None):
        self._fn("transform", x)(op, _p(x), _p(_info(x_info)), _p(z), _p(_info(z_info)), _p(extra))

    def transform_strided(self, op, x, xs, z, zs, extra, n):
        self._fn("transform_strided", x)(op, _p(x), xs, _p(z), zs, _p(extra), n)

    def reduce3_scalar(self, op, x, x_info, y, y_info, extra=None):
        out = np.zeros(1, x.dtype)
        self._fn("reduce3_scalar", x)(op, _p(x), _p(_info(x_info)), _p(extra), _p(y), _p(_info(y_info)), _p(out))
        return out[0]

    def _reduce3(self, which, op, x, x_info, y, y_info, z, z_info, dims, extra):
        d = _ints(dims)
        self._fn(which, x)(op, _p(x), _p(_info(x_info)), _p(extra), _p(y), _p(_info(y_info)), _p(z), _p(_info(z_info)),
                           _p(d), len(dims))

    def reduce3(self, op, x, x_info, y, y_info, z, z_info, dims, extra=None):
        self._reduce3("reduce3", op, x, x_info, y, y_info, z, z_info, dims, extra)

    def reduce3_tad(self, op, x, x_info, y, y_info, z, z_info, dims, extra=None):
        self._reduce3("reduce3_tad", op, x, x_info, y, y_info, z, z_info, dims, extra)

    def reduce3_all(self, op, x, x_info, y, y_info, z, z_info, dims, extra=None):
        self._reduce3("reduce3_all", op, x, x_info, y, y_info, z, z_info, dims, extra)

    def scalar(self, op, x, x_info, z, z_info, scalar, extra=None):
        self._fn("scalar", x)(op, _p(x), _p(_info(x_info)), _p(z), _p(_info(z_info)), float(scalar), _p(extra) if extra is not None else None)

    def scalar_strided(self, op, x, xs, z, zs, scalar, extra, n):
        self._fn("scalar_strided", x)(op, _p(x), xs, _p(z), zs, float(scalar), _p(extra) if extra is not None else None, n)

    def scalar_tad(self, op, x, x_info, z, z_info, scalars, extra, dims):
        d = _ints(dims)
        self._fn("scalar_tad", x)(op, _p(x), _p(_info(x_info)), _p(z), _p(_info(z_info)), _p(scalars),
                                  _p(extra) if extra is not None else None, _p(d), len(dims))

    def pairwise(self, op, x, x_info, y, y_info, z, z_info, extra=None):
        self._fn("pairwise", x)(op, _p(x), _p(_info(x_info)), _p(y), _p(_info(y_info)), _p(z), _p(_info(z_info)),
                                _p(extra))

    def pairwise_strided(self, op, x, xs, y, ys, z, zs, extra, n):
        self._fn("pairwise_strided", x)(op, _p(x), xs, _p(y), ys, _p(z), zs, _p(extra), n)

    def broadcast(self, op, x, x_info, y, y_info, z, z_info, dims):
        d = _ints(dims)
        self._fn("broadcast", x)(op, _p(x), _p(_info(x_info)), _p(y), _p(_info(y_info)), _p(z), _p(_info(z_info)),
                                 _p(d), len(d))

    def reduce(self, op, x, x_info, extra, z, z_info, dims):
        d = _ints(dims)
        self._fn("reduce", x)(op, _p(x), _p(_info(x_info)), _p(extra), _p(z), _p(_info(z_info)), _p(d), len(d))

    def reduce_scalar(self, op, x, x_info, extra=None):
        out = np.zeros(1, dtype=x.dtype)
        self._fn("reduce_scalar", x)(op, _p(x), _p(_info(x_info)), _p(extra), _p(out))
        return out[0]

    def indexreduce(self, op, x, x_info, extra, z, z_info, dims):
        d = _ints(dims)
        self._fn("indexreduce", x)(op, _p(x), _p(_info(x_info)), _p(extra), _p(z), _p(_info(z_info)), _p(d), len(d))

    def indexreduce_scalar(self, op, x, x_info, extra=None):
        out = np.zeros(1, dtype=x.dtype)
        self._fn("indexreduce_scalar", x)(op, _p(x), _p(_info(x_info)), _p(extra), _p(out))
        return out[0]

    def summarystats(self, op, bias, x, x_info, z, z_info, dims):
        d = _ints(dims)
        self._fn("summarystats", x)(op, int(bool(bias)), _p(x), _p(_info(x_info)), None, _p(z), _p(_info(z_info)),
                                    _p(d), len(d))

    def summarystats_scalar(self, op, bias, x, x_info):
        out = np.zeros(1, dtype=x.dtype)
        self._fn("summarystats_scalar", x)(op, int(bool(bias)), _p(x), _p(_info(x_info)), None, _p(out))
        return out[0]

    # -- rng ----------------------------------------------------------------------------------------
    def rng_init(self, seed, size):
        buf = np.zeros(size, dtype=np.uint64)
        st = self.lib.nd4j_cpu_rng_init(seed, size, buf.ctypes.data)
        return CpuRng(self, st, buf)

    # -- shape --------------------------------------------------------------------------------------
    def tad(self, x_info, dims):
        x_info = _info(x_info)
        d = _ints(dims)
        n = self.lib.nd4j_cpu_tad_count(_p(x_info), _p(d), len(d))
        rank = int(x_info[0])
        target = np.zeros(2 * max(rank, 2) + 4, dtype=np.int64)
        offsets = np.zeros(max(int(n), 1), dtype=np.int64)
        self.lib.nd4j_cpu_tad_only_shape_info(_p(x_info), _p(d), len(d), _p(target), _p(offsets))
        r = int(target[0])
        return target[:2 * r + 4].copy(), offsets[:int(n)].copy()

    def shape_buffer(self, shape, order):
        shp = np.ascontiguousarray(shape, dtype=np.int64)
        out = np.zeros(2 * len(shape) + 4, dtype=np.int64)
        self.lib.nd4j_cpu_shape_buffer(len(shape), _p(shp), ord(order), _p(out))
        return out

    def compute_ews(self, shape, strides, f_order=False):
        shp = np.ascontiguousarray(shape, dtype=np.int64)
        st = np.ascontiguousarray(strides, dtype=np.int64)
        return self.lib.nd4j_cpu_compute_ews(len(shape), _p(shp), _p(st), 1 if f_order else 0)

    def set_threads(self, n):
        self.lib.nd4j_cpu_set_threads(n)


class CpuRng(object):
    def __init__(self, lib, state, buf):
        self.lib = lib
        self.state = state
        self.buffer = buf

    def elements(self, start, n):
        out = np.zeros(n, dtype=np.uint64)
        self.lib.lib.nd4j_cpu_rng_elements(self.state, start, n, out.ctypes.data)
        return out

    def get_state(self):
        """(size, offset, seed, generation, amplifier)"""
        out = np.zeros(5, dtype=np.int64)
        self.lib.lib.nd4j_cpu_rng_state(self.state, out.ctypes.data)
        return tuple(int(v) for v in out)

    def refresh(self, seed):
        self.lib.lib.nd4j_cpu_rng_refresh(self.state, seed)

    def reseed(self, seed):
        self.lib.lib.nd4j_cpu_rng_reseed(self.state, seed)

    def rewind(self, n):
        self.lib.lib.nd4j_cpu_rng_rewind(self.state, n)

    def random_z(self, op, z, z_info, args):
        self.lib._fn("random_z", z)(op, self.state, _p(z), _p(_info(z_info)), _p(args))

    def random_xz(self, op, x, x_info, z, z_info, args):
        self.lib._fn("random_xz", z)(op, self.state, _p(x), _p(_info(x_info)), _p(z), _p(_info(z_info)), _p(args))

    def random_xyz(self, op, x, x_info, y, y_info, z, z_info, args):
        self.lib._fn("random_xyz", z)(op, self.state, _p(x), _p(_info(x_info)), _p(y), _p(_info(y_info)), _p(z),
                                      _p(_info(z_info)), _p(args))

    def destroy(self):
        if self.state:
            self.lib.lib.nd4j_cpu_rng_destroy(self.state)
            self.state = None


def load_oracle():
    if not os.path.exists(ORACLE_PATH):
        raise ImportError("%s missing: run `make -C oracle oracle`" % ORACLE_PATH)
    return CpuLib(ORACLE_PATH)


def load_reference():
    """The compiled reference, or None when it was not built (no reference tree at build time)."""
    if not os.path.exists(REF_PATH):
        return None
    return CpuLib(REF_PATH)
