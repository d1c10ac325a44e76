"""Two interchangeable ways of running one legacy op on numpy data, so that the same parity checks can be
pointed at a CPU checker (oracle restatement or compiled reference) or at the HIP path.

  CpuBackend(lib)  calls the nd4j_cpu_* interface of tests/cpu_ref.py on host arrays.
  GpuBackend()     uploads the operands, builds shapeInfo / TAD tables / extraPointers as a host of the
                   library would, calls libnd4j_amd.so through its C ABI, and downloads the result.

Array arguments are flat numpy buffers (the memory of the view); *_info are shapeInfo arrays.
"""
import ctypes

import numpy as np

from golden_inputs import shape_info_np


def _vec_info(n):
    return shape_info_np([1, int(n)])


def _span(info):
    r = int(info[0])
    span = 1
    for s, t in zip(info[1:1 + r], info[1 + r:1 + 2 * r]):
        if s > 0:
            span += (int(s) - 1) * abs(int(t))
    return span


class CpuBackend(object):
    name = "cpu"

    def __init__(self, lib):
        self.lib = lib
        self.kind = lib.kind

    def transform(self, op, x, x_info, z_info, extra=None, z=None):
        z = np.zeros(_span(z_info), x.dtype) if z is None else z.copy()
        self.lib.transform(op, x, x_info, z, z_info, extra)
        return z

    def transform_inplace(self, op, x, x_info, extra=None):
        z = x.copy()
        self.lib.transform(op, z, x_info, z, x_info, extra)
        return z

    def transform_strided(self, op, x, xs, zs, extra, n, zsize=None):
        z = np.zeros(zsize if zsize is not None else max(1, (n - 1) * zs + 1), x.dtype)
        self.lib.transform_strided(op, x, xs, z, zs, extra, n)
        return z

    def pairwise(self, op, x, x_info, y, y_info, z_info, extra=None):
        z = np.zeros(_span(z_info), x.dtype)
        self.lib.pairwise(op, x, x_info, y, y_info, z, z_info, extra)
        return z

    def scalar(self, op, x, x_info, z_info, scalar, extra=None):
        z = np.zeros(_span(z_info), x.dtype)
        self.lib.scalar(op, x, x_info, z, z_info, scalar, extra)
        return z

    def scalar_strided(self, op, x, xs, zs, scalar, extra, n):
        z = np.zeros(max(1, (n - 1) * zs + 1), x.dtype)
        self.lib.scalar_strided(op, x, xs, z, zs, scalar, extra, n)
        return z

    def scalar_tad(self, op, x, x_info, scalars, extra, dims):
        z = np.zeros(_span(x_info), x.dtype)
        self.lib.scalar_tad(op, x, x_info, z, x_info, scalars, extra, dims)
        return z

    def pairwise_strided(self, op, x, xs, y, ys, zs, extra, n):
        z = np.zeros(max(1, (n - 1) * zs + 1), x.dtype)
        self.lib.pairwise_strided(op, x, xs, y, ys, z, zs, extra, n)
        return z

    def broadcast(self, op, x, x_info, y, y_info, z_info, dims):
        z = np.zeros(_span(z_info), x.dtype)
        self.lib.broadcast(op, x, x_info, y, y_info, z, z_info, dims)
        return z

    def reduce(self, op, x, x_info, extra, dims, out_len):
        z = np.zeros(out_len, x.dtype)
        self.lib.reduce(op, x, x_info, extra, z, _vec_info(out_len), dims)
        return z

    def reduce_scalar(self, op, x, x_info, extra=None):
        return self.lib.reduce_scalar(op, x, x_info, extra)

    def indexreduce(self, op, x, x_info, extra, dims, out_len):
        z = np.zeros(out_len, x.dtype)
        self.lib.indexreduce(op, x, x_info, extra, z, _vec_info(out_len), dims)
        return z

    def reduce3_scalar(self, op, x, x_info, y, y_info, extra=None):
        return self.lib.reduce3_scalar(op, x, x_info, y, y_info, extra)

    def reduce3(self, op, x, x_info, y, y_info, extra, dims, out_len, tad_way=False):
        """tad_way: the reference's variant that is handed the x TAD tables (its only defined one when y is a
        single TAD); the other checkers treat both alike"""
        z = np.zeros(out_len, x.dtype)
        fn = self.lib.reduce3_tad if tad_way else self.lib.reduce3
        fn(op, x, x_info, y, y_info, z, _vec_info(out_len), dims, extra)
        return z

    def reduce3_all(self, op, x, x_info, y, y_info, extra, dims, out_len):
        z = np.zeros(out_len, x.dtype)
        self.lib.reduce3_all(op, x, x_info, y, y_info, z, _vec_info(out_len), dims, extra)
        return z

    def indexreduce_scalar(self, op, x, x_info, extra=None):
        return self.lib.indexreduce_scalar(op, x, x_info, extra)

    def summarystats(self, op, bias, x, x_info, dims, out_len):
        z = np.zeros(out_len, x.dtype)
        self.lib.summarystats(op, bias, x, x_info, z, _vec_info(out_len), dims)
        return z

    def summarystats_scalar(self, op, bias, x, x_info):
        return self.lib.summarystats_scalar(op, bias, x, x_info)

    # ---- data movement ---------------------------------------------------------------------------
    def flatten(self, offset, order, x, x_info, z_len, z_info=None):
        z = np.zeros(z_len, x.dtype)
        self.lib.flatten(offset, order, z, _vec_info(z_len) if z_info is None else z_info, x, x_info)
        return z

    def concat(self, dim, arrays, infos, z_info):
        z = np.zeros(_span(z_info), arrays[0].dtype)
        self.lib.concat(dim, arrays, infos, z, z_info)
        return z

    def pullrows(self, x, x_info, z_info, indexes, tad, z_tad):
        z = np.zeros(_span(z_info), x.dtype)
        self.lib.pullrows(x, x_info, z, z_info, indexes, tad, z_tad)
        return z

    def tear(self, x, x_info, z_info, tad):
        targets = [np.zeros(_span(z_info), x.dtype) for _ in range(len(tad[1]))]
        self.lib.tear(x, x_info, targets, z_info, tad)
        return targets

    def shuffle(self, arrays, infos, shuffle_map, tads):
        out = [a.copy() for a in arrays]
        self.lib.shuffle(out, infos, shuffle_map, tads)
        return out

    def average(self, arrays, propagate=False, with_z=True):
        """returns (z or None, the inputs afterwards)"""
        xs = [a.copy() for a in arrays]
        z = np.zeros(xs[0].size, xs[0].dtype) if with_z else None
        self.lib.average(xs, z, propagate)
        return z, xs

    def accumulate(self, arrays):
        z = np.zeros(arrays[0].size, arrays[0].dtype)
        self.lib.accumulate([a.copy() for a in arrays], z)
        return z

    def convert(self, src_type, x, dst_type):
        z = np.zeros(x.size, TYPE_OF_CODE[dst_type])
        assert self.lib.convert(src_type, x, dst_type, z) == 1
        return z

    def tad(self, x_info, dims):
        return self.lib.tad(x_info, dims)

    def rng(self, seed, size):
        return _CpuRng(self.lib.rng_init(seed, size))


class _CpuRng(object):
    def __init__(self, g):
        self.g = g

    def elements(self, start, n):
        return self.g.elements(start, n)

    def state(self):
        return self.g.get_state()

    def rewind(self, n):
        self.g.rewind(n)

    def reseed(self, seed):
        self.g.reseed(seed)

    def refresh(self, seed):
        self.g.refresh(seed)

    @property
    def buffer(self):
        return self.g.buffer

    def random_z(self, op, n_or_info, args, dtype=np.float32):
        info = _vec_info(n_or_info) if np.isscalar(n_or_info) else n_or_info
        z = np.zeros(_span(info), dtype)
        self.g.random_z(op, z, info, np.asarray(args, dtype))
        return z

    def random_xz(self, op, x, args, inplace=True, info=None):
        info = _vec_info(x.size) if info is None else info
        xx = x.copy()
        a = np.asarray(args, x.dtype)
        if inplace:
            self.g.random_xz(op, xx, info, xx, info, a)
            return xx
        z = np.zeros_like(x)
        self.g.random_xz(op, xx, info, z, info, a)
        return z

    def random_xyz(self, op, x, y, args, mode="separate", n=None, dtype=np.float32):
        a = np.asarray(args, dtype)
        if mode == "inplace_all":  # x == y == z, the way ND4J issues the special distributions
            z = np.zeros(n, dtype)
            info = _vec_info(n)
            self.g.random_xyz(op, z, info, z, info, z, info, a)
            return z
        info = _vec_info(x.size)
        z = np.zeros_like(x)
        self.g.random_xyz(op, x.copy(), info, y.copy(), _vec_info(y.size), z, info, a)
        return z

    def choice(self, values, v_info, probs, p_info, z_info):
        """Choice (random op 5): z[i] = the value whose cumulative probability first reaches the i-th draw."""
        z = np.zeros(_span(z_info), values.dtype)
        self.g.random_xyz(5, values.copy(), v_info, probs.copy(), p_info, z, z_info, np.zeros(1, values.dtype))
        return z

    def destroy(self):
        self.g.destroy()


TYPE_OF_CODE = {3: np.float16, 6: np.float32, 7: np.float64}


class GpuBackend(object):
    name = "gpu"
    kind = "hip"

    def __init__(self):
        from libnd4j_amd import harness
        self.h = harness
        self.dev = harness.Device()
        self.ops = self.dev.ops

    def _suffix(self, a):
        return self.h.SUFFIX_OF[np.dtype(a.dtype)]

    def _op(self, data, info):
        return self.h.Operand(self.dev, np.ascontiguousarray(data), info)

    def _up(self, a, dtype=None):
        if a is None:
            return None, None
        arr = np.ascontiguousarray(a, dtype=dtype)
        d = self.dev.upload(arr)
        return d, d.ptr

    def _finish(self, *operands):
        self.dev.sync()
        for o in operands:
            if o is not None:
                o.free()
        self.dev.release()

    # ---- data movement ---------------------------------------------------------------------------
    def _ptr_table(self, device_arrays):
        return self.dev.upload(np.array([d.ptr for d in device_arrays], dtype=np.uint64))

    def flatten(self, offset, order, x, x_info, z_len, z_info=None):
        z_info = _vec_info(z_len) if z_info is None else z_info
        X = self._op(x, x_info)
        Z = self._op(np.zeros(z_len, x.dtype), z_info)
        ptrs = self.dev.extra(y_info=x_info)  # the input's host shapeInfo travels in slot 7
        getattr(self.ops, "flatten" + self._suffix(x))(ptrs, offset, order.encode(), Z.ptr, Z.info_ptr, X.ptr, X.info_ptr)
        out = Z.get()
        self._finish(X, Z)
        return out

    def concat(self, dim, arrays, infos, z_info, host_shapes=True):
        ops = [self._op(a, i) for a, i in zip(arrays, infos)]
        Z = self._op(np.zeros(_span(z_info), arrays[0].dtype), z_info)
        data_tab = self._ptr_table([o.buf for o in ops])
        info_tab = self._ptr_table([o.dinfo for o in ops])
        ptrs = self.dev.extra(z_info)  # the result's host shapeInfo travels in slot 0
        host_infos = [np.ascontiguousarray(i, dtype=np.int64) for i in infos]
        host_tab = (ctypes.c_void_p * len(infos))(*[h.ctypes.data for h in host_infos])
        if host_shapes:
            ptrs[9] = ctypes.cast(host_tab, ctypes.c_void_p)
        data = (ctypes.c_void_p * 1)(data_tab.ptr)
        shapes = (ctypes.c_void_p * 1)(info_tab.ptr)
        getattr(self.ops, "concat" + self._suffix(arrays[0]))(ptrs, dim, len(arrays), data, shapes, Z.ptr, Z.info_ptr, None, None)
        out = Z.get()
        self._finish(Z, data_tab, info_tab, *ops)
        return out

    def pullrows(self, x, x_info, z_info, indexes, tad, z_tad):
        X = self._op(x, x_info)
        Z = self._op(np.zeros(_span(z_info), x.dtype), z_info)
        I, i = self._up(indexes, np.int64)
        parts = [self._up(v, np.int64) for v in (tad[0], tad[1], z_tad[0], z_tad[1])]
        getattr(self.ops, "pullRows" + self._suffix(x))(self.dev.extra(x_info), X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, len(indexes), i,
                                                        *[p[1] for p in parts])
        out = Z.get()
        self._finish(X, Z, I, *[p[0] for p in parts])
        return out

    def tear(self, x, x_info, z_info, tad):
        X = self._op(x, x_info)
        n = len(tad[1])
        span = _span(z_info)
        targets = [self.dev.upload(np.zeros(span, x.dtype)) for _ in range(n)]
        tab = self._ptr_table(targets)
        ZI, zi = self._up(z_info, np.int64)
        TI, ti = self._up(tad[0], np.int64)
        TO, to = self._up(tad[1], np.int64)
        getattr(self.ops, "tear" + self._suffix(x))(self.dev.extra(x_info), X.ptr, X.info_ptr, tab.ptr, zi, ti, to)
        self.dev.sync()
        out = [t.download(x.dtype, span) for t in targets]
        self._finish(X, tab, ZI, TI, TO, *targets)
        return out

    def shuffle(self, arrays, infos, shuffle_map, tads):
        ops = [self._op(a, i) for a, i in zip(arrays, infos)]
        tis = [self.dev.upload(np.ascontiguousarray(t[0], dtype=np.int64)) for t in tads]
        tos = [self.dev.upload(np.ascontiguousarray(t[1], dtype=np.int64)) for t in tads]
        x_tab = self._ptr_table([o.buf for o in ops])
        i_tab = self._ptr_table([o.dinfo for o in ops])
        ti_tab, to_tab = self._ptr_table(tis), self._ptr_table(tos)
        M, m = self._up(shuffle_map, np.int32)
        getattr(self.ops, "shuffle" + self._suffix(arrays[0]))(self.dev.extra(), x_tab.ptr, i_tab.ptr, x_tab.ptr, i_tab.ptr,
                                                               len(arrays), m, ti_tab.ptr, to_tab.ptr)
        out = [o.get() for o in ops]
        self._finish(x_tab, i_tab, ti_tab, to_tab, M, *(ops + tis + tos))
        return out

    def average(self, arrays, propagate=False, with_z=True):
        xs = [self.dev.upload(np.ascontiguousarray(a)) for a in arrays]
        tab = self._ptr_table(xs)
        n, dt = arrays[0].size, arrays[0].dtype
        Z = self.dev.upload(np.zeros(n, dt)) if with_z else None
        getattr(self.ops, "average" + self._suffix(arrays[0]))(self.dev.extra(), tab.ptr, Z.ptr if with_z else None, len(arrays), n,
                                                               int(propagate))
        self.dev.sync()
        z = Z.download(dt, n) if with_z else None
        out = [x.download(dt, n) for x in xs]
        self._finish(tab, Z, *xs)
        return z, out

    def accumulate(self, arrays):
        xs = [self.dev.upload(np.ascontiguousarray(a)) for a in arrays]
        tab = self._ptr_table(xs)
        n, dt = arrays[0].size, arrays[0].dtype
        Z = self.dev.upload(np.full(n, 7, dt))  # stale contents must not leak into the sum
        getattr(self.ops, "accumulate" + self._suffix(arrays[0]))(self.dev.extra(), tab.ptr, Z.ptr, len(arrays), n)
        z = Z.download(dt, n)
        self._finish(tab, Z, *xs)
        return z

    def convert(self, src_type, x, dst_type):
        X, xp = self._up(x)
        dt = np.dtype(TYPE_OF_CODE[dst_type])
        Z = self.dev.upload(np.zeros(x.size, dt))
        self.ops.convertTypes(self.dev.extra(), src_type, xp, x.size, dst_type, Z.ptr)
        out = Z.download(dt, x.size)
        self._finish(X, Z)
        return out

    # ---- elementwise ---------------------------------------------------------------------------
    def transform(self, op, x, x_info, z_info, extra=None, z=None):
        X = self._op(x, x_info)
        Z = self._op(np.zeros(_span(z_info), x.dtype) if z is None else z, z_info)
        E, e = self._up(extra, x.dtype)
        ptrs = self.dev.extra(x_info, z_info=z_info)
        D = None
        if op == 41 and extra is not None:
            # IsMax along dimensions: the CUDA convention carries them in extraPointers[15] (device int array) and
            # [18] (their count); extraParams only has to be non-null
            dims = [int(v) for v in np.asarray(extra)[1:1 + int(np.asarray(extra)[0])]]
            D, d = self._up(np.array(dims, np.int32))
            ptrs[15] = d
            ptrs[18] = len(dims)
        getattr(self.ops, "execTransform" + self._suffix(x))(ptrs, op, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, e)
        out = Z.get()
        self._finish(X, Z, E, D)
        return out

    def transform_inplace(self, op, x, x_info, extra=None):
        X = self._op(x, x_info)
        E, e = self._up(extra, x.dtype)
        getattr(self.ops, "execTransform" + self._suffix(x))(self.dev.extra(x_info, z_info=x_info), op, X.ptr, X.info_ptr,
                                                              X.ptr, X.info_ptr, e)
        out = X.get()
        self._finish(X, E)
        return out

    def transform_strided(self, op, x, xs, zs, extra, n, zsize=None):
        zsize = zsize if zsize is not None else max(1, (n - 1) * zs + 1)
        X, xp = self._up(x)
        Z, zp = self._up(np.zeros(zsize, x.dtype))
        E, e = self._up(extra, x.dtype)
        getattr(self.ops, "execTransform" + self._suffix(x))(self.dev.extra(), op, xp, int(xs), zp, int(zs), e, int(n))
        out = Z.download(x.dtype, zsize)
        self._finish(X, Z, E)
        return out

    def pairwise(self, op, x, x_info, y, y_info, z_info, extra=None):
        X, Y = self._op(x, x_info), self._op(y, y_info)
        Z = self._op(np.zeros(_span(z_info), x.dtype), z_info)
        E, e = self._up(extra, x.dtype)
        getattr(self.ops, "execPairwiseTransform" + self._suffix(x))(self.dev.extra(x_info, y_info, z_info), op, X.ptr,
                                                                      X.info_ptr, Y.ptr, Y.info_ptr, Z.ptr, Z.info_ptr, e)
        out = Z.get()
        self._finish(X, Y, Z, E)
        return out

    def scalar(self, op, x, x_info, z_info, scalar, extra=None):
        X = self._op(x, x_info)
        Z = self._op(np.zeros(_span(z_info), x.dtype), z_info)
        E, e = self._up(extra, x.dtype)
        getattr(self.ops, "execScalar" + self._suffix(x))(self.dev.extra(x_info, z_info=z_info), op, X.ptr, X.info_ptr, Z.ptr,
                                                           Z.info_ptr, float(scalar), e)
        out = Z.get()
        self._finish(X, Z, E)
        return out

    def scalar_strided(self, op, x, xs, zs, scalar, extra, n):
        zsize = max(1, (n - 1) * zs + 1)
        X, xp = self._up(x)
        Z, zp = self._up(np.zeros(zsize, x.dtype))
        E, e = self._up(extra, x.dtype)
        getattr(self.ops, "execScalar" + self._suffix(x))(self.dev.extra(), op, xp, int(xs), zp, int(zs), float(scalar), e, int(n))
        out = Z.download(x.dtype, zsize)
        self._finish(X, Z, E)
        return out

    def scalar_tad(self, op, x, x_info, scalars, extra, dims, pass_tads=True):
        X = self._op(x, x_info)
        Z = self._op(np.zeros(_span(x_info), x.dtype), x_info)
        S, sp = self._up(scalars, x.dtype)
        E, e = self._up(extra, x.dtype)
        D, d = self._up(np.array(list(dims), np.int32))
        tad = self.dev.tad(x_info, dims) if pass_tads else None
        getattr(self.ops, "execScalar" + self._suffix(x))(self.dev.extra(x_info, z_info=x_info, tad=tad, tad_z=tad), op, X.ptr,
                                                           X.info_ptr, Z.ptr, Z.info_ptr, sp, e, d, len(dims))
        out = Z.get()
        self._finish(X, Z, S, E, D)
        return out

    def pairwise_strided(self, op, x, xs, y, ys, zs, extra, n):
        zsize = max(1, (n - 1) * zs + 1)
        X, xp = self._up(x)
        Y, yp = self._up(y)
        Z, zp = self._up(np.zeros(zsize, x.dtype))
        E, e = self._up(extra, x.dtype)
        getattr(self.ops, "execPairwiseTransform" + self._suffix(x))(self.dev.extra(), op, xp, int(xs), yp, int(ys), zp,
                                                                      int(zs), e, int(n))
        out = Z.download(x.dtype, zsize)
        self._finish(X, Y, Z, E)
        return out

    def broadcast(self, op, x, x_info, y, y_info, z_info, dims, pass_tads=True):
        X, Y = self._op(x, x_info), self._op(y, y_info)
        Z = self._op(np.zeros(_span(z_info), x.dtype), z_info)
        D, d = self._up(np.array(list(dims), np.int32))
        tad = self.dev.tad(x_info, dims) if pass_tads else None
        tad_z = self.dev.tad(z_info, dims) if pass_tads else None
        getattr(self.ops, "execBroadcast" + self._suffix(x))(
            self.dev.extra(x_info, y_info, z_info, tad=tad, tad_z=tad_z), op, X.ptr, X.info_ptr, Y.ptr, Y.info_ptr,
            Z.ptr, Z.info_ptr, d, len(dims))
        out = Z.get()
        self._finish(X, Y, Z, D)
        return out

    # ---- reductions ----------------------------------------------------------------------------
    def _reduce_like(self, member, op, x, x_info, extra, dims, out_len, trailing=(), pass_tads=True):
        X = self._op(x, x_info)
        zi = _vec_info(out_len)
        Z = self._op(np.zeros(out_len, x.dtype), zi)
        E, e = self._up(extra, x.dtype)
        D, d = self._up(np.array(list(dims), np.int32))
        tad = self.dev.tad(x_info, dims) if (pass_tads and len(dims) < int(x_info[0])) else None
        getattr(self.ops, member + self._suffix(x))(self.dev.extra(x_info, z_info=zi, tad=tad), op, X.ptr, X.info_ptr, e,
                                                     Z.ptr, Z.info_ptr, d, len(dims), *trailing)
        out = Z.get()
        self._finish(X, Z, E, D)
        return out

    def reduce(self, op, x, x_info, extra, dims, out_len, pass_tads=True):
        return self._reduce_like("execReduce", op, x, x_info, extra, dims, out_len, pass_tads=pass_tads)

    def reduce3_scalar(self, op, x, x_info, y, y_info, extra=None):
        X, Y = self._op(x, x_info), self._op(y, y_info)
        E, e = self._up(extra, x.dtype)
        r = getattr(self.ops, "execReduce3Scalar" + self._suffix(x))(self.dev.extra(x_info, y_info), op, X.ptr, X.info_ptr, e,
                                                                    Y.ptr, Y.info_ptr)
        self._finish(X, Y, E)
        return x.dtype.type(r)

    def reduce3(self, op, x, x_info, y, y_info, extra, dims, out_len, tad_way=False, pass_tads=True):
        X, Y = self._op(x, x_info), self._op(y, y_info)
        zi = _vec_info(out_len)
        Z = self._op(np.zeros(out_len, x.dtype), zi)
        E, e = self._up(extra, x.dtype)
        D, d = self._up(np.array(list(dims), np.int32))
        tad = self.dev.tad(x_info, dims) if (pass_tads and len(dims) < int(x_info[0])) else None
        getattr(self.ops, "execReduce3" + self._suffix(x))(self.dev.extra(x_info, y_info, zi, tad=tad), op, X.ptr, X.info_ptr, e,
                                                            Y.ptr, Y.info_ptr, Z.ptr, Z.info_ptr, d, len(dims))
        out = Z.get()
        self._finish(X, Y, Z, E, D)
        return out

    def reduce3_all(self, op, x, x_info, y, y_info, extra, dims, out_len, pass_tads=False):
        """pass_tads: hand over what nd4j does - x's host TAD shapeInfo in extraPointers[9] and the device TAD tables of
        both operands as arguments - instead of leaving the library to build them from the (device) dimensions"""
        X, Y = self._op(x, x_info), self._op(y, y_info)
        zi = _vec_info(out_len)
        Z = self._op(np.zeros(out_len, x.dtype), zi)
        E, e = self._up(extra, x.dtype)
        D, d = self._up(np.array(list(dims), np.int32))
        tables = [None] * 4
        if pass_tads:
            ptrs = self.dev.extra(x_info, y_info, zi, tad=self.dev.tad(x_info, dims), tad_z=self.dev.tad(y_info, dims))
            tables = [ptrs[10], ptrs[11], ptrs[12], ptrs[13]]
            ptrs[12] = ptrs[13] = None  # the y tables travel as arguments, not in the slots of a result's TADs
        else:
            ptrs = self.dev.extra(x_info, y_info, zi)
        getattr(self.ops, "execReduce3All" + self._suffix(x))(ptrs, op, X.ptr, X.info_ptr, e, Y.ptr, Y.info_ptr, Z.ptr, Z.info_ptr, d,
                                                               len(dims), *tables)
        out = Z.get()
        self._finish(X, Y, Z, E, D)
        return out

    def indexreduce(self, op, x, x_info, extra, dims, out_len, pass_tads=True):
        return self._reduce_like("execIndexReduce", op, x, x_info, extra, dims, out_len, pass_tads=pass_tads)

    def summarystats(self, op, bias, x, x_info, dims, out_len, pass_tads=True):
        return self._reduce_like("execSummaryStats", op, x, x_info, None, dims, out_len, trailing=(int(bool(bias)),),
                                 pass_tads=pass_tads)

    def _scalar(self, member, op, x, x_info, extra, trailing=(), raw=False):
        X = self._op(x, x_info)
        E, e = self._up(extra, x.dtype)
        r = getattr(self.ops, member + self._suffix(x))(self.dev.extra(x_info), op, X.ptr, X.info_ptr, e, *trailing)
        self._finish(X, E)
        return float(r) if raw else x.dtype.type(r)

    def reduce_scalar(self, op, x, x_info, extra=None):
        return self._scalar("execReduceScalar", op, x, x_info, extra)

    def indexreduce_scalar(self, op, x, x_info, extra=None, raw=False):
        """raw: the value as the entry point returns it (a float also for half data) rather than cast to x's type"""
        return self._scalar("execIndexReduceScalar", op, x, x_info, extra, raw=raw)

    def summarystats_scalar(self, op, bias, x, x_info):
        return self._scalar("execSummaryStatsScalar", op, x, x_info, None, trailing=(int(bool(bias)),))

    def tad(self, x_info, dims):
        return self.dev.tad(x_info, dims)

    def rng(self, seed, size):
        return _GpuRng(self, seed, size)


class _GpuRng(object):
    def __init__(self, be, seed, size):
        self.be = be
        self.dev = be.dev
        self.ops = be.ops
        self.host = np.zeros(size, np.uint64)
        self.devbuf = self.dev.empty(size * 8)
        self.ptr = self.ops.initRandom(self.dev.extra(host_buffer=self.host.ctypes.data), seed, size, self.devbuf.ptr)

    @property
    def buffer(self):
        return self.host

    def elements(self, start, n):
        out = self.dev.empty(n * 8)
        self.ops.amd_rngDump(self.dev.extra(), self.ptr, int(start), int(n), out.ptr)
        r = out.download(np.uint64, n)
        out.free()
        return r

    def state(self):
        st = np.zeros(5, np.int64)
        self.ops.amd_rngState(self.ptr, st.ctypes.data)
        return tuple(int(v) for v in st)

    def rewind(self, n):
        # the boundary has no bare rewind: a Linspace fill of n elements advances the state by n
        if n > 0:
            self.random_z(4, n, [0, 1])

    def reseed(self, seed):
        self.ops.reSeedBuffer(self.dev.extra(), seed, self.ptr)

    def refresh(self, seed):
        self.ops.refreshBuffer(self.dev.extra(host_buffer=self.host.ctypes.data), seed, self.ptr)

    def _exec(self, suffix, *args):
        return getattr(self.ops, "execRandom" + suffix)(*args)

    def random_z(self, op, n_or_info, args, dtype=np.float32):
        info = _vec_info(n_or_info) if np.isscalar(n_or_info) else n_or_info
        dtype = np.dtype(dtype)
        Z = self.be._op(np.zeros(_span(info), dtype), info)
        A, a = self.be._up(np.asarray(args, dtype))
        self._exec(self.be._suffix(np.zeros(0, dtype)), self.dev.extra(), op, self.ptr, Z.ptr, Z.info_ptr, a)
        out = Z.get()
        self.be._finish(Z, A)
        return out

    def random_xz(self, op, x, args, inplace=True, info=None):
        info = _vec_info(x.size) if info is None else info
        X = self.be._op(x, info)
        A, a = self.be._up(np.asarray(args, x.dtype))
        if inplace:
            self._exec(self.be._suffix(x), self.dev.extra(), op, self.ptr, X.ptr, X.info_ptr, X.ptr, X.info_ptr, a)
            out = X.get()
            self.be._finish(X, A)
            return out
        Z = self.be._op(np.zeros_like(x), info)
        self._exec(self.be._suffix(x), self.dev.extra(), op, self.ptr, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, a)
        out = Z.get()
        self.be._finish(X, Z, A)
        return out

    def random_xyz(self, op, x, y, args, mode="separate", n=None, dtype=np.float32):
        dtype = np.dtype(dtype)
        A, a = self.be._up(np.asarray(args, dtype))
        if mode == "inplace_all":
            info = _vec_info(n)
            Z = self.be._op(np.zeros(n, dtype), info)
            self._exec(self.be._suffix(np.zeros(0, dtype)), self.dev.extra(), op, self.ptr, Z.ptr, Z.info_ptr, Z.ptr,
                       Z.info_ptr, Z.ptr, Z.info_ptr, a)
            out = Z.get()
            self.be._finish(Z, A)
            return out
        X = self.be._op(x, _vec_info(x.size))
        Y = self.be._op(y, _vec_info(y.size))
        Z = self.be._op(np.zeros_like(x), _vec_info(x.size))
        self._exec(self.be._suffix(x), self.dev.extra(), op, self.ptr, X.ptr, X.info_ptr, Y.ptr, Y.info_ptr, Z.ptr,
                   Z.info_ptr, a)
        out = Z.get()
        self.be._finish(X, Y, Z, A)
        return out

    def choice(self, values, v_info, probs, p_info, z_info):
        X, Y = self.be._op(values, v_info), self.be._op(probs, p_info)
        Z = self.be._op(np.zeros(_span(z_info), values.dtype), z_info)
        A, a = self.be._up(np.zeros(1, values.dtype))
        try:
            self._exec(self.be._suffix(values), self.dev.extra(z_info), 5, self.ptr, X.ptr, X.info_ptr, Y.ptr,
                       Y.info_ptr, Z.ptr, Z.info_ptr, a)
            out = Z.get()
        finally:
            self.be._finish(X, Y, Z, A)
        return out

    def destroy(self):
        self.dev.sync()
        self.ops.destroyRandom(self.ptr)
        self.devbuf.free()
