"""The benchmark / full-size parity workloads: one builder per configuration of the headline benchmark
(transform, pairwise + broadcast, reductions, summary statistics + softmax-style chain, random).

A builder generates the synthetic inputs on the host (seeded numpy generators), keeps them resident on the
device, prepares shapeInfo / TAD tables / extraPointers once (as nd4j's executioner caches them) and returns
``Case`` objects.  ``case.gpu()`` enqueues exactly one call of the library on the device stream;
``case.cpu(lib)`` runs the same call on a CPU checker from tests/cpu_ref.py and returns its output (used by
bench.py's CPU baseline and by the tests only).  ``case.bytes`` is the algorithmic traffic of one call: every input element read once,
every output element written once.
"""
import numpy as np

from . import harness

F32 = np.float32

# opNums (reference: include/loops/legacy_ops.h)
T_EXP, T_TANH, T_TANH_DERIVATIVE = 3, 15, 23
T_SOFTMAX, T_LOGSOFTMAX, T_ISMAX = 38, 40, 41
P_ADD, P_MUL = 0, 6
S_MUL = 2  # scalar family
B_ADD, B_SUB, B_DIV = 0, 1, 3
R_MEAN, R_SUM, R_MAX = 0, 1, 3
I_MAX = 0
S_VAR, S_STD = 0, 1
RND_UNIFORM, RND_DROPOUT, RND_GAUSSIAN = 0, 1, 6


ROTATE_BYTES = 3 << 29  # device copies of the operands are made until they span 1.5 GiB


class Case(object):
    """One call of the library.  The operands exist in several device copies ("sets") and ``gpu(k)`` runs the
    call on set ``k % sets``: a timing loop that passes its iteration counter never finds its operands in the
    256 MiB last-level cache left there by the previous iteration, so what it measures is HBM traffic."""

    def __init__(self, name, family, elements, nbytes, gpu, cpu, contiguous, result=None):
        self.name = name
        self.family = family
        self.elements = int(elements)
        self.bytes = int(nbytes)
        self._gpu = [gpu]
        self._result = [result]
        self.cpu = cpu
        self.contiguous = contiguous
        self.note = None  # printed beside the case by the benchmark
        self.bound = "hbm"  # what limits the case: "hbm", "valu" when instruction issue does, "mfma" (with `flops` set) for the matrix unit
        self.cpu_once = False  # the benchmark times a single cold CPU pass of this case

    @property
    def sets(self):
        return len(self._gpu)

    def gpu(self, k=0):
        self._gpu[k % len(self._gpu)]()

    def result(self, k=0):
        """numpy array of what the last gpu(k) call wrote"""
        return self._result[k % len(self._result)]()

    def add_set(self, other):
        self._gpu += other._gpu
        self._result += other._result


class Workload(object):
    """Cases of one configuration plus the host copies of their inputs."""

    def __init__(self, dev, name):
        self.dev = dev
        self.name = name
        self.cases = []
        self.host = {}
        self._operands = []

    def operand(self, data, info):
        o = harness.Operand(self.dev, np.ascontiguousarray(data), info)
        self._operands.append(o)
        return o

    def raw(self, array):
        d = self.dev.upload(np.ascontiguousarray(array))
        self._operands.append(d)
        return d

    def case(self, name):
        for c in self.cases:
            if c.name == name:
                return c
        raise KeyError(name)

    def free(self):
        self.dev.sync()
        for o in self._operands:
            o.free()
        self._operands = []
        self.dev.release()


def _vec(n):
    return harness.shape_info([1, int(n)])


def _replicated(dev, name, set_bytes, host, device_set, copies=None):
    """Builds a Workload from ``device_set(w) -> [Case]``, called once per device copy of the operands."""
    w = Workload(dev, name)
    w.host.update(host)
    if copies is None:
        copies = max(2, -(-ROTATE_BYTES // int(set_bytes)))
    w.cases = device_set(w)
    for _ in range(copies - 1):
        for c, extra in zip(w.cases, device_set(w)):
            c.add_set(extra)
    w.copies = copies
    return w


def _normal(rs, n, dtype):
    return rs.standard_normal(n, dtype=F32).astype(dtype, copy=False)


def _uniform(rs, n, lo, hi, dtype=F32):
    return (rs.random(n, dtype=F32) * F32(hi - lo) + F32(lo)).astype(dtype, copy=False)


def _suffix(dtype):
    return harness.SUFFIX_OF[np.dtype(dtype)]


# ---- configs[0]: tanh over 2^24 ------------------------------------------------------------------------
def transform_tanh(dev, n=1 << 24, seed=42, copies=None):
    x = _uniform(np.random.default_rng(seed), n, -4, 4)
    xi = _vec(n)
    zc = np.zeros(n, F32)
    ops = dev.ops

    def device_set(w):
        X, Z = w.operand(x, xi), w.operand(np.zeros(n, F32), xi)
        ex = dev.extra(xi, z_info=xi)
        cases = [Case("transform_tanh", "transform", n, 8 * n,
                      lambda: ops.execTransformFloat(ex, T_TANH, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, None),
                      lambda lib: (lib.transform(T_TANH, x, xi, zc, xi, None), zc)[1], True, Z.get),
                 # 1 - tanh^2 keeps the C library's tanhf, replayed bit for bit, for every element (near saturation one
                 # ULP of tanh is a multiple of the result): what tanh itself cost while it did the same
                 Case("transform_tanh_derivative", "transform", n, 8 * n,
                      lambda: ops.execTransformFloat(ex, T_TANH_DERIVATIVE, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, None),
                      lambda lib: (lib.transform(T_TANH_DERIVATIVE, x, xi, zc, xi, None), zc)[1], True, Z.get)]
        cases[1].bound = "valu"
        return cases

    return _replicated(dev, "transform tanh fp32 1-D 2^%d" % int(np.log2(n)), 8 * n, dict(x=x, xi=xi, z_cpu=zc),
                       device_set, copies)


# ---- configs[1]: pairwise add / multiply and broadcast add of a row ----------------------------------
def pairwise_broadcast(dev, rows=65536, cols=1024, seed=7, dtype=F32, copies=None):
    dtype = np.dtype(dtype)
    rs = np.random.default_rng(seed)
    n = rows * cols
    x, y = _normal(rs, n, dtype), _normal(rs, n, dtype)
    bias = _uniform(rs, cols, -1, 1, dtype)
    xi, bi = harness.shape_info([rows, cols]), _vec(cols)
    ops, suf, sz = dev.ops, _suffix(dtype), dtype.itemsize
    pw, bc, scl = getattr(ops, "execPairwiseTransform" + suf), getattr(ops, "execBroadcast" + suf), getattr(ops, "execScalar" + suf)
    tad = dev.tad(xi, [1])
    zc = np.zeros(n, dtype)
    tag = "" if dtype == F32 else "_" + dtype.name

    def device_set(w):
        X, Y, Z, B = w.operand(x, xi), w.operand(y, xi), w.operand(np.zeros(n, dtype), xi), w.operand(bias, bi)
        ex_p = dev.extra(xi, xi, xi)
        ex_b = dev.extra(xi, bi, xi, tad=tad, tad_z=tad)
        D = w.raw(np.array([1], np.int32))

        def mk_pw(op):
            return lambda: pw(ex_p, op, X.ptr, X.info_ptr, Y.ptr, Y.info_ptr, Z.ptr, Z.info_ptr, None)

        def gpu_bc():
            bc(ex_b, B_ADD, X.ptr, X.info_ptr, B.ptr, B.info_ptr, Z.ptr, Z.info_ptr, D.ptr, 1)

        ex_s = dev.extra(xi, z_info=xi)
        extra_cases = [Case("scalar_multiply" + tag, "scalar", n, 2 * sz * n,
                            lambda: scl(ex_s, S_MUL, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, 1.5, None),
                            lambda lib: (lib.scalar(S_MUL, x, xi, zc, xi, 1.5, None), zc)[1], True, Z.get)]
        return extra_cases[:0] + [Case("pairwise_add" + tag, "pairwise", n, 3 * sz * n, mk_pw(P_ADD),
                     lambda lib: (lib.pairwise(P_ADD, x, xi, y, xi, zc, xi, None), zc)[1], True, Z.get),
                Case("pairwise_multiply" + tag, "pairwise", n, 3 * sz * n, mk_pw(P_MUL),
                     lambda lib: (lib.pairwise(P_MUL, x, xi, y, xi, zc, xi, None), zc)[1], True, Z.get),
                Case("broadcast_add_row" + tag, "broadcast", n, 2 * sz * n + sz * cols, gpu_bc,
                     lambda lib: (lib.broadcast(B_ADD, x, xi, bias, bi, zc, xi, [1]), zc)[1], True, Z.get)] + extra_cases

    return _replicated(dev, "pairwise add+multiply, broadcast add row; %s [%d,%d] c-order" % (dtype.name, rows, cols),
                       3 * sz * n, dict(x=x, y=y, bias=bias, xi=xi, bi=bi, z_cpu=zc), device_set, copies)


# ---- configs[2]: reduce sum / max / mean and argmax along rows, columns and over everything ----------
def reductions(dev, rows=16384, cols=4096, seed=11, copies=None):
    n = rows * cols
    x = _normal(np.random.default_rng(seed), n, F32)
    xi = harness.shape_info([rows, cols])
    ops = dev.ops
    tads = {1: dev.tad(xi, [1]), 0: dev.tad(xi, [0])}
    host_out = {(dim, out_len): np.zeros(out_len, F32) for dim, out_len in ((1, rows), (0, cols))}

    def device_set(w):
        cases = []
        X = w.operand(x, xi)
        scalar_out = {}
        for dim, out_len in ((1, rows), (0, cols)):
            zi = _vec(out_len)
            Z = w.operand(np.zeros(out_len, F32), zi)
            D = w.raw(np.array([dim], np.int32))
            ex = dev.extra(xi, z_info=zi, tad=tads[dim])
            zc = host_out[(dim, out_len)]
            for fam, member, cpu_name, op, opname in (("reduce", ops.execReduceFloat, "reduce", R_SUM, "sum"),
                                                      ("reduce", ops.execReduceFloat, "reduce", R_MAX, "max"),
                                                      ("reduce", ops.execReduceFloat, "reduce", R_MEAN, "mean"),
                                                      ("indexreduce", ops.execIndexReduceFloat, "indexreduce", I_MAX, "argmax")):
                def gpu(member=member, op=op, Z=Z, D=D, ex=ex):
                    member(ex, op, X.ptr, X.info_ptr, None, Z.ptr, Z.info_ptr, D.ptr, 1)

                def cpu(lib, cpu_name=cpu_name, op=op, zc=zc, zi=zi, dim=dim):
                    getattr(lib, cpu_name)(op, x, xi, None, zc, zi, [dim])
                    return zc

                cases.append(Case("%s_dim%d" % (opname, dim), fam, n, 4 * n + 4 * out_len, gpu, cpu, dim == 1, Z.get))
        ex_s = dev.extra(xi)
        for fam, member, cpu_name, op, opname in (("reduce", ops.execReduceScalarFloat, "reduce_scalar", R_SUM, "sum"),
                                                  ("reduce", ops.execReduceScalarFloat, "reduce_scalar", R_MAX, "max"),
                                                  ("reduce", ops.execReduceScalarFloat, "reduce_scalar", R_MEAN, "mean"),
                                                  ("indexreduce", ops.execIndexReduceScalarFloat, "indexreduce_scalar", I_MAX, "argmax")):
            def gpu(member=member, op=op, opname=opname):
                scalar_out[opname] = member(ex_s, op, X.ptr, X.info_ptr, None)

            def cpu(lib, cpu_name=cpu_name, op=op):
                return getattr(lib, cpu_name)(op, x, xi, None)

            cases.append(Case("%s_full" % opname, fam, n, 4 * n + 4, gpu, cpu, True,
                              lambda opname=opname: np.array([scalar_out[opname]], F32)))
            cases[-1].note = "returns the scalar to the host: launch and hand-over latency included"
        # the same whole-array reductions with the result left on the device (the array-result overload, all
        # dimensions named): nothing waits for the call, so successive calls queue up as the per-dimension ones do
        z1 = _vec(1)
        Z1 = w.operand(np.zeros(1, F32), z1)
        ex_d = dev.extra(xi, z_info=z1)
        D01 = w.raw(np.array([0, 1], np.int32))
        for fam, member, cpu_name, op, opname in (("reduce", ops.execReduceFloat, "reduce_scalar", R_SUM, "sum"),
                                                  ("indexreduce", ops.execIndexReduceFloat, "indexreduce_scalar", I_MAX, "argmax")):
            def gpu(member=member, op=op):
                member(ex_d, op, X.ptr, X.info_ptr, None, Z1.ptr, Z1.info_ptr, D01.ptr, 2)

            def cpu(lib, cpu_name=cpu_name, op=op):
                return getattr(lib, cpu_name)(op, x, xi, None)

            cases.append(Case("%s_full_to_device" % opname, fam, n, 4 * n + 4, gpu, cpu, True, Z1.get))
        return cases

    return _replicated(dev, "reduce sum/max/mean + argmax; fp32 [%d,%d] c-order; dim 1, dim 0, full" % (rows, cols),
                       4 * n, dict(x=x, xi=xi), device_set, copies)


# ---- reduce3 family on the configs[2] shape: dot over everything, Euclidean and cosine per row ----------
def reduce3_pairs(dev, rows=16384, cols=4096, seed=12, copies=None):
    n = rows * cols
    rs = np.random.default_rng(seed)
    x, y = _normal(rs, n, F32), _normal(rs, n, F32)
    xi = harness.shape_info([rows, cols])
    zi = _vec(rows)
    ops = dev.ops
    tad = dev.tad(xi, [1])
    zc = np.zeros(rows, F32)

    def device_set(w):
        X, Y = w.operand(x, xi), w.operand(y, xi)
        Z = w.operand(np.zeros(rows, F32), zi)
        D = w.raw(np.array([1], np.int32))
        ex = dev.extra(xi, xi, zi, tad=tad)
        ex_s = dev.extra(xi, xi)
        out = {}
        cases = []
        for op, opname in ((1, "euclidean"), (2, "cosine")):
            def gpu(op=op):
                ops.execReduce3Float(ex, op, X.ptr, X.info_ptr, None, Y.ptr, Y.info_ptr, Z.ptr, Z.info_ptr, D.ptr, 1)

            def cpu(lib, op=op):
                lib.reduce3(op, x, xi, y, xi, zc, zi, [1], None)
                return zc

            cases.append(Case("%s_dim1" % opname, "reduce3", n, 8 * n + 4 * rows, gpu, cpu, True, Z.get))

        def gpu_dot():
            out["dot"] = ops.execReduce3ScalarFloat(ex_s, 3, X.ptr, X.info_ptr, None, Y.ptr, Y.info_ptr)

        cases.append(Case("dot_full", "reduce3", n, 8 * n + 4, gpu_dot, lambda lib: lib.reduce3_scalar(3, x, xi, y, xi, None), True,
                          lambda: np.array([out["dot"]], F32)))
        cases[-1].note = "returns the scalar to the host: launch and hand-over latency included"
        # every row of a [2048,1024] piece of x (its first 2 Mi elements) against every row of the same piece of y: 2048 x 2048
        # dot products.
        # Not a streaming case: each operand is read from HBM once and reused from LDS (its "bytes" are the 16 MiB of
        # operands and the 16 MiB of results): a matrix product, bound by the matrix unit; `elements` counts the pairs.
        ar, al = min(2048, rows), min(1024, cols)
        ai, azi = harness.shape_info([ar, al]), harness.shape_info([ar, ar])
        ZA = w.operand(np.zeros(ar * ar, F32), azi)
        ex_a = dev.extra(ai, ai, azi, tad=dev.tad(ai, [1]))  # host TAD shapeInfo in slot 9, device tables in 10 / 11
        AI = w.raw(np.ascontiguousarray(ai, dtype=np.int64))
        za = np.zeros(ar * ar, F32)
        case = Case("dot_all_pairs", "reduce3", ar * ar * al, 8 * ar * al + 4 * ar * ar,
                    lambda: ops.execReduce3AllFloat(ex_a, 3, X.ptr, AI.ptr, None, Y.ptr, AI.ptr, ZA.ptr, ZA.info_ptr, D.ptr, 1, ex_a[10],
                                                    ex_a[11], ex_a[10], ex_a[11]),
                    lambda lib: (lib.reduce3_all(3, x[:ar * al], ai, y[:ar * al], ai, za, azi, [1], None), za)[1], True, ZA.get)
        case.note = "compute-bound: %.0f G pairs, fp32 on the matrix unit (v_mfma_f32_32x32x2_f32)" % (ar * ar * al / 1e9)
        case.bound = "mfma"
        case.flops = 2 * ar * ar * al  # a multiplication and an addition per pair
        case.cpu_once = True  # one pass of the reference takes seconds
        cases.append(case)
        return cases

    return _replicated(dev, "reduce3 euclidean/cosine per row + dot; fp32 [%d,%d] c-order" % (rows, cols), 8 * n,
                       dict(x=x, y=y, xi=xi), device_set, copies)


# ---- configs[3]: summary statistics and a softmax-style chain on an f-order matrix ---------------------
def stats_softmax(dev, rows=32768, cols=2048, seed=23, copies=None):
    n = rows * cols
    x = _uniform(np.random.default_rng(seed), n, -10, 10)  # memory order of the f-order matrix
    xi = harness.shape_info([rows, cols], "f")
    ops = dev.ops
    tad1, tad0 = dev.tad(xi, [1]), dev.tad(xi, [0])
    ri = _vec(rows)
    ci = harness.shape_info([rows, 1])
    xci = harness.shape_info([rows, cols], "c")
    mc, sc, tc = np.zeros(rows, F32), np.zeros(rows, F32), np.zeros(n, F32)
    host_out = {(dim, out_len): np.zeros(out_len, F32) for dim, out_len in ((1, rows), (0, cols))}

    def device_set(w):
        cases = []
        X = w.operand(x, xi)
        for dim, out_len, tad in ((1, rows, tad1), (0, cols, tad0)):
            zi = _vec(out_len)
            Z = w.operand(np.zeros(out_len, F32), zi)
            D = w.raw(np.array([dim], np.int32))
            ex = dev.extra(xi, z_info=zi, tad=tad)
            zc = host_out[(dim, out_len)]
            for op, opname in ((S_VAR, "variance"), (S_STD, "std")):
                def gpu(op=op, Z=Z, D=D, ex=ex):
                    ops.execSummaryStatsFloat(ex, op, X.ptr, X.info_ptr, None, Z.ptr, Z.info_ptr, D.ptr, 1, 1)

                def cpu(lib, op=op, zc=zc, zi=zi, dim=dim):
                    lib.summarystats(op, 1, x, xi, zc, zi, [dim])
                    return zc

                # dim 0 TADs are the contiguous columns of the f-order matrix, dim 1 TADs have stride `rows`
                cases.append(Case("%s_dim%d" % (opname, dim), "summarystats", n, 4 * n + 4 * out_len, gpu, cpu, dim == 0, Z.get))

        # softmax along dimension 1 as five calls: m = max(x, 1); t = x - m; t = exp(t); s = sum(t, 1); t = t / s
        M, S, T = w.operand(np.zeros(rows, F32), ri), w.operand(np.zeros(rows, F32), ri), w.operand(np.zeros(n, F32), xi)
        D1, D0 = w.raw(np.array([1], np.int32)), w.raw(np.array([0], np.int32))
        ex_r = dev.extra(xi, z_info=ri, tad=tad1)
        ex_b = dev.extra(xi, ci, xi, tad=tad0, tad_z=tad0)
        ex_t = dev.extra(xi, z_info=xi)
        steps = [
            ("softmax_1_max", "reduce", 4 * n + 4 * rows,
             lambda: ops.execReduceFloat(ex_r, R_MAX, X.ptr, X.info_ptr, None, M.ptr, M.info_ptr, D1.ptr, 1),
             lambda lib: (lib.reduce(R_MAX, x, xi, None, mc, ri, [1]), mc)[1]),
            ("softmax_2_subtract", "broadcast", 8 * n + 4 * rows,
             lambda: ops.execBroadcastFloat(ex_b, B_SUB, X.ptr, X.info_ptr, M.ptr, M.info_ptr, T.ptr, T.info_ptr, D0.ptr, 1),
             lambda lib: (lib.broadcast(B_SUB, x, xi, mc, ci, tc, xi, [0]), tc)[1]),
            ("softmax_3_exp", "transform", 8 * n,
             lambda: ops.execTransformFloat(ex_t, T_EXP, T.ptr, T.info_ptr, T.ptr, T.info_ptr, None),
             lambda lib: (lib.transform(T_EXP, tc, xi, tc, xi, None), tc)[1]),
            ("softmax_4_sum", "reduce", 4 * n + 4 * rows,
             lambda: ops.execReduceFloat(ex_r, R_SUM, T.ptr, T.info_ptr, None, S.ptr, S.info_ptr, D1.ptr, 1),
             lambda lib: (lib.reduce(R_SUM, tc, xi, None, sc, ri, [1]), sc)[1]),
            ("softmax_5_divide", "broadcast", 8 * n + 4 * rows,
             lambda: ops.execBroadcastFloat(ex_b, B_DIV, T.ptr, T.info_ptr, S.ptr, S.info_ptr, T.ptr, T.info_ptr, D0.ptr, 1),
             lambda lib: (lib.broadcast(B_DIV, tc, xi, sc, ci, tc, xi, [0]), tc)[1]),
        ]
        for name, fam, nbytes, gpu, cpu in steps:
            cases.append(Case(name, fam, n, nbytes, gpu, cpu, False, T.get))

        def chain_gpu():
            for st in steps:
                st[3]()

        def chain_cpu(lib):
            for st in steps:
                st[4](lib)
            return tc

        cases.append(Case("softmax_chain", "chain", n, sum(st[2] for st in steps), chain_gpu, chain_cpu, False, T.get))

        # the same softmax as ONE call (transform opNum 38), on the f-order matrix and on the same memory read as a
        # c-order [rows, cols] matrix (rows contiguous); IsMax over the whole array and along dimension 1
        XCI = w.raw(np.ascontiguousarray(xci, dtype=np.int64))
        ex_c = dev.extra(xci, z_info=xci)
        cases.append(Case("softmax_fused_forder", "special", n, 8 * n,
                          lambda: ops.execTransformFloat(ex_t, T_SOFTMAX, X.ptr, X.info_ptr, T.ptr, T.info_ptr, None),
                          lambda lib: (lib.transform(T_SOFTMAX, x, xi, tc, xi, None), tc)[1], False, T.get))
        # yardstick: a plain copy of the same matrix in the fused f-order kernel's tiles and block order (no arithmetic, no
        # exchange between blocks) - what its access pattern, 256-byte pieces of columns 128 KiB apart, costs by itself
        cases.append(Case("yardstick_copy_forder_tiles", "yardstick", n, 8 * n,
                          lambda: ops.amd_forderTileCopy(ex_t, T.ptr, X.ptr, rows, cols),
                          None, False, T.get))
        cases[-1].note = "not an op: the fused f-order softmax's memory accesses without its arithmetic"
        cases.append(Case("softmax_fused_corder", "special", n, 8 * n,
                          lambda: ops.execTransformFloat(ex_c, T_SOFTMAX, X.ptr, XCI.ptr, T.ptr, XCI.ptr, None),
                          lambda lib: (lib.transform(T_SOFTMAX, x, xci, tc, xci, None), tc)[1], True, T.get))
        cases.append(Case("logsoftmax_fused_corder", "special", n, 8 * n,
                          lambda: ops.execTransformFloat(ex_c, T_LOGSOFTMAX, X.ptr, XCI.ptr, T.ptr, XCI.ptr, None),
                          lambda lib: (lib.transform(T_LOGSOFTMAX, x, xci, tc, xci, None), tc)[1], True, T.get))
        # few long rows (the same memory as [rows / 64, cols * 64]): row maxima and sums come from the sliced reductions
        xli = harness.shape_info([rows // 64, cols * 64], "c")
        XLI = w.raw(np.ascontiguousarray(xli, dtype=np.int64))
        ex_l = dev.extra(xli, z_info=xli)
        cases.append(Case("softmax_fused_long_rows", "special", n, 8 * n,
                          lambda: ops.execTransformFloat(ex_l, T_SOFTMAX, X.ptr, XLI.ptr, T.ptr, XLI.ptr, None),
                          lambda lib: (lib.transform(T_SOFTMAX, x, xli, tc, xli, None), tc)[1], True, T.get))
        cases.append(Case("ismax_whole", "special", n, 8 * n,
                          lambda: ops.execTransformFloat(ex_c, T_ISMAX, X.ptr, XCI.ptr, T.ptr, XCI.ptr, None),
                          lambda lib: (lib.transform(T_ISMAX, x, xci, tc, xci, None), tc)[1], True, T.get))
        DM = w.raw(np.array([1], np.int32))
        EP = w.raw(np.array([1, 1], F32))
        ex_m = dev.extra(xci, z_info=xci, tad=dev.tad(xci, [1]))  # TAD tables in slots 9-11, as nd4j passes them
        ex_m[15] = DM.ptr
        ex_m[18] = 1
        ismax_params = np.array([1, 1], F32)
        cases.append(Case("ismax_dim1", "special", n, 8 * n,
                          lambda: ops.execTransformFloat(ex_m, T_ISMAX, X.ptr, XCI.ptr, T.ptr, XCI.ptr, EP.ptr),
                          lambda lib: (lib.transform(T_ISMAX, x, xci, tc, xci, ismax_params), tc)[1], True, T.get))
        return cases

    return _replicated(dev, "summary stats var/std + softmax-style chain; fp32 [%d,%d] f-order" % (rows, cols), 8 * n,
                       dict(x=x, xi=xi, softmax_cpu=tc), device_set, copies)


# ---- general views: multi-dimensional TADs, broadcasts over several dimensions, padded views --------------------------
def general_views(dev, seed=61, copies=None):
    """What nd4j's everyday multi-dimensional calls look like to the loops: TADs over several dimensions (their
    shapeInfo carries no element-wise stride, whatever their layout), broadcasts of a sub-array, and views with a row
    pitch.  A batch-norm style sum / variance over dimensions {0,2,3} of an NCHW array [128,128,56,56]; argmax over
    dimensions {1,2} of [4096,128,128]; add of a [56,56] plane along dimensions {2,3} of the NCHW array and of a
    [256,256] matrix along dimensions {0,2} of [256,1024,256]; pairwise add and exp on a [65536,1024] view whose rows
    are 1032 elements apart."""
    rs = np.random.default_rng(seed)
    ops = dev.ops
    nchw, cube, slab = [128, 128, 56, 56], [4096, 128, 128], [256, 1024, 256]
    n1, n2, n3 = int(np.prod(nchw)), int(np.prod(cube)), int(np.prod(slab))
    x1, x2, x3 = _normal(rs, n1, F32), _normal(rs, n2, F32), _normal(rs, n3, F32)
    i1, i2, i3 = harness.shape_info(nchw), harness.shape_info(cube), harness.shape_info(slab)
    plane, mat = _uniform(rs, 56 * 56, -1, 1), _uniform(rs, 256 * 256, -1, 1)
    pi, mi = harness.shape_info([56, 56]), harness.shape_info([256, 256])
    rows, cols, pitch = 65536, 1024, 1032
    vi = harness.shape_info([rows, cols], strides=[pitch, 1])
    nv, span = rows * cols, harness.span_of(vi)
    xv, yv = _normal(rs, span, F32), _normal(rs, span, F32)
    tad1_023, tad1_23 = dev.tad(i1, [0, 2, 3]), dev.tad(i1, [2, 3])
    tad2_12, tad3_02 = dev.tad(i2, [1, 2]), dev.tad(i3, [0, 2])
    bias_v, bvi, tad_v = _uniform(rs, cols, -1, 1), _vec(cols), dev.tad(vi, [1])
    tad1_02 = dev.tad(i1, [0, 2])
    cw_out, ocw = _vec(nchw[1] * nchw[3]), np.zeros(nchw[1] * nchw[3], F32)
    c_out, r_out = _vec(nchw[1]), _vec(cube[0])
    zc1, zc2, zc3 = np.zeros(n1, F32), np.zeros(n3, F32), np.zeros(span, F32)
    oc1, oc2 = np.zeros(nchw[1], F32), np.zeros(cube[0], F32)

    def device_set(w):
        cases = []
        X1, Z1 = w.operand(x1, i1), w.operand(np.zeros(n1, F32), i1)
        C = w.operand(np.zeros(nchw[1], F32), c_out)
        D023, D23 = w.raw(np.array([0, 2, 3], np.int32)), w.raw(np.array([2, 3], np.int32))
        ex = dev.extra(i1, z_info=c_out, tad=tad1_023)
        cases.append(Case("sum_nchw_dims023", "reduce", n1, 4 * n1 + 4 * nchw[1],
                          lambda: ops.execReduceFloat(ex, R_SUM, X1.ptr, X1.info_ptr, None, C.ptr, C.info_ptr, D023.ptr, 3),
                          lambda lib: (lib.reduce(R_SUM, x1, i1, None, oc1, c_out, [0, 2, 3]), oc1)[1], False, C.get))
        cases.append(Case("variance_nchw_dims023", "summarystats", n1, 4 * n1 + 4 * nchw[1],
                          lambda: ops.execSummaryStatsFloat(ex, S_VAR, X1.ptr, X1.info_ptr, None, C.ptr, C.info_ptr, D023.ptr, 3, 1),
                          lambda lib: (lib.summarystats(S_VAR, 1, x1, i1, oc1, c_out, [0, 2, 3]), oc1)[1], False, C.get))
        # dimensions {0, 2}: the TADs' innermost dimension is strided (56 elements apart), neighbouring TADs are neighbours
        CW = w.operand(np.zeros(nchw[1] * nchw[3], F32), cw_out)
        D02n = w.raw(np.array([0, 2], np.int32))
        ex02 = dev.extra(i1, z_info=cw_out, tad=tad1_02)
        cases.append(Case("sum_nchw_dims02", "reduce", n1, 4 * n1 + 4 * nchw[1] * nchw[3],
                          lambda: ops.execReduceFloat(ex02, R_SUM, X1.ptr, X1.info_ptr, None, CW.ptr, CW.info_ptr, D02n.ptr, 2),
                          lambda lib: (lib.reduce(R_SUM, x1, i1, None, ocw, cw_out, [0, 2]), ocw)[1], False, CW.get))
        P = w.operand(plane, pi)
        ex_b = dev.extra(i1, pi, i1, tad=tad1_23, tad_z=tad1_23)
        cases.append(Case("broadcast_add_nchw_dims23", "broadcast", n1, 8 * n1 + 4 * plane.size,
                          lambda: ops.execBroadcastFloat(ex_b, B_ADD, X1.ptr, X1.info_ptr, P.ptr, P.info_ptr, Z1.ptr, Z1.info_ptr, D23.ptr, 2),
                          lambda lib: (lib.broadcast(B_ADD, x1, i1, plane, pi, zc1, i1, [2, 3]), zc1)[1], False, Z1.get))
        X2 = w.operand(x2, i2)
        R = w.operand(np.zeros(cube[0], F32), r_out)
        D12 = w.raw(np.array([1, 2], np.int32))
        ex2 = dev.extra(i2, z_info=r_out, tad=tad2_12)
        cases.append(Case("argmax_cube_dims12", "indexreduce", n2, 4 * n2 + 4 * cube[0],
                          lambda: ops.execIndexReduceFloat(ex2, I_MAX, X2.ptr, X2.info_ptr, None, R.ptr, R.info_ptr, D12.ptr, 2),
                          lambda lib: (lib.indexreduce(I_MAX, x2, i2, None, oc2, r_out, [1, 2]), oc2)[1], False, R.get))
        X3, Z3 = w.operand(x3, i3), w.operand(np.zeros(n3, F32), i3)
        M = w.operand(mat, mi)
        D02 = w.raw(np.array([0, 2], np.int32))
        ex3 = dev.extra(i3, mi, i3, tad=tad3_02, tad_z=tad3_02)
        cases.append(Case("broadcast_add_slab_dims02", "broadcast", n3, 8 * n3 + 4 * mat.size,
                          lambda: ops.execBroadcastFloat(ex3, B_ADD, X3.ptr, X3.info_ptr, M.ptr, M.info_ptr, Z3.ptr, Z3.info_ptr, D02.ptr, 2),
                          lambda lib: (lib.broadcast(B_ADD, x3, i3, mat, mi, zc2, i3, [0, 2]), zc2)[1], False, Z3.get))
        XV, YV, ZV = w.operand(xv, vi), w.operand(yv, vi), w.operand(np.zeros(span, F32), vi)
        exv = dev.extra(vi, vi, vi)
        cases.append(Case("pairwise_add_padded_rows", "pairwise", nv, 12 * nv,
                          lambda: ops.execPairwiseTransformFloat(exv, P_ADD, XV.ptr, XV.info_ptr, YV.ptr, YV.info_ptr, ZV.ptr, ZV.info_ptr, None),
                          lambda lib: (lib.pairwise(P_ADD, xv, vi, yv, vi, zc3, vi, None), zc3)[1], False, ZV.get))
        BV = w.operand(bias_v, bvi)
        DV = w.raw(np.array([1], np.int32))
        exbv = dev.extra(vi, bvi, vi, tad=tad_v, tad_z=tad_v)
        cases.append(Case("broadcast_add_row_padded_rows", "broadcast", nv, 8 * nv + 4 * cols,
                          lambda: ops.execBroadcastFloat(exbv, B_ADD, XV.ptr, XV.info_ptr, BV.ptr, BV.info_ptr, ZV.ptr, ZV.info_ptr, DV.ptr, 1),
                          lambda lib: (lib.broadcast(B_ADD, xv, vi, bias_v, bvi, zc3, vi, [1]), zc3)[1], False, ZV.get))
        cases.append(Case("transform_exp_padded_rows", "transform", nv, 8 * nv,
                          lambda: ops.execTransformFloat(exv, T_EXP, XV.ptr, XV.info_ptr, ZV.ptr, ZV.info_ptr, None),
                          lambda lib: (lib.transform(T_EXP, xv, vi, zc3, vi, None), zc3)[1], False, ZV.get))
        for c in cases:
            c.cpu_once = True  # the reference walks these element by element through coordinate arithmetic: a pass takes long
        return cases

    return _replicated(dev, "general views: multi-dimensional TADs on [128,128,56,56] / [4096,128,128] / [256,1024,256], rows with a pitch",
                       4 * n1 + 4 * n2 + 8 * n3, dict(x1=x1, i1=i1, x2=x2, i2=i2, x3=x3, i3=i3, plane=plane, pi=pi, mat=mat, mi=mi,
                                                      xv=xv, yv=yv, vi=vi, bias_v=bias_v), device_set, copies)


# ---- data-movement specials: gathers, concatenations, reorders, conversions ---------------------------------
def data_movement(dev, rows=65536, cols=1024, seed=31, copies=None):
    import ctypes
    n = rows * cols
    rs = np.random.default_rng(seed)
    x = _normal(rs, n, F32)
    xi = harness.shape_info([rows, cols])
    xfi = harness.shape_info([rows, cols], "f")
    flat = _vec(n)
    ops = dev.ops
    tad_rows = dev.tad(xi, [1])
    perm = rs.permutation(rows).astype(np.int64)
    smap = -np.ones(rows, np.int32)
    smap[perm[0::2]] = perm[1::2]
    parts0, parts1 = 8, 4
    r0, c1 = rows // parts0, cols // parts1
    i0, i1 = harness.shape_info([r0, cols]), harness.shape_info([rows, c1])
    x2 = x.reshape(rows, cols)
    in0 = [np.ascontiguousarray(x2[k * r0:(k + 1) * r0]).ravel() for k in range(parts0)]
    in1 = [np.ascontiguousarray(x2[:, k * c1:(k + 1) * c1]).ravel() for k in range(parts1)]
    t_rows, t_len = 1024, n // 1024
    ti_x = harness.shape_info([t_rows, t_len])
    tad_tear = dev.tad(ti_x, [1])
    ti_z = harness.shape_info([1, t_len])
    zc = np.zeros(n, F32)
    hc = np.zeros(n, np.float16)
    xh = x.astype(np.float16)

    def table(device_arrays):
        return np.array([d.ptr for d in device_arrays], dtype=np.uint64)

    def device_set(w):
        X, Z = w.operand(x, xi), w.operand(np.zeros(n, F32), xi)
        XF = w.raw(np.ascontiguousarray(xfi, dtype=np.int64))
        FL = w.raw(np.ascontiguousarray(flat, dtype=np.int64))
        cases = []
        # pullRows: every row of x lands at a random row of z
        IDX = w.raw(perm)
        TI, TO = w.raw(tad_rows[0]), w.raw(tad_rows[1])
        ex = dev.extra(xi)
        cases.append(Case("pullrows_permute", "pullrows", n, 8 * n + 8 * rows,
                          lambda: ops.pullRowsFloat(ex, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, rows, IDX.ptr, TI.ptr, TO.ptr, TI.ptr,
                                                    TO.ptr),
                          lambda lib: (lib.pullrows(x, xi, zc, xi, perm, tad_rows, tad_rows), zc)[1], True, Z.get))
        # concat along dimension 0 (whole-array runs) and along dimension 1 (1 KiB runs)
        for name, dim, parts, pinfo in (("concat_dim0", 0, in0, i0), ("concat_dim1", 1, in1, i1)):
            P = [w.operand(p, pinfo) for p in parts]
            DT, ST = w.raw(table([o.buf for o in P])), w.raw(table([o.dinfo for o in P]))
            exc = dev.extra(xi)
            host_infos = [np.ascontiguousarray(pinfo, dtype=np.int64) for _ in parts]
            host_tab = (ctypes.c_void_p * len(parts))(*[h.ctypes.data for h in host_infos])
            exc[9] = ctypes.cast(host_tab, ctypes.c_void_p)
            exc._keep_concat = (host_infos, host_tab)
            data, shapes = (ctypes.c_void_p * 1)(DT.ptr), (ctypes.c_void_p * 1)(ST.ptr)

            def gpu(dim=dim, k=len(parts), exc=exc, data=data, shapes=shapes):
                ops.concatFloat(exc, dim, k, data, shapes, Z.ptr, Z.info_ptr, None, None)

            def cpu(lib, dim=dim, parts=parts, pinfo=pinfo):
                lib.concat(dim, parts, [pinfo] * len(parts), zc, xi)
                return zc

            cases.append(Case(name, "concat", n, 8 * n, gpu, cpu, True, Z.get))
        # flatten: a dense copy, and an f-order matrix read out in C order (a transpose)
        exf = dev.extra(y_info=xi)
        cases.append(Case("flatten_same_order", "flatten", n, 8 * n,
                          lambda: ops.flattenFloat(exf, 0, b"c", Z.ptr, FL.ptr, X.ptr, X.info_ptr),
                          lambda lib: (lib.flatten(0, "c", zc, flat, x, xi), zc)[1], True, Z.get))
        exff = dev.extra(y_info=xfi)
        cases.append(Case("flatten_f_to_c", "flatten", n, 8 * n,
                          lambda: ops.flattenFloat(exff, 0, b"c", Z.ptr, FL.ptr, X.ptr, XF.ptr),
                          lambda lib: (lib.flatten(0, "c", zc, flat, x, xfi), zc)[1], False, Z.get))
        # tear: 1024 rows of 256 KiB into 1024 separate buffers
        TG = [dev.empty(4 * t_len) for _ in range(t_rows)]
        w._operands.extend(TG)
        TT = w.raw(table(TG))
        TXI, TZI = w.raw(np.ascontiguousarray(ti_x, dtype=np.int64)), w.raw(np.ascontiguousarray(ti_z, dtype=np.int64))
        TTI, TTO = w.raw(tad_tear[0]), w.raw(tad_tear[1])
        cases.append(Case("tear_rows", "tear", n, 8 * n,
                          lambda: ops.tearFloat(ex, X.ptr, TXI.ptr, TT.ptr, TZI.ptr, TTI.ptr, TTO.ptr),
                          None, True, lambda: TG[5].download(F32, t_len)))
        # shuffle: every row trades places with a partner, in place
        S = w.operand(x, xi)
        SX, SI = w.raw(table([S.buf])), w.raw(table([S.dinfo]))
        STI, STO = w.raw(table([TI])), w.raw(table([TO]))
        M = w.raw(smap)
        cases.append(Case("shuffle_rows", "shuffle", n, 8 * n,
                          lambda: ops.shuffleFloat(ex, SX.ptr, SI.ptr, SX.ptr, SI.ptr, 1, M.ptr, STI.ptr, STO.ptr),
                          None, True, S.get))
        # conversions
        H = w.raw(xh)
        cases.append(Case("convert_float_to_half", "convert", n, 6 * n,
                          lambda: ops.convertTypes(ex, 6, X.ptr, n, 3, H.ptr),
                          lambda lib: (lib.convert(6, x, 3, hc), hc)[1], True, lambda: H.download(np.float16, n)))
        cases.append(Case("convert_half_to_float", "convert", n, 6 * n,
                          lambda: ops.convertTypes(ex, 3, H.ptr, n, 6, Z.ptr),
                          lambda lib: (lib.convert(3, xh, 6, zc), zc)[1], True, Z.get))
        return cases

    return _replicated(dev, "data movement: pullRows, concat, flatten, tear, shuffle, convert; fp32 [%d,%d]" % (rows, cols), 8 * n,
                       dict(x=x, xi=xi, perm=perm, smap=smap), device_set, copies)


# ---- configs[4]: random fills and dropout ---------------------------------------------------------------
def random_fills(dev, n=1 << 26, side=8192, seed=119, buffer_longs=1 << 20, data_seed=5, copies=None):
    ops = dev.ops
    host_buf = np.zeros(buffer_longs, np.uint64)
    dev_buf = dev.upload(np.zeros(buffer_longs, np.uint64))
    gen = ops.initRandom(dev.extra(host_buffer=host_buf.ctypes.data), seed, buffer_longs, dev_buf.ptr)
    zi = _vec(n)
    m = side * side
    di = harness.shape_info([side, side])
    xd = _normal(np.random.default_rng(data_seed), m, F32)
    cpu_state = {}

    def cpu_gen(lib):
        if "g" not in cpu_state:
            cpu_state["g"] = lib.rng_init(seed, buffer_longs)
            cpu_state["z"] = np.zeros(n, F32)
            cpu_state["x"] = xd.copy()
        return cpu_state["g"]

    def device_set(w):
        Z = w.operand(np.zeros(n, F32), zi)
        a_uni, a_gau, a_drop = w.raw(np.array([0, 1], F32)), w.raw(np.array([0, 1], F32)), w.raw(np.array([0.5], F32))
        # the host copy of the result's shapeInfo in slot 0, as nd4j passes it on these calls: without it the library
        # reads the shapeInfo back from the device, which synchronises the stream
        ex, ex_d = dev.extra(zi), dev.extra(di)
        Xd = w.operand(xd, di)
        return [
            Case("uniform_fill", "random", n, 4 * n,
                 lambda: ops.execRandomFloat(ex, RND_UNIFORM, gen, Z.ptr, Z.info_ptr, a_uni.ptr),
                 lambda lib: (cpu_gen(lib).random_z(RND_UNIFORM, cpu_state["z"], zi, np.array([0, 1], F32)), cpu_state["z"])[1], True, Z.get),
            Case("gaussian_fill", "random", n, 4 * n,
                 lambda: ops.execRandomFloat(ex, RND_GAUSSIAN, gen, Z.ptr, Z.info_ptr, Z.ptr, Z.info_ptr, Z.ptr, Z.info_ptr, a_gau.ptr),
                 lambda lib: (cpu_gen(lib).random_xyz(RND_GAUSSIAN, cpu_state["z"], zi, cpu_state["z"], zi, cpu_state["z"], zi,
                                                     np.array([0, 1], F32)), cpu_state["z"])[1], True, Z.get),
            Case("dropout_inplace", "random", m, 8 * m,
                 lambda: ops.execRandomFloat(ex_d, RND_DROPOUT, gen, Xd.ptr, Xd.info_ptr, Xd.ptr, Xd.info_ptr, a_drop.ptr),
                 lambda lib: (cpu_gen(lib).random_xz(RND_DROPOUT, cpu_state["x"], di, cpu_state["x"], di, np.array([0.5], F32)), cpu_state["x"])[1],
                 True, Xd.get)]

    def valu_bound(cases):
        # bound by the instruction count of the reference's 64-bit integer stream, not by HBM
        for c in cases:
            c.bound = "valu"
            c.note = "the arithmetic of the reference's u64 stream: valu.issue_ms prices a wave64 vector instruction at 4 cycles of its SIMD"
        return cases

    inner_set = device_set
    device_set = lambda w: valu_bound(inner_set(w))
    host_cpu_state = cpu_state
    w = _replicated(dev, "random uniform / gaussian fill 2^%d fp32, dropout p=0.5 in place [%d,%d]" % (int(np.log2(n)), side, side),
                    4 * n + 4 * m, dict(rng_buffer=host_buf, generator=gen, seed=seed, buffer_longs=buffer_longs,
                                        dropout_x=xd, di=di, zi=zi, cpu_state=host_cpu_state), device_set, copies)
    free0 = w.free

    def free():
        dev.sync()
        ops.destroyRandom(gen)
        dev_buf.free()
        free0()

    w.free = free
    return w


# ---- the whole-array transforms: Reverse, Histogram, Im2col, Col2Im, Pooling2D ------------------------------------------
def whole_array_transforms(dev, n=1 << 26, seed=41, copies=None):
    """Reverse and Histogram over 2^26 floats; Im2col / Col2Im on a [32, 64, 56, 56] image (3 x 3 kernel, stride 1,
    padding 1); 2 x 2 / stride 2 max and average pooling of a [64, 64, 112, 112] image (205 MB: the 26 MB of the other
    image are gone in the time a launch takes)."""
    rs = np.random.default_rng(seed)
    x = _uniform(rs, n, -3, 3)
    vi = _vec(n)
    bins = 256
    bi = _vec(bins)
    img, col = [32, 64, 56, 56], [32, 64, 3, 3, 56, 56]
    big, pooled = [64, 64, 112, 112], [64, 64, 56, 56]
    ii, ci, bgi, pi = harness.shape_info(img), harness.shape_info(col), harness.shape_info(big), harness.shape_info(pooled)
    n_img, n_col, n_big, n_pool = int(np.prod(img)), int(np.prod(col)), int(np.prod(big)), int(np.prod(pooled))
    image = _uniform(rs, n_img, -3, 3)
    big_image = _uniform(rs, n_big, -3, 3)
    e_hist = np.array([bins, -2.5, 2.75], F32)
    e_im2col = np.array([3, 3, 1, 1, 1, 1, 1, 1, 0, 0], F32)
    e_col2im = np.array([1, 1, 1, 1, 56, 56, 1, 1], F32)
    e_pool = {0: np.array([2, 2, 2, 2, 0, 0, 1, 1, 0, 0, 0], F32), 1: np.array([2, 2, 2, 2, 0, 0, 1, 1, 0, 1, 0], F32)}
    ops = dev.ops
    zc, hc, colc, imgc, poolc = np.zeros(n, F32), np.zeros(bins, F32), np.zeros(n_col, F32), np.zeros(n_img, F32), np.zeros(n_pool, F32)

    def device_set(w):
        X, Z = w.operand(x, vi), w.operand(np.zeros(n, F32), vi)
        H = w.operand(np.zeros(bins, F32), bi)
        I, C, P = w.operand(image, ii), w.operand(np.zeros(n_col, F32), ci), w.operand(np.zeros(n_pool, F32), pi)
        B = w.operand(big_image, bgi)
        I2 = w.operand(np.zeros(n_img, F32), ii)
        EH, EI, EC = w.raw(e_hist), w.raw(e_im2col), w.raw(e_col2im)
        EP = {k: w.raw(v) for k, v in e_pool.items()}
        cases = []
        ex = dev.extra(vi, z_info=vi)
        cases.append(Case("reverse", "transform", n, 8 * n,
                          lambda: ops.execTransformFloat(ex, 70, X.ptr, X.info_ptr, Z.ptr, Z.info_ptr, None),
                          lambda lib: (lib.transform(70, x, vi, zc, vi, None), zc)[1], True, Z.get))
        exh = dev.extra(vi, z_info=bi)
        cases.append(Case("histogram_256_bins", "transform", n, 4 * n + 8 * bins,
                          lambda: ops.execTransformFloat(exh, 48, X.ptr, X.info_ptr, H.ptr, H.info_ptr, EH.ptr),
                          lambda lib: (hc.fill(0), lib.transform(48, x, vi, hc, bi, e_hist), hc)[2], True, H.get))
        cases[-1].note = "counts accumulate over the calls of a timing loop"
        exi = dev.extra(ii, z_info=ci)
        cases.append(Case("im2col_3x3", "transform", n_col, 4 * n_img + 4 * n_col,
                          lambda: ops.execTransformFloat(exi, 37, I.ptr, I.info_ptr, C.ptr, C.info_ptr, EI.ptr),
                          lambda lib: (lib.transform(37, image, ii, colc, ci, e_im2col), colc)[1], True, C.get))
        exc = dev.extra(ci, z_info=ii)
        cases.append(Case("col2im_3x3", "transform", n_col, 4 * n_img + 4 * n_col,
                          lambda: ops.execTransformFloat(exc, 36, C.ptr, C.info_ptr, I2.ptr, I2.info_ptr, EC.ptr),
                          None, True, I2.get))
        exp_ = dev.extra(bgi, z_info=pi)
        for mode, name in ((0, "maxpool_2x2"), (1, "avgpool_2x2")):
            cases.append(Case(name, "transform", n_big, 4 * n_big + 4 * n_pool,
                              lambda mode=mode: ops.execTransformFloat(exp_, 71, B.ptr, B.info_ptr, P.ptr, P.info_ptr, EP[mode].ptr),
                              lambda lib, mode=mode: (lib.transform(71, big_image, bgi, poolc, pi, e_pool[mode]), poolc)[1], True, P.get))
        return cases

    return _replicated(dev, "whole-array transforms: reverse / histogram 2^26; im2col, col2im on [32,64,56,56]; pooling on [64,64,112,112]",
                       8 * n + 8 * n_col + 4 * n_big, dict(x=x, image=image, big_image=big_image), device_set, copies)


BUILDERS = [transform_tanh, pairwise_broadcast, reductions, reduce3_pairs, stats_softmax, random_fills]
