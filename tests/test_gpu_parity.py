"""Parity of the HIP path, driven through the C ABI of libnd4j_amd.so, against the CPU checkers.

Sizes: the vector / fixture replays are tiny; the seeded comparisons use shapes the CPU checker finishes in
seconds; the benchmark-size runs are in test_gpu_configs.py.  Tolerances are those of tests/checks.py.
"""
import itertools

import numpy as np
import pytest

import backends
import checks
from golden_inputs import BROADCAST_OPS, shape_info_np, ulp_distance
from libnd4j_amd import harness

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cpu(cpu_checker):
    return backends.CpuBackend(cpu_checker)


def test_native_library_is_the_one_running(gpu):
    import os
    from libnd4j_amd import native
    assert os.path.exists(native.LIBRARY_PATH)
    maps = open("/proc/self/maps").read()
    assert "libnd4j_amd.so" in maps
    assert gpu.ops.getAvailableDevices() >= 1
    assert gpu.ops.getDeviceTotalMemory(None) > (1 << 30)
    assert gpu.ops.getDeviceMajor(None) >= 9


def test_reference_fixtures(gpu):
    checks.check_reference_fixtures(gpu)


def test_op_vectors(gpu):
    checks.check_op_vectors(gpu)


def test_half_vectors(gpu):
    checks.check_half_vectors(gpu, exact=False)
    # reductions against the reference's own fp16-accumulating loops: within 1e-2, index reductions bit for bit
    checks.check_half_reduction_vectors(gpu, exact=False)


def test_rng_vectors(gpu):
    checks.check_rng_vectors(gpu)


def test_closed_forms(gpu):
    checks.check_closed_forms(gpu)


def test_rng_closed_forms(gpu):
    checks.check_rng_closed_forms(gpu)


def test_index_is_stored_in_the_data_type(gpu):
    n = (1 << 24) + 2
    x = np.zeros(n, np.float32)
    x[(1 << 24) + 1] = 5.0
    assert float(gpu.indexreduce_scalar(0, x, shape_info_np([1, n]))) == 16777216.0


# ---- views: dense c / f, strided, permuted -------------------------------------------------------------
VIEWS = [("c", [33, 65], "c", None, None), ("f", [33, 65], "f", None, None), ("c3", [5, 6, 7], "c", None, None),
         ("f3", [5, 6, 7], "f", None, None), ("strided", [9, 10], "c", [20, 2], None),
         ("permuted", [4, 5, 3], "c", [3, 12, 1], None), ("vec", [1, 19], "c", [1, 3], 3),
         ("c4", [3, 2, 4, 5], "c", None, None)]


def _mk(view, rs, lo=-3, hi=3):
    name, shape, order, strides, ews = view
    info = harness.shape_info(shape, order, strides=strides, ews=ews)
    return rs.uniform(lo, hi, harness.span_of(info)).astype(np.float32), info


def _touched(info):
    return harness.element_offsets(info)


def test_transform_and_pairwise_on_views(gpu, cpu):
    rs = np.random.RandomState(21)
    for vx in VIEWS:
        x, xi = _mk(vx, rs)
        for vz in VIEWS:
            if vz[1] != vx[1]:
                continue
            _, zi = _mk(vz, rs)
            sel = _touched(zi)
            for op in (15, 3, 6, 10):
                g, c = gpu.transform(op, x, xi, zi), cpu.transform(op, x, xi, zi)
                assert ulp_distance(g[sel], c[sel]).max() <= 2, (vx[0], vz[0], op)
                untouched = np.setdiff1d(np.arange(g.size), sel)
                assert np.all(g[untouched] == 0), "wrote outside the view"
            y, yi = _mk(vx, rs)
            for op in (0, 6, 2, 13):
                g, c = gpu.pairwise(op, x, xi, y, yi, zi), cpu.pairwise(op, x, xi, y, yi, zi)
                assert np.array_equal(g[sel], c[sel]), (vx[0], vz[0], op)
        # in place
        g, c = gpu.transform_inplace(15, x, xi), cpu.transform_inplace(15, x, xi)
        assert ulp_distance(g, c).max() <= 2, vx[0]


def test_rows_with_a_pitch(gpu, cpu):
    """Matrices whose rows lie a pitch apart (different pitches for the operand and the result, row lengths that are and are
    not multiples of the 16-byte vector, odd pitches that leave most rows off a 16-byte boundary): one-operand calls, calls
    with a scalar and a row added to every row take the kernel written for this layout; two full operands keep the general
    walk."""
    rs = np.random.RandomState(211)
    for dtype, tol in ((np.float32, 2), (np.float64, 2), (np.float16, None)):
        for rows, cols, px, pz in ((37, 41, 45, 43), (64, 128, 132, 128), (5, 1030, 1032, 1040), (300, 8, 9, 12), (3, 3, 5, 4)):
            xi = harness.shape_info([rows, cols], "c", strides=[px, 1])
            zi = harness.shape_info([rows, cols], "c", strides=[pz, 1])
            sel = _touched(zi)
            x = rs.uniform(-3, 3, harness.span_of(xi)).astype(dtype)
            y = rs.uniform(-3, 3, harness.span_of(xi)).astype(dtype)
            row = rs.uniform(-3, 3, cols).astype(dtype)

            def same(g, c, what):
                if tol is None:
                    g64, c64 = g[sel].astype(np.float64), c[sel].astype(np.float64)
                    assert np.all(np.abs(g64 - c64) <= 1e-2 * np.maximum(np.abs(c64), 1e-2)), what
                elif dtype == np.float32:
                    assert ulp_distance(g[sel], c[sel]).max() <= tol, what
                else:
                    assert np.allclose(g[sel], c[sel], rtol=1e-14, atol=0), what
                untouched = np.setdiff1d(np.arange(g.size), sel)
                assert np.all(g[untouched] == 0), ("wrote outside the view", what)

            case = (dtype.__name__, rows, cols, px, pz)
            for op in (3, 6, 0):  # exp (lookup tables), neg, abs
                same(gpu.transform(op, x, xi, zi), cpu.transform(op, x, xi, zi), case + ("transform", op))
            same(gpu.scalar(0, x, xi, zi, 1.5), cpu.scalar(0, x, xi, zi, 1.5), case + ("scalar",))
            same(gpu.pairwise(0, x, xi, y, xi, zi), cpu.pairwise(0, x, xi, y, xi, zi), case + ("pairwise",))
            # (handed no tables for the result, the reference walks it with the operand's: its answer exists for equal pitches
            # only; with different ones the sum itself is the check - one rounding in every type)
            g, c = gpu.broadcast(0, x, xi, row, shape_info_np([1, cols]), xi, [1]), cpu.broadcast(0, x, xi, row, shape_info_np([1, cols]), xi, [1])
            at = _touched(xi)
            assert np.array_equal(g[at], c[at]) and np.all(g[np.setdiff1d(np.arange(g.size), at)] == 0), case + ("broadcast",)
            g = gpu.broadcast(0, x, xi, row, shape_info_np([1, cols]), zi, [1])
            assert np.array_equal(g[sel].reshape(rows, cols), x[at].reshape(rows, cols) + row[None, :]), case + ("broadcast, own pitch",)
            assert np.all(g[np.setdiff1d(np.arange(g.size), sel)] == 0), case + ("broadcast, own pitch",)
            if pz >= px:
                # no tables for the result: it is walked with the operand's pitch, whatever its own shapeInfo says
                # (cpu/broadcasting.cpp:79-82) - the reference's answer, every element of the buffer compared
                g = gpu.broadcast(0, x, xi, row, shape_info_np([1, cols]), zi, [1], pass_tads=False)
                c = cpu.broadcast(0, x, xi, row, shape_info_np([1, cols]), zi, [1])
                assert np.array_equal(g, c), case + ("broadcast, no tables for the result",)


def test_pairwise_branches(gpu, cpu):
    rs = np.random.RandomState(22)
    # scalar y
    x, xi = _mk(VIEWS[0], rs)
    ys = np.array([1.75], np.float32)
    for zi in (xi, harness.shape_info([33, 65], "f")):
        assert np.array_equal(gpu.pairwise(0, x, xi, ys, shape_info_np([1, 1]), zi), cpu.pairwise(0, x, xi, ys, shape_info_np([1, 1]), zi))
    # different shapes, same length, all c order with EWS 1: walks length(y) elements linearly
    a = rs.randn(60).astype(np.float32)
    b = rs.randn(60).astype(np.float32)
    ai, bi = shape_info_np([6, 10]), shape_info_np([10, 6])
    assert np.array_equal(gpu.pairwise(6, a, ai, b, bi, ai), cpu.pairwise(6, a, ai, b, bi, ai))
    # different shapes and orders: every operand by its own C-order index
    bf = harness.shape_info([10, 6], "f")
    assert np.array_equal(gpu.pairwise(0, a, ai, b, bf, ai), cpu.pairwise(0, a, ai, b, bf, ai))
    # strided overloads, including negative-free odd strides and a tail that is not a multiple of the vector
    for n, xs, ys_, zs in ((1000, 1, 1, 1), (1001, 1, 1, 1), (7, 1, 1, 1), (333, 2, 3, 1), (333, 1, 1, 4), (0, 1, 1, 1)):
        xx = rs.randn(max(1, n * xs)).astype(np.float32)
        yy = rs.randn(max(1, n * ys_)).astype(np.float32)
        assert np.array_equal(gpu.pairwise_strided(0, xx, xs, yy, ys_, zs, None, n), cpu.pairwise_strided(0, xx, xs, yy, ys_, zs, None, n))
        g, c = gpu.transform_strided(15, xx, xs, zs, None, n), cpu.transform_strided(15, xx, xs, zs, None, n)
        assert ulp_distance(g, c).max() <= 2


def test_misaligned_buffers(gpu, cpu):
    # operands that start 4, 8 and 12 bytes past a 16-byte boundary, equal and unequal misalignment
    rs = np.random.RandomState(23)
    n = 4099
    base = rs.randn(n + 8).astype(np.float32)
    dev = gpu.dev
    X = dev.upload(base)
    Z = dev.upload(np.zeros(n + 8, np.float32))
    for xo, zo in ((1, 1), (2, 2), (3, 3), (1, 2), (0, 3)):
        gpu.ops.memset(Z.ptr, 0, (n + 8) * 4, 0, None)
        gpu.ops.execTransformFloat(dev.extra(), 0, X.ptr + 4 * xo, 1, Z.ptr + 4 * zo, 1, None, n)
        got = Z.download(np.float32)
        assert np.array_equal(got[zo:zo + n], np.abs(base[xo:xo + n])), (xo, zo)
        assert np.all(got[:zo] == 0) and np.all(got[zo + n:] == 0), (xo, zo)
    X.free()
    Z.free()
    dev.release()


def test_ismax_whole_array_dense_operands(gpu, cpu):
    # IsMax over a whole dense array finds the maximum and clears the result in one pass when x and z start on the same
    # offset from a 16-byte boundary and are one array or two apart; otherwise in two.  Lengths around the vector and
    # block sizes, operands 0..3 elements past a boundary, in place and out of place, ties, three types.
    rs = np.random.RandomState(77)
    dev = gpu.dev
    pad = 16
    for dt, name in ((np.float32, "Float"), (np.float64, "Double"), (np.float16, "Half")):
        item = np.dtype(dt).itemsize
        # (the winning index travels in the data type, as the index reductions store it: a half holds it up to 2048)
        for n in ((1, 3, 4, 5, 8, 9, 1023, 2047) if dt == np.float16 else (1, 3, 4, 5, 1023, 4099, 70001, (1 << 20) + 7)):
            # values the type holds exactly, the maximum twice: the first one wins
            base = rs.randint(-1000, 1000, n + pad).astype(dt)
            info = dev.upload(shape_info_np([1, n]))
            for xo, zo, inplace in ((0, 0, False), (1, 1, False), (3, 3, False), (1, 2, False), (0, 3, False), (0, 0, True),
                                    (2, 2, True)):
                x = base.copy()
                first = int(rs.randint(0, n))
                x[xo + first] = 1500
                if first + 2 < n:
                    x[xo + first + 2] = 1500
                X = dev.upload(x)
                Z = X if inplace else dev.upload(np.full(n + pad, 7, dt))
                getattr(gpu.ops, "execTransform" + name)(dev.extra(shape_info_np([1, n]), z_info=shape_info_np([1, n])), 41,
                                                         X.ptr + item * xo, info.ptr, Z.ptr + item * zo, info.ptr, None)
                got = Z.download(dt)
                want = np.zeros(n, dt)
                want[first] = 1
                assert np.array_equal(got[zo:zo + n], want), (name, n, xo, zo, inplace)
                if inplace:
                    assert np.array_equal(got[:zo], x[:zo]) and np.array_equal(got[zo + n:], x[zo + n:]), (name, n, xo, zo)
                else:
                    assert np.all(got[:zo] == 7) and np.all(got[zo + n:] == 7), (name, n, xo, zo)
                    assert np.array_equal(X.download(dt), x), ("input untouched", name, n, xo, zo)
                    Z.free()
                X.free()
            info.free()
    dev.release()


def _dims_of(rank):
    for k in range(1, rank):
        for dims in itertools.combinations(range(rank), k):
            yield list(dims)


def test_reductions_on_views(gpu, cpu):
    rs = np.random.RandomState(24)
    for vx in VIEWS:
        x, xi = _mk(vx, rs)
        shape = vx[1]
        rank = len(shape)
        absx = float(np.abs(x).sum())
        for dims in _dims_of(rank) if rank > 1 else []:
            out_len = int(np.prod(shape) // np.prod([shape[d] for d in dims]))
            tad_len = int(np.prod(shape)) // out_len
            for op in (1, 0, 3, 4, 6, 8, 19):
                if op == 19 and out_len == 1:
                    # the reference hands a one-element result to its whole-array loop with the caller's
                    # extraParams, and LogSumExp reads extraParams[0] there (reduce.cpp exec -> execScalar):
                    # with extraParams == null that is a null read in the reference itself, so no oracle exists
                    continue
                g, c = gpu.reduce(op, x, xi, None, dims, out_len), cpu.reduce(op, x, xi, None, dims, out_len)
                checks.assert_reduction_close(g, c, absx / out_len / np.sqrt(tad_len) if op in (1,) else 0, "%s reduce %d dims %s" % (vx[0], op, dims),
                                              rtol=1e-5 if op != 8 else 1e-4)
            for op in range(4):
                assert np.array_equal(gpu.indexreduce(op, x, xi, None, dims, out_len), cpu.indexreduce(op, x, xi, None, dims, out_len)), (vx[0], op, dims)
            for op in (0, 1):
                for bias in (0, 1):
                    g = gpu.summarystats(op, bias, x, xi, dims, out_len)
                    c = cpu.summarystats(op, bias, x, xi, dims, out_len)
                    checks.assert_reduction_close(g, c, 0, "%s stats %d/%d dims %s" % (vx[0], op, bias, dims))
        checks.assert_reduction_close([gpu.reduce_scalar(1, x, xi)], [cpu.reduce_scalar(1, x, xi)], absx / np.sqrt(x.size), vx[0] + " sum")
        assert float(gpu.reduce_scalar(3, x, xi)) == float(cpu.reduce_scalar(3, x, xi))
        checks.assert_reduction_close([gpu.reduce_scalar(19, x, xi)], [cpu.reduce_scalar(19, x, xi)], 0, vx[0] + " logsumexp")
        for op in range(4):
            assert float(gpu.indexreduce_scalar(op, x, xi)) == float(cpu.indexreduce_scalar(op, x, xi)), (vx[0], op)
        checks.assert_reduction_close([gpu.summarystats_scalar(1, 1, x, xi)], [cpu.summarystats_scalar(1, 1, x, xi)], 0, vx[0] + " std")


def test_reductions_without_caller_tad_tables(gpu, cpu):
    # extraPointers without TAD slots: the library computes and caches the tables itself
    rs = np.random.RandomState(25)
    x, xi = _mk(VIEWS[2], rs)
    for dims in ([1], [0, 2]):
        out_len = int(np.prod(VIEWS[2][1]) // np.prod([VIEWS[2][1][d] for d in dims]))
        for _ in range(2):  # second call hits the cache
            g = gpu.reduce(3, x, xi, None, dims, out_len, pass_tads=False)
            assert np.array_equal(g, cpu.reduce(3, x, xi, None, dims, out_len))
            assert np.array_equal(gpu.indexreduce(0, x, xi, None, dims, out_len, pass_tads=False), cpu.indexreduce(0, x, xi, None, dims, out_len))
    y = rs.randn(6).astype(np.float32)
    assert np.array_equal(gpu.broadcast(0, x, xi, y, shape_info_np([1, 6]), xi, [1], pass_tads=False),
                          cpu.broadcast(0, x, xi, y, shape_info_np([1, 6]), xi, [1]))


def test_tad_shapes_of_every_kernel_variant(gpu, cpu):
    # contiguous TADs of length 5 .. 20000 (sub-wave, wave, block kernels), strided TADs with and without splits
    rs = np.random.RandomState(26)
    for rows, cols in ((300, 5), (64, 31), (40, 64), (33, 300), (7, 4100), (3, 20011), (2000, 3), (5, 1), (1, 17),
                       (1500, 1028), (130, 2050), (515, 516)):
        x = rs.randn(rows * cols).astype(np.float32)
        xi = shape_info_np([rows, cols])
        scale1 = np.abs(x).reshape(rows, cols).sum(axis=1) / np.sqrt(cols)
        scale0 = np.abs(x).reshape(rows, cols).sum(axis=0) / np.sqrt(rows)
        if cols > 1 and rows > 1:
            checks.assert_reduction_close(gpu.reduce(1, x, xi, None, [1], rows), cpu.reduce(1, x, xi, None, [1], rows), scale1, "sum rows %dx%d" % (rows, cols))
            checks.assert_reduction_close(gpu.reduce(1, x, xi, None, [0], cols), cpu.reduce(1, x, xi, None, [0], cols), scale0, "sum cols %dx%d" % (rows, cols))
            assert np.array_equal(gpu.reduce(3, x, xi, None, [1], rows), cpu.reduce(3, x, xi, None, [1], rows))
            assert np.array_equal(gpu.indexreduce(0, x, xi, None, [1], rows), cpu.indexreduce(0, x, xi, None, [1], rows))
            assert np.array_equal(gpu.indexreduce(0, x, xi, None, [0], cols), cpu.indexreduce(0, x, xi, None, [0], cols))
            checks.assert_reduction_close(gpu.summarystats(0, 1, x, xi, [1], rows), cpu.summarystats(0, 1, x, xi, [1], rows), 0, "var rows")
            checks.assert_reduction_close(gpu.summarystats(0, 1, x, xi, [0], cols), cpu.summarystats(0, 1, x, xi, [0], cols), 0, "var cols")
            y = rs.randn(cols).astype(np.float32)
            assert np.array_equal(gpu.broadcast(0, x, xi, y, shape_info_np([1, cols]), xi, [1]), cpu.broadcast(0, x, xi, y, shape_info_np([1, cols]), xi, [1]))
            yc = rs.randn(rows).astype(np.float32)
            assert np.array_equal(gpu.broadcast(2, x, xi, yc, shape_info_np([rows, 1]), xi, [0]), cpu.broadcast(2, x, xi, yc, shape_info_np([rows, 1]), xi, [0]))
        assert float(gpu.indexreduce_scalar(0, x, xi)) == float(cpu.indexreduce_scalar(0, x, xi))


def test_tads_over_several_dimensions(gpu, cpu):
    """TADs over several dimensions carry no element-wise stride; which kernel walks them follows from their layout.  Shapes
    for each: dimensions that merge into one contiguous or strided run, contiguous runs placed by outer dimensions (long
    TADs cut into slices, TADs a wave or sixteen lanes share, runs whose length is no multiple of the vector width), and
    a strided innermost dimension (a lane per TAD)."""
    rs = np.random.RandomState(52)
    for shape, dims in (([12, 9, 16, 8], [2, 3]), ([12, 9, 16, 8], [0, 1]), ([130, 7, 300], [0, 2]), ([40, 50, 24], [0, 2]),
                        ([9, 400, 6], [0, 2]), ([33, 20, 5, 7], [0, 2, 3]), ([6, 40, 5, 8], [0, 2]), ([3, 70, 4, 9], [0, 2]), ([6, 150, 5, 8], [0, 2]), ([40, 9, 30, 64], [0, 2]),
                        ([5, 1100, 3, 2], [0, 2]), ([64, 3, 4100], [0, 2]), ([2, 3, 70000], [0, 2])):
        n = int(np.prod(shape))
        x = rs.randn(n).astype(np.float32)
        xi = shape_info_np(shape)
        x64 = x.astype(np.float64).reshape(shape)
        axes = tuple(dims)
        out_len = n // int(np.prod([shape[d] for d in dims]))
        tad_len = n // out_len
        what = "%s dims %s" % (shape, dims)
        scale = np.abs(x64).sum(axis=axes).ravel() / np.sqrt(tad_len)
        g, c = gpu.reduce(1, x, xi, None, dims, out_len).astype(np.float64), cpu.reduce(1, x, xi, None, dims, out_len).astype(np.float64)
        truth = x64.sum(axis=axes).ravel()
        bound = 1e-5 * np.maximum(np.abs(truth), scale)
        assert np.all(np.abs(g - truth) <= bound), what
        # (the reference's sequential fp32 sum of a long TAD drifts from the exact value by more than the bar: allow it its drift)
        assert np.all(np.abs(g - c) <= np.abs(c - truth) + bound), what
        assert np.array_equal(gpu.reduce(3, x, xi, None, dims, out_len), cpu.reduce(3, x, xi, None, dims, out_len)), what
        for op in (0, 1):
            assert np.array_equal(gpu.indexreduce(op, x, xi, None, dims, out_len), cpu.indexreduce(op, x, xi, None, dims, out_len)), what
        checks.assert_reduction_close(gpu.summarystats(0, 1, x, xi, dims, out_len), cpu.summarystats(0, 1, x, xi, dims, out_len), 0, "var " + what)
        if n <= 2000000:
            yshape = [shape[d] for d in dims]
            y = rs.uniform(1, 2, tad_len).astype(np.float32)
            yi = shape_info_np(yshape)
            for op in (0, 3):
                assert np.array_equal(gpu.broadcast(op, x, xi, y, yi, xi, dims), cpu.broadcast(op, x, xi, y, yi, xi, dims)), ("broadcast", op, what)
    # ties and half / double storage through the run-wise kernel
    shape, dims = [8, 5, 64], [0, 2]
    xi = shape_info_np(shape)
    for dt in (np.float16, np.float64):
        x = rs.randint(0, 4, int(np.prod(shape))).astype(dt)
        assert np.array_equal(gpu.indexreduce(0, x, xi, None, dims, 5), cpu.indexreduce(0, x, xi, None, dims, 5)), dt
        if dt == np.float64:
            assert np.array_equal(gpu.reduce(1, x, xi, None, dims, 5), cpu.reduce(1, x, xi, None, dims, 5))
        y = rs.uniform(1, 2, 8 * 64).astype(dt)
        g, c = gpu.broadcast(0, x, xi, y, shape_info_np([8, 64]), xi, dims), cpu.broadcast(0, x, xi, y, shape_info_np([8, 64]), xi, dims)
        assert np.array_equal(g, c), dt


def test_strided_reductions_with_many_row_ranges(gpu, cpu):
    """Reductions along dimension 0 of c-order matrices tall enough for the strided vector kernel to cut every column tile
    into eight row ranges or more (rows dealt to the ranges a batch at a time, a last batch that is short, a last tile
    that is not full): sums and maxima finish in one launch (the tile's last block merges the ranges), index pairs and
    moments in two; all three storage types, ties included."""
    rs = np.random.RandomState(57)
    for dt, shape in ((np.float32, [3001, 1100]), (np.float32, [4096, 512]), (np.float64, [2050, 530]), (np.float16, [2300, 1032])):
        rows, cols = shape
        xi = shape_info_np(shape)
        x = (rs.randint(-8, 9, rows * cols) / 4.0).astype(dt)  # many ties; sums of quarters are exact in every type's accumulator
        x64 = x.astype(np.float64).reshape(shape)
        what = "%s %s" % (np.dtype(dt).name, shape)
        for k in range(2):  # (the second call meets the slots the first one left behind)
            got = gpu.reduce(1, x, xi, None, [0], cols).astype(np.float64)
            want = x64.sum(axis=0)
            tol = 1e-2 * np.abs(x64).sum(axis=0) if dt == np.float16 else 0.0
            assert np.all(np.abs(got - want) <= tol), what
            assert np.array_equal(gpu.reduce(3, x, xi, None, [0], cols), cpu.reduce(3, x, xi, None, [0], cols)), what
            for op in (0, 1):
                assert np.array_equal(gpu.indexreduce(op, x, xi, None, [0], cols), cpu.indexreduce(op, x, xi, None, [0], cols)), what
        var = gpu.summarystats(0, 1, x, xi, [0], cols).astype(np.float64)
        truth = x64.var(axis=0, ddof=1)
        assert np.all(np.abs(var - truth) <= (1e-2 if dt == np.float16 else 1e-5) * np.maximum(truth, 1e-30)), what


def test_strided_reductions_in_short_groups(gpu, cpu):
    """TADs that are strided while the last dimension they leave out is the contiguous one and short (the rows of image
    planes summed, a sequence pooled over time): groups of a few neighbouring TADs, walked plane by plane.  Shapes on both
    sides of that kernel's conditions (range lengths, group widths, a pitch, one or several row ranges, three types)."""
    rs = np.random.RandomState(331)
    cases = (([12, 5, 30, 40], None, [0, 2]), ([16, 500, 24], None, [1]), ([2, 4000, 24], None, [1]), ([3, 700, 252], None, [1]),
             ([16, 500, 24], [500 * 32, 32, 1], [1]), ([20, 5, 30, 40], None, [0, 2]), ([4, 90, 16], None, [1]), ([5, 2000, 20], None, [1]),
             ([7, 3, 400, 8], None, [2]))
    for dtype in (np.float32, np.float64, np.float16):
        for shape, strides, dims in cases:
            xi = harness.shape_info(shape, "c", strides=strides)
            lo, hi = (0.5, 1.5) if dtype == np.float16 else (-2, 2)
            x = rs.uniform(lo, hi, harness.span_of(xi)).astype(dtype)
            out = int(np.prod([shape[d] for d in range(len(shape)) if d not in dims]))
            case = (dtype.__name__, shape, strides, dims)
            g, c = gpu.indexreduce(0, x, xi, None, dims, out), cpu.indexreduce(0, x, xi, None, dims, out)
            assert np.array_equal(g, c), case + ("index of the maximum",)
            assert np.array_equal(gpu.reduce(3, x, xi, None, dims, out), cpu.reduce(3, x, xi, None, dims, out)), case + ("max",)
            g = gpu.reduce(1, x, xi, None, dims, out).astype(np.float64)
            kept = [d for d in range(len(shape)) if d not in dims]
            v = x[harness.element_offsets(xi)].astype(np.float64).reshape(shape)
            exact = np.transpose(v, kept + list(dims)).reshape(out, -1)
            tol = (1e-2 if dtype == np.float16 else 1e-5) * np.abs(exact).sum(axis=1)
            assert np.all(np.abs(g - exact.sum(axis=1)) <= tol), case + ("sum",)
            if dtype != np.float16:
                assert np.allclose(gpu.reduce(0, x, xi, None, dims, out), cpu.reduce(0, x, xi, None, dims, out), rtol=1e-5, atol=1e-6), case + ("mean",)


def test_broadcast_on_views_all_ops(gpu, cpu):
    rs = np.random.RandomState(27)
    for shape, order, dims in (([17, 33], "c", [1]), ([17, 33], "c", [0]), ([17, 33], "f", [0]), ([17, 33], "f", [1]),
                               ([3, 4, 5], "c", [0, 2]), ([3, 4, 5], "c", [1]), ([3, 4, 5], "f", [1, 2]), ([2, 3, 4, 5], "c", [1, 3])):
        xi = harness.shape_info(shape, order)
        x = rs.uniform(1.5, 4, int(np.prod(shape))).astype(np.float32)
        yshape = [shape[d] for d in dims]
        yi = harness.shape_info(yshape if len(yshape) > 1 else [1, yshape[0]], order if len(yshape) > 1 else "c")
        y = rs.uniform(1.5, 4, int(np.prod(yshape))).astype(np.float32)
        for op in BROADCAST_OPS:
            g, c = gpu.broadcast(op, x, xi, y, yi, xi, dims), cpu.broadcast(op, x, xi, y, yi, xi, dims)
            assert ulp_distance(g, c).max() <= 2, (shape, order, dims, op)


def test_broadcast_over_outer_and_inner_dimensions(gpu, cpu):
    """y spans the outer and the inner part of a dense array ([A, B, C] along {0, 2}, [A, B, C, D] along {0, 2, 3}): inner
    extents that are multiples of the 16-byte vector take a kernel of their own, the others the general ones; three types."""
    rs = np.random.RandomState(341)
    for dtype in (np.float32, np.float64, np.float16):
        for shape, dims in (([6, 7, 8], [0, 2]), ([2, 3, 4, 8], [0, 2, 3]), ([5, 300, 64], [0, 2]), ([3, 9, 6], [0, 2]), ([4, 1, 16], [0, 2]),
                            ([40, 33, 24], [0, 2])):
            xi = harness.shape_info(shape, "c")
            x = rs.uniform(1.5, 4, int(np.prod(shape))).astype(dtype)
            yshape = [shape[d] for d in dims]
            yi = harness.shape_info(yshape, "c")
            y = rs.uniform(1.5, 4, int(np.prod(yshape))).astype(dtype)
            for op in (0, 1, 2, 3):
                g, c = gpu.broadcast(op, x, xi, y, yi, xi, dims), cpu.broadcast(op, x, xi, y, yi, xi, dims)
                if dtype == np.float32:
                    assert ulp_distance(g, c).max() <= 2, (shape, dims, op)
                else:
                    assert np.allclose(g.astype(np.float64), c.astype(np.float64), rtol=1e-2 if dtype == np.float16 else 1e-14, atol=0), (dtype.__name__, shape, dims, op)


def test_scalar_family(gpu, cpu):
    from golden_inputs import SCALAR_OPS
    rs = np.random.RandomState(32)
    n = 20000
    x = (rs.uniform(1.2, 50, n) * rs.choice([-1, 1], n)).astype(np.float32)
    xi = shape_info_np([1, n])
    for s in (1.7, -2.25):
        multiples = (np.arange(1, n + 1).astype(np.float32) * np.float32(s)).astype(np.float32)
        for op in SCALAR_OPS:
            assert ulp_distance(gpu.scalar(op, x, xi, xi, s), cpu.scalar(op, x, xi, xi, s)).max() <= 2, (op, s)
            assert ulp_distance(gpu.scalar(op, multiples, xi, xi, s), cpu.scalar(op, multiples, xi, xi, s)).max() <= 2, (op, s)
    for op in (0, 3, 20, 23):
        assert np.array_equal(gpu.scalar_strided(op, x, 3, 2, 1.7, None, n // 3), cpu.scalar_strided(op, x, 3, 2, 1.7, None, n // 3))
        assert np.array_equal(gpu.scalar_strided(op, x, 1, 1, 1.7, None, n), cpu.scalar_strided(op, x, 1, 1, 1.7, None, n))
    # views: dense f -> c, strided, permuted
    for vx in VIEWS:
        xv, xinfo = _mk(vx, rs)
        for op in (0, 3, 4, 13):
            assert np.array_equal(gpu.scalar(op, xv, xinfo, xinfo, 0.37), cpu.scalar(op, xv, xinfo, xinfo, 0.37)), (vx[0], op)
    fi, ci = harness.shape_info([100, 200], "f"), harness.shape_info([100, 200], "c")
    assert np.array_equal(gpu.scalar(1, x, fi, ci, 0.37), cpu.scalar(1, x, fi, ci, 0.37))
    # one scalar per TAD: contiguous rows, strided columns, both orders, with and without the caller's TAD tables
    for rows, cols in ((300, 150), (64, 1024), (5, 7), (257, 1023), (1021, 33)):  # also odd lengths and counts
        m = rs.uniform(1.2, 9, rows * cols).astype(np.float32)
        for order in ("c", "f"):
            mi = harness.shape_info([rows, cols], order)
            for dims, count in (([1], rows), ([0], cols)):
                sc = rs.uniform(1.2, 5, count).astype(np.float32)
                for op in (0, 2, 3, 6, 14, 20, 23):
                    want = cpu.scalar_tad(op, m, mi, sc, None, dims)
                    assert np.array_equal(gpu.scalar_tad(op, m, mi, sc, None, dims), want), (rows, cols, order, dims, op)
                assert np.array_equal(gpu.scalar_tad(0, m, mi, sc, None, dims, pass_tads=False), cpu.scalar_tad(0, m, mi, sc, None, dims))
    # rank 3: TADs over the trailing, the leading and the middle dimension, both orders (the TAD numbering follows memory
    # order only for some of them; the others take the kernels that read the offset tables)
    for order in ("c", "f"):
        mi = harness.shape_info([6, 5, 28], order)
        m = rs.uniform(1.2, 9, 6 * 5 * 28).astype(np.float32)
        for dims in ([2], [0], [1]):
            sc = rs.uniform(1.2, 5, 840 // [6, 5, 28][dims[0]]).astype(np.float32)
            assert np.array_equal(gpu.scalar_tad(0, m, mi, sc, None, dims), cpu.scalar_tad(0, m, mi, sc, None, dims)), (order, dims)
    # fp16: the scalar is rounded to fp16 before use; fp64
    xh = rs.uniform(1, 4, 4096).astype(np.float16)
    hi = shape_info_np([1, 4096])
    g, c = gpu.scalar(2, xh, hi, hi, 1.2345678), cpu.scalar(2, xh, hi, hi, 1.2345678)
    assert np.all(np.abs(g.astype(np.float64) - c.astype(np.float64)) <= 1e-2 * np.abs(c.astype(np.float64)))
    assert np.array_equal(gpu.scalar(13, xh, hi, hi, 1.2345678), np.full(4096, np.float16(1.2345678)))
    xd = rs.randn(1000)
    di = shape_info_np([1, 1000])
    assert np.allclose(gpu.scalar(3, xd, di, di, 1.7), cpu.scalar(3, xd, di, di, 1.7), rtol=1e-15, atol=0)
    # unknown opNum: output untouched
    assert np.all(gpu.scalar(99, x, xi, xi, 1.0) == 0)


def test_reduce3_family(gpu, cpu):
    rs = np.random.RandomState(34)
    eps = np.array([0.05], np.float32)

    def close(a, b, what):
        # relative 1e-5 on the sums; cosine / Jaccard distances are 1 - ratio, so the 1e-5 of the ratio (of order one)
        # is an absolute error on them
        assert np.allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), rtol=1e-5, atol=2e-5), what

    # whole arrays: contiguous (vector kernel, sliced), odd lengths, f-order, strided views, mixed orders
    for shape, order in (([1, 777], "c"), ([1, 300001], "c"), ([33, 65], "c"), ([33, 65], "f"), ([5, 6, 7], "c"), ([3, 2, 4, 5], "f")):
        xi = harness.shape_info(shape, order)
        n = int(np.prod(shape))
        x = rs.uniform(0.1, 2, n).astype(np.float32)
        y = (x + rs.uniform(-0.1, 0.1, n)).astype(np.float32)
        y[::7] = x[::7]
        for op in range(8):
            e = eps if op == 4 else None
            close(gpu.reduce3_scalar(op, x, xi, y, xi, e), cpu.reduce3_scalar(op, x, xi, y, xi, e), (shape, order, op))
        other = harness.shape_info(shape, "f" if order == "c" else "c")
        for op in (0, 2, 3):
            close(gpu.reduce3_scalar(op, x, xi, y, other), cpu.reduce3_scalar(op, x, xi, y, other), (shape, "mixed", op))
    vx = VIEWS[4]  # strided
    xs, xsi = _mk(vx, rs)
    ys = (xs + 0.25).astype(np.float32)
    for op in (0, 1, 3, 7):
        close(gpu.reduce3_scalar(op, xs, xsi, ys, xsi), cpu.reduce3_scalar(op, xs, xsi, ys, xsi), ("strided", op))
    # along dimensions: TAD against TAD, TAD against one vector (with and without the caller's TAD tables)
    for shape, order, dims in (([33, 65], "c", [1]), ([33, 65], "c", [0]), ([6, 5, 7], "c", [2]), ([6, 5, 7], "c", [1, 2]),
                               ([6, 5, 7], "c", [0]), ([40, 5000], "c", [1]), ([300, 130], "f", [0]),
                               ([5, 40003], "c", [1]), ([3, 70000], "c", [1])):  # few long runs: sliced over the chip
        xi = harness.shape_info(shape, order)
        n = int(np.prod(shape))
        x = rs.uniform(0.1, 2, n).astype(np.float32)
        y = (x + rs.uniform(-0.1, 0.1, n)).astype(np.float32)
        out_len = n // int(np.prod([shape[d] for d in dims]))
        tad_len = n // out_len
        for op in (0, 1, 2, 3, 5, 6, 7):
            # without element-wise strides on the arrays and their TADs the reference keeps one set of running norms
            # for all TADs (reduce3.h:1322-1341) and its cosine / Jaccard results drift: no checker for those
            if not ((len(dims) > 1 or order == "f") and op in (2, 5, 6)):
                close(gpu.reduce3(op, x, xi, y, xi, None, dims, out_len), cpu.reduce3(op, x, xi, y, xi, None, dims, out_len), (shape, dims, op))
            yv = y[:tad_len].copy()
            yi = shape_info_np([1, tad_len])
            want = cpu.reduce3(op, x, xi, yv, yi, None, dims, out_len, tad_way=True)
            close(gpu.reduce3(op, x, xi, yv, yi, None, dims, out_len), want, (shape, dims, op, "vector y"))
            close(gpu.reduce3(op, x, xi, yv, yi, None, dims, out_len, pass_tads=False), want, (shape, dims, op, "no tables"))
    # all pairs of TADs
    xi, yi = shape_info_np([7, 190]), shape_info_np([4, 190])
    x, y = rs.uniform(0.1, 2, 7 * 190).astype(np.float32), rs.uniform(0.1, 2, 4 * 190).astype(np.float32)
    for op in (0, 1, 2, 3, 5, 6, 7):
        close(gpu.reduce3_all(op, x, xi, y, yi, None, [1], 28), cpu.reduce3_all(op, x, xi, y, yi, None, [1], 28), ("all", op))
    # a few long runs, every pair of them: sliced, not tiled
    xi, yi = shape_info_np([3, 50001]), shape_info_np([2, 50001])
    x, y = rs.uniform(0.1, 2, 3 * 50001).astype(np.float32), rs.uniform(0.1, 2, 2 * 50001).astype(np.float32)
    for op in (0, 1, 2, 3, 5, 6, 7):
        close(gpu.reduce3_all(op, x, xi, y, yi, None, [1], 6), cpu.reduce3_all(op, x, xi, y, yi, None, [1], 6), ("long all", op))
    # enough pairs for the tiled kernel: ragged tile edges, a run length that ends inside a staged step, misaligned runs
    # (the last shape has enough 64 x 64 tiles for the larger tile; the others run 32 x 32 ones)
    # (from the fifth shape on there are enough 64 x 64 tiles for the larger tile, which for dot and the cosines is the
    # matrix-unit kernel: ragged runs that end inside a step, whole aligned runs, and whole runs with ragged tile edges; the
    # last two have enough 64 x 128 tiles for its wider form, ragged and whole)
    for (nx, ny, length) in ((70, 33, 100), (64, 128, 256), (17, 16, 9), (130, 65, 1027), (1450, 1420, 43), (1536, 1408, 96),
                             (1500, 1480, 64), (2100, 2000, 70), (2048, 2048, 64)):
        xi, yi = shape_info_np([nx, length]), shape_info_np([ny, length])
        x, y = rs.uniform(0.1, 2, nx * length).astype(np.float32), rs.uniform(0.1, 2, ny * length).astype(np.float32)
        x64, y64 = x.astype(np.float64).reshape(nx, length), y.astype(np.float64).reshape(ny, length)
        for op in (0, 1, 2, 3, 5, 6, 7):
            got = gpu.reduce3_all(op, x, xi, y, yi, None, [1], nx * ny)
            close(got, cpu.reduce3_all(op, x, xi, y, yi, None, [1], nx * ny), ("tiled all", nx, ny, length, op))
        dots = x64 @ y64.T
        assert np.allclose(gpu.reduce3_all(3, x, xi, y, yi, None, [1], nx * ny).reshape(nx, ny), dots, rtol=1e-5)
        norms = np.sqrt((x64 * x64).sum(axis=1))[:, None] * np.sqrt((y64 * y64).sum(axis=1))[None, :]
        assert np.allclose(gpu.reduce3_all(2, x, xi, y, yi, None, [1], nx * ny).reshape(nx, ny), dots / norms, rtol=1e-5)
        assert np.allclose(gpu.reduce3_all(5, x, xi, y, yi, None, [1], nx * ny).reshape(nx, ny), 1 - dots / norms, rtol=1e-4, atol=1e-6)
        if nx * ny > 100000:
            xh, yh = x.astype(np.float16), y.astype(np.float16)
            doth = xh.astype(np.float64).reshape(nx, length) @ yh.astype(np.float64).reshape(ny, length).T
            goth = gpu.reduce3_all(3, xh, xi, yh, yi, None, [1], nx * ny).astype(np.float64).reshape(nx, ny)
            assert np.allclose(goth, doth, rtol=2e-3), ("half dots", nx, ny, length)
        # with the caller's TAD tables (nothing is read back from the device then)
        before = gpu.ops.amd_hostFetchCount()
        assert np.allclose(gpu.reduce3_all(3, x, xi, y, yi, None, [1], nx * ny, pass_tads=True).reshape(nx, ny), dots, rtol=1e-5)
        assert gpu.ops.amd_hostFetchCount() == before
        if nx * ny > 100000:
            if nx * ny * length < 100000000:  # (the check's own temporary holds nx * ny * length doubles)
                xd, yd = rs.randn(nx * length), rs.randn(ny * length)
                assert np.allclose(gpu.reduce3_all(1, xd, xi, yd, yi, None, [1], nx * ny).reshape(nx, ny),
                                   np.sqrt(((xd.reshape(nx, 1, length) - yd.reshape(1, ny, length)) ** 2).sum(axis=2)), rtol=1e-12)
            continue
        # EqualsWithEps counts the pairs that differ: elements staged beyond the end of a run must not be counted
        y2 = x[:ny * length].copy() if nx >= ny else np.resize(x, ny * length)
        y2[::7] += 1.0
        xa, yb = x.reshape(nx, 1, length), y2.reshape(1, ny, length)
        diff, eps = np.abs(xa - yb), np.float32(1e-5)  # the op's rule (ops.h EqualsWithEps), in float as the op applies it
        want = ((diff > eps) & (diff > np.maximum(np.abs(xa), np.abs(yb)) * eps)).sum(axis=2)
        got = gpu.reduce3_all(4, x, xi, y2, yi, np.array([1e-5, 0, 0], np.float32), [1], nx * ny).reshape(nx, ny)
        assert np.array_equal(got, want.astype(np.float32)), ("equals", nx, ny, length)
        xd, yd = rs.randn(nx * length), rs.randn(ny * length)
        assert np.allclose(gpu.reduce3_all(3, xd, xi, yd, yi, None, [1], nx * ny).reshape(nx, ny),
                           xd.reshape(nx, length) @ yd.reshape(ny, length).T, rtol=1e-12, atol=1e-12)
        xh, yh = x.astype(np.float16), y.astype(np.float16)
        hd = xh.astype(np.float64).reshape(nx, length) @ yh.astype(np.float64).reshape(ny, length).T
        assert np.allclose(gpu.reduce3_all(3, xh, xi, yh, yi, None, [1], nx * ny).astype(np.float64).reshape(nx, ny), hd, rtol=1e-2)
    # float64 ground truth at a size the sliced kernel splits
    n = 1 << 20
    x = rs.randn(n).astype(np.float32)
    y = rs.randn(n).astype(np.float32)
    vi = shape_info_np([1, n])
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    scale = np.abs(x64 * y64).sum() / np.sqrt(n)
    assert abs(float(gpu.reduce3_scalar(3, x, vi, y, vi)) - np.dot(x64, y64)) <= 1e-5 * max(abs(np.dot(x64, y64)), scale)
    assert abs(float(gpu.reduce3_scalar(1, x, vi, y, vi)) - np.linalg.norm(x64 - y64)) <= 1e-5 * np.linalg.norm(x64 - y64)
    cos = np.dot(x64, y64) / (np.linalg.norm(x64) * np.linalg.norm(y64))
    assert abs(float(gpu.reduce3_scalar(2, x, vi, y, vi)) - cos) <= 1e-5
    # fp16 and fp64
    xh, yh = rs.uniform(0.5, 1.5, 4096).astype(np.float16), rs.uniform(0.5, 1.5, 4096).astype(np.float16)
    hi = shape_info_np([1, 4096])
    dot = np.dot(xh.astype(np.float64), yh.astype(np.float64))
    assert abs(float(gpu.reduce3_scalar(3, xh, hi, yh, hi)) - dot) <= 1e-2 * dot
    xd, yd = rs.randn(5000), rs.randn(5000)
    di = shape_info_np([1, 5000])
    assert abs(float(gpu.reduce3_scalar(0, xd, di, yd, di)) - np.abs(xd - yd).sum()) <= 1e-12 * np.abs(xd - yd).sum()
    # unknown opNum
    assert float(gpu.reduce3_scalar(42, x, vi, y, vi)) == 0.0


def test_special_transforms(gpu, cpu):
    rs = np.random.RandomState(36)

    def close(a, b, what):
        a64, b64 = np.asarray(a, np.float64), np.asarray(b, np.float64)
        assert np.all(np.abs(a64 - b64) <= 1e-5 * np.abs(b64) + 1e-7), what

    # softmax family: short / wave / block rows, vectors, f-order (rows adjacent in memory), f -> c
    # (row lengths chosen to reach every register-resident variant: 16 / 64 / 256 lanes per row with 2..16 vectors each,
    # and the f-order kernel with 2, 8 and 16 vectors per thread, next to the shapes that fall back to three passes)
    for shape, order in (([37, 129], "c"), ([300, 17], "c"), ([9, 5000], "c"), ([1, 500], "c"), ([700, 1], "c"), ([1, 70001], "c"),
                         ([7, 100], "c"), ([6, 200], "c"), ([4, 600], "c"), ([5, 3000], "c"), ([3, 16384], "c"), ([2, 16388], "c"),
                         ([257, 96], "f"), ([64, 300], "f"), ([128, 200], "f"), ([96, 1500], "f"), ([64, 2048], "f"),
                         ([64, 2052], "f"), ([8, 8], "c"),
                         # rows too long for registers: maxima and sums from the reduction kernels (sliced from 16384 on)
                         ([32, 50257], "c"), ([4, 100000], "c"), ([3, 20000], "c"), ([6, 9001], "c"), ([100000, 1], "c"),
                         ([256, 4100], "f"), ([300, 2500], "f"), ([600, 16500], "c"), ([520, 4100], "c"),
                         # many rows of 16385..65536 floats: one 1024-thread block keeps a row in registers
                         # (from 128 rows on; fewer rows, or longer ones, go through the reduction kernels)
                         ([128, 20000], "c"), ([130, 65536], "c"), ([129, 50001], "c"), ([128, 65537], "c"), ([128, 65540], "c"),
                         ([127, 40000], "c")):
        n = int(np.prod(shape))
        xi = harness.shape_info(shape, order)
        x = rs.uniform(-6, 6, n).astype(np.float32)
        logical = x.astype(np.float64).reshape(shape, order="F" if order == "f" else "C")
        rows = logical if min(shape) > 1 else logical.reshape(1, -1)
        truth = np.exp(rows - rows.max(axis=1, keepdims=True))
        truth /= truth.sum(axis=1, keepdims=True)
        for op, f in ((38, lambda v: v), (39, lambda v: v * (1 - v)), (40, np.log)):
            got = gpu.transform(op, x, xi, xi).astype(np.float64).reshape(shape, order="F" if order == "f" else "C")
            got = got if min(shape) > 1 else got.reshape(1, -1)
            assert np.all(np.abs(got - f(truth)) <= 2e-5 * np.abs(f(truth)) + 1e-7), (shape, order, op)
        if order == "c":
            close(gpu.transform(38, x, xi, xi), cpu.transform(38, x, xi, xi), (shape, "vs cpu"))
            if shape[1] != 1:
                close(gpu.transform_inplace(40, x, xi), cpu.transform_inplace(40, x, xi), (shape, "log in place"))
    fi, ci = harness.shape_info([40, 50], "f"), harness.shape_info([40, 50], "c")
    x = rs.uniform(-3, 3, 2000).astype(np.float32)
    got = gpu.transform(38, x, fi, ci).reshape(40, 50).astype(np.float64)
    rows = x.astype(np.float64).reshape(40, 50, order="F")
    truth = np.exp(rows - rows.max(axis=1, keepdims=True))
    truth /= truth.sum(axis=1, keepdims=True)
    assert np.all(np.abs(got - truth) <= 2e-5 * truth)
    # half and double, row-major and column-major, short and long rows
    for shape, order in (([64, 96], "c"), ([5, 4000], "c"), ([3, 30000], "c"), ([128, 600], "f"), ([64, 1100], "f"),
                         ([2, 70000], "c"), ([300, 4500], "f"), ([3, 100000], "c"),  # a half row sum beyond 65504 stays finite
                         ([128, 12000], "c"), ([130, 16383], "c")):  # doubles: rows of 8193..16384 in 1024-thread blocks
        n = shape[0] * shape[1]
        od = "F" if order == "f" else "C"
        info = harness.shape_info(shape, order)
        xh = rs.uniform(-2, 2, n).astype(np.float16)
        g = gpu.transform(38, xh, info, info).astype(np.float64).reshape(shape, order=od)
        rows = xh.astype(np.float64).reshape(shape, order=od)
        truth = np.exp(rows - rows.max(axis=1, keepdims=True))
        truth /= truth.sum(axis=1, keepdims=True)
        assert np.all(np.abs(g - truth) <= 1e-2 * truth + 1e-4), ("half", shape, order)
        xd = rs.randn(n)
        rows = xd.reshape(shape, order=od)
        truth = np.exp(rows - rows.max(axis=1, keepdims=True))
        truth /= truth.sum(axis=1, keepdims=True)
        for op, f in ((38, lambda v: v), (39, lambda v: v * (1 - v)), (40, np.log)):
            got = gpu.transform(op, xd, info, info).reshape(shape, order=od)
            assert np.allclose(got, f(truth), rtol=1e-12, atol=1e-300), ("double", shape, order, op)
    # IsMax: whole array (also a large one, f-order and 3-D), and along a dimension
    for shape, order in (([1, 300], "c"), ([12, 40], "c"), ([5, 6, 7], "c"), ([12, 40], "f"), ([1, 200003], "c")):
        n = int(np.prod(shape))
        xi = harness.shape_info(shape, order)
        x = rs.permutation(n).astype(np.float32)
        got = gpu.transform(41, x, xi, xi)
        assert np.array_equal(got, cpu.transform(41, x, xi, xi)), (shape, order)
        assert got.sum() == 1 and got[np.argmax(x)] == 1
    tie = np.array([1, 7, 7, 3, 7, 0], np.float32)
    assert np.array_equal(gpu.transform(41, tie, shape_info_np([1, 6]), shape_info_np([1, 6])), [0, 1, 0, 0, 0, 0])
    for shape, order in (([12, 40], "c"), ([12, 40], "f"), ([300, 700], "c"), ([3, 9000], "c"), ([2, 9001], "c")):  # long rows: pieces
        xi = harness.shape_info(shape, order)
        n = shape[0] * shape[1]
        x = rs.permutation(n).astype(np.float32)
        m = x.reshape(shape, order="F" if order == "f" else "C")
        for dim in (0, 1):
            e = np.array([1, dim], np.float32)
            got = gpu.transform(41, x, xi, xi, e)
            want = (m == m.max(axis=dim, keepdims=True)).astype(np.float32)
            assert np.array_equal(got.reshape(shape, order="F" if order == "f" else "C"), want), (shape, order, dim)
            if order == "c":
                assert np.array_equal(got, cpu.transform(41, x, xi, xi, e)), (shape, dim)


def test_reductions_over_few_very_long_rows(gpu, cpu):
    """A handful of contiguous TADs of several hundred thousand elements are reduced in slices (one block per TAD would
    idle most of the chip): same results as the CPU checker and as float64 arithmetic."""
    rs = np.random.RandomState(21)
    for rows, cols in ((3, 200000), (1, 70001 * 3), (7, 65536)):
        if rows == 1:
            continue  # a single TAD is a full-array reduction, covered elsewhere
        info = shape_info_np([rows, cols])
        x = rs.randn(rows * cols).astype(np.float32)
        m = x.astype(np.float64).reshape(rows, cols)
        scale = np.abs(m).sum(axis=1) / np.sqrt(cols)
        got = gpu.reduce(1, x, info, None, [1], rows).astype(np.float64)
        assert np.all(np.abs(got - m.sum(axis=1)) <= 1e-5 * np.maximum(np.abs(m.sum(axis=1)), scale)), (rows, cols, "sum")
        assert np.array_equal(gpu.reduce(3, x, info, None, [1], rows), m.max(axis=1).astype(np.float32)), (rows, cols, "max")
        got = gpu.reduce(0, x, info, None, [1], rows).astype(np.float64)
        assert np.all(np.abs(got - m.mean(axis=1)) <= 1e-5 * np.maximum(np.abs(m.mean(axis=1)), scale / cols)), (rows, cols, "mean")
        assert np.array_equal(gpu.indexreduce(0, x, info, None, [1], rows), np.argmax(m, axis=1).astype(np.float32)), (rows, cols)
        assert np.array_equal(gpu.indexreduce(0, x, info, None, [1], rows), cpu.indexreduce(0, x, info, None, [1], rows))
        var = m.var(axis=1, ddof=1)
        got = gpu.summarystats(0, 1, x, info, [1], rows).astype(np.float64)
        assert np.all(np.abs(got - var) <= 1e-5 * var), (rows, cols, "variance")
        xd = rs.randn(rows * cols)
        assert np.allclose(gpu.reduce(1, xd, info, None, [1], rows), xd.reshape(rows, cols).sum(axis=1), rtol=1e-10, atol=1e-9)
        xh = (rs.randn(rows * cols) * 0.1).astype(np.float16)
        got = gpu.reduce(3, xh, info, None, [1], rows)
        assert np.array_equal(got, xh.reshape(rows, cols).max(axis=1))


def test_broadcast_over_gap_free_tads(gpu):
    """Rows of a dense c-order array and columns of a dense f-order one go through the kernel that walks the array as
    one vector; every result is a single IEEE operation, so numpy gives the expected bits.  Shapes whose TAD length is
    not a multiple of the vector width, and a result laid out differently, take the other broadcast kernels."""
    rs = np.random.RandomState(5)
    for dt in (np.float32, np.float16, np.float64):
        for shape, order, dim in (([33, 64], "c", 1), ([64, 33], "f", 0), ([5, 7, 24], "c", 2), ([40, 3, 2], "f", 0), ([33, 62], "c", 1),
                                  ([1000, 1024], "c", 1), ([2048, 300], "f", 0),
                                  # odd row lengths, and an element count that leaves single elements after the last vector
                                  ([700, 1023], "c", 1), ([513, 1025], "c", 1), ([7, 9], "c", 1), ([1021, 67], "f", 0), ([3, 5, 11], "c", 2),
                                  # any other single dimension of a dense array: runs of `stride` elements share one y
                                  ([33, 64], "c", 0), ([64, 33], "f", 1), ([5, 7, 24], "c", 1), ([5, 7, 24], "c", 0), ([40, 3, 2], "f", 1),
                                  ([700, 1023], "c", 0), ([9, 5, 11], "f", 1), ([9, 5, 11], "f", 2), ([2, 3, 5, 7], "c", 2), ([1000, 7], "c", 0)):
            od = "F" if order == "f" else "C"
            n = int(np.prod(shape))
            info = harness.shape_info(shape, order)
            x = rs.randn(n).astype(dt)
            y = rs.randn(shape[dim]).astype(dt)
            logical = x.reshape(shape, order=od)
            bshape = [1] * len(shape)
            bshape[dim] = shape[dim]
            for op, f in ((0, np.add), (2, np.multiply), (1, np.subtract)):
                got = gpu.broadcast(op, x, info, y, shape_info_np([1, shape[dim]]), info, [dim]).reshape(shape, order=od)
                want = f(logical, y.reshape(bshape)).astype(dt)
                assert np.array_equal(got, want), (np.dtype(dt).name, shape, order, op)
    # c-order input into an f-order result: not gap-free on the result side
    xi, zi = harness.shape_info([16, 32], "c"), harness.shape_info([16, 32], "f")
    x = rs.randn(512).astype(np.float32)
    y = rs.randn(32).astype(np.float32)
    got = gpu.broadcast(0, x, xi, y, shape_info_np([1, 32]), zi, [1]).reshape(16, 32, order="F")
    assert np.array_equal(got, x.reshape(16, 32) + y[None, :])


def test_data_movement(gpu):
    """flatten / concat / pullRows / tear / shuffle / convertTypes through the C ABI, bit for bit against numpy (the
    same check the CPU restatement and the compiled reference pass)."""
    checks.check_data_movement(gpu, big=True)
    # concat without the host table of input shapes (extraPointers[9] absent): same result
    from libnd4j_amd.harness import shape_info
    arrays = [np.arange(12, dtype=np.float32), np.arange(100, 118, dtype=np.float32)]
    infos = [shape_info([2, 6]), shape_info([3, 6])]
    got = gpu.concat(0, arrays, infos, shape_info([5, 6]), host_shapes=False)
    assert np.array_equal(got, np.concatenate(arrays))


def test_nan_and_special_values(gpu, cpu):
    x = np.array([np.nan, 1.0, -np.inf, np.inf, 0.0, -0.0, 3.0, np.nan, 2.0, -1e38, 1e38, 5.0], np.float32)
    xi = shape_info_np([1, x.size])
    for op in (79, 80, 81, 0, 6, 46):
        g, c = gpu.transform(op, x, xi, xi, np.array([7, 0, 0, 0], np.float32)), cpu.transform(op, x, xi, xi, np.array([7, 0, 0, 0], np.float32))
        assert ulp_distance(g, c).max() == 0 and np.array_equal(np.isnan(g), np.isnan(c)), op
    # NaN never wins an index reduction; IndexMax over the finite part
    assert float(gpu.indexreduce_scalar(0, x, xi)) == float(cpu.indexreduce_scalar(0, x, xi)) == 3.0
    assert float(gpu.indexreduce_scalar(1, x, xi)) == float(cpu.indexreduce_scalar(1, x, xi))


def test_empty_and_single_element_inputs(gpu, cpu):
    """Lengths 0 and 1, the smallest TADs and the smallest number of TADs: what the reference's loops do when a caller
    hands them nothing or next to nothing (strided overloads with n == 0 write nothing)."""
    x = np.array([3.5, -2.0, 7.0, 1.0], np.float32)
    for n, want in ((0, [0, 0, 0, 0]), (1, [3.5, 0, 0, 0])):
        assert np.array_equal(gpu.transform_strided(0, x, 1, 1, None, n, zsize=4), want), n
    assert gpu.pairwise_strided(0, x, 1, x, 1, 1, None, 0)[0] == 0.0 and gpu.pairwise_strided(0, x, 1, x, 1, 1, None, 1)[0] == 7.0
    assert gpu.scalar_strided(0, x, 1, 1, 2.0, None, 0)[0] == 0.0 and gpu.scalar_strided(0, x, 1, 1, 2.0, None, 1)[0] == 5.5
    one = shape_info_np([1, 1])
    v = np.array([-4.25], np.float32)
    assert gpu.transform(0, v, one, one)[0] == 4.25
    assert gpu.pairwise(6, v, one, v, one, one)[0] == np.float32(-4.25) * np.float32(-4.25)
    assert float(gpu.reduce_scalar(1, v, one)) == float(cpu.reduce_scalar(1, v, one)) == -4.25
    assert float(gpu.reduce_scalar(3, v, one)) == -4.25
    assert float(gpu.indexreduce_scalar(0, v, one)) == float(cpu.indexreduce_scalar(0, v, one)) == 0.0
    for bias in (False, True):
        assert float(gpu.summarystats_scalar(0, bias, v, one)) == float(cpu.summarystats_scalar(0, bias, v, one)) == 0.0
    # TADs of length 1 (reducing a column vector along its unit dimension) and a single TAD spanning the array
    col, row = shape_info_np([5, 1]), shape_info_np([1, 5])
    w = np.array([2.0, -1.0, 9.0, 9.0, 0.5], np.float32)
    for op in (0, 1, 3):
        assert np.array_equal(gpu.reduce(op, w, col, None, [1], 5), cpu.reduce(op, w, col, None, [1], 5)), op
        assert np.array_equal(gpu.reduce(op, w, row, None, [1], 1), cpu.reduce(op, w, row, None, [1], 1)), op
    assert np.array_equal(gpu.indexreduce(0, w, col, None, [1], 5), np.zeros(5, np.float32))
    assert np.array_equal(gpu.indexreduce(0, w, row, None, [1], 1), [2.0])
    assert np.array_equal(gpu.summarystats(0, True, w, col, [1], 5), cpu.summarystats(0, True, w, col, [1], 5))
    # softmax of a single element and of a single row; IsMax of a single element
    assert gpu.transform(38, v, one, one)[0] == 1.0
    assert gpu.transform(41, v, one, one)[0] == 1.0
    sm = gpu.transform(38, w, row, row).astype(np.float64)
    assert abs(sm.sum() - 1.0) <= 1e-6 and sm[2] == sm[3] == sm.max()
    # broadcast of a one-element vector along a unit dimension
    assert np.array_equal(gpu.broadcast(0, w, col, np.array([10.0], np.float32), shape_info_np([1, 1]), col, [1]),
                          cpu.broadcast(0, w, col, np.array([10.0], np.float32), shape_info_np([1, 1]), col, [1]))


def test_unknown_op_leaves_output_untouched(gpu, capfd):
    x = np.ones(64, np.float32)
    xi = shape_info_np([1, 64])
    got = gpu.transform(500, x, xi, xi, z=np.full(64, 9.0, np.float32))
    assert np.all(got == 9.0)
    assert float(gpu.reduce_scalar(2, x, xi)) == 0.0  # opNum 2 is a gap in the reduce table


def test_whole_array_transforms_vectors_and_closed_forms(gpu):
    checks.check_whole_array_vectors(gpu)
    checks.check_whole_array_closed_forms(gpu)


def test_whole_array_transforms(gpu, cpu):
    # Col2Im 36, Im2col 37, Histogram 48, Reverse 70, Pooling2D 71 on generated shapes, strides and geometries
    done = checks.check_whole_array_transforms(gpu, cpu, 41, 500)
    assert all(done.get(k, 0) >= 50 for k in range(5)), done
    checks.check_whole_array_transforms(gpu, cpu, 42, 200, dtypes=(np.float16,))


def test_whole_array_transforms_larger(gpu, cpu):
    rs = np.random.RandomState(43)
    f = np.float32
    # Reverse of odd lengths (misaligned mirrored vectors), out of place and in place, three types
    for n in (1, 2, 7, 4099, (1 << 20) + 3, (1 << 22)):
        for dt in (np.float32, np.float64, np.float16):
            x = rs.uniform(-3, 3, n).astype(dt)
            vi = shape_info_np([1, n])
            assert np.array_equal(gpu.transform(70, x, vi, vi), x[::-1]), ("reverse", n, dt)
            assert np.array_equal(gpu.transform_inplace(70, x, vi), x[::-1]), ("reverse in place", n, dt)
    # Histogram over a few million elements: bins in LDS, handed over as a table of one row per block (up to 2048 bins) or
    # with atomics on one row, and, beyond 8192 bins, counted in global memory
    n = (1 << 22) + 5
    x = rs.uniform(-3, 3, n).astype(f)
    for bins in (10, 300, 2048, 2049, 8192, 20000):
        extra = np.array([bins, -2.5, 2.75], f)
        xi, zi = shape_info_np([1, n]), shape_info_np([1, bins])
        assert np.array_equal(gpu.transform(48, x, xi, zi, extra), cpu.transform(48, x, xi, zi, extra)), ("histogram", bins)
    # a convolution-sized image through Im2col and back through Col2Im, and pooled
    img, col, pooled = [4, 16, 56, 56], [4, 16, 3, 3, 56, 56], [4, 16, 28, 28]
    ii, ci, pi = shape_info_np(img), shape_info_np(col), shape_info_np(pooled)
    x = rs.uniform(-3, 3, int(np.prod(img))).astype(f)
    e_im = np.array([3, 3, 1, 1, 1, 1, 1, 1, 0, 0], f)
    g, c = gpu.transform(37, x, ii, ci, e_im), cpu.transform(37, x, ii, ci, e_im)
    assert np.array_equal(g, c), "im2col"
    e_col = np.array([1, 1, 1, 1, 56, 56, 1, 1], f)
    assert np.array_equal(gpu.transform(36, g, ci, ii, e_col), cpu.transform(36, c, ci, ii, e_col)), "col2im"
    for mode, p0 in ((0, 0.0), (1, 0.0), (1, 1.0), (2, 2.0)):
        e_pool = np.array([2, 2, 2, 2, 0, 0, 1, 1, 0, mode, p0], f)
        gp, cp = gpu.transform(71, x, ii, pi, e_pool), cpu.transform(71, x, ii, pi, e_pool)
        if mode == 0:
            assert np.array_equal(gp, cp), "max pooling"
        else:
            assert np.allclose(gp, cp, rtol=1e-5, atol=1e-6), ("pooling", mode, p0)


def test_whole_array_transforms_usual_windows(gpu, cpu):
    # The shapes that have kernels of their own: Im2col with a block per channel (1024 (batch, channel) pairs or more),
    # Col2Im with the window compiled in (1x1, 2x2, 3x3, 5x5) and with a run-time window (3x2, 7x7), 2x2 / stride 2
    # pooling with its paired loads (even and odd row pitches, result rows of even and odd length), for the three types.
    rs = np.random.RandomState(47)
    for dt in (np.float32, np.float64, np.float16):
        for (kH, kW, pad) in ((3, 3, 1), (1, 1, 0), (2, 2, 0), (5, 5, 2), (3, 2, 1), (7, 7, 3)):
            bS, iC, iH, iW = 16, 64, 14, 12
            oH, oW = iH + 2 * pad - kH + 1, iW + 2 * pad - kW + 1
            img, col = [bS, iC, iH, iW], [bS, iC, kH, kW, oH, oW]
            ii, ci = shape_info_np(img), shape_info_np(col)
            x = rs.randint(-8, 9, int(np.prod(img))).astype(dt)  # small integers: every sum is exact in every type
            e_im = np.array([kH, kW, 1, 1, pad, pad, 1, 1, 0, 0], dt)
            g, c = gpu.transform(37, x, ii, ci, e_im), cpu.transform(37, x, ii, ci, e_im)
            assert np.array_equal(g, c), ("im2col", dt, kH, kW)
            e_col = np.array([1, 1, pad, pad, iH, iW, 1, 1], dt)
            assert np.array_equal(gpu.transform(36, g, ci, ii, e_col), cpu.transform(36, c, ci, ii, e_col)), ("col2im", dt, kH, kW)
        # planes large enough for a channel's vectors to be spread over several blocks (two, and three)
        for (iH, iW, kH, kW, pad) in ((40, 44, 3, 3, 1), (56, 56, 3, 3, 1)):
            bS, iC = 8, 128
            oH, oW = iH + 2 * pad - kH + 1, iW + 2 * pad - kW + 1
            img, col = [bS, iC, iH, iW], [bS, iC, kH, kW, oH, oW]
            ii, ci = shape_info_np(img), shape_info_np(col)
            x = rs.randint(-8, 9, int(np.prod(img))).astype(dt)
            e_im = np.array([kH, kW, 1, 1, pad, pad, 1, 1, 0, 0], dt)
            assert np.array_equal(gpu.transform(37, x, ii, ci, e_im), cpu.transform(37, x, ii, ci, e_im)), ("im2col", dt, iH, iW)
        for iH, iW in ((56, 56), (9, 57), (10, 54), (7, 7)):
            img, pooled = [3, 5, iH, iW], [3, 5, iH // 2, iW // 2]
            ii, pi = shape_info_np(img), shape_info_np(pooled)
            x = rs.randint(-8, 9, int(np.prod(img))).astype(dt)
            for mode, p0 in ((0, 0.0), (1, 0.0), (1, 1.0), (1, 2.0), (2, 2.0), (3, 0.0)):
                e_pool = np.array([2, 2, 2, 2, 0, 0, 1, 1, 0, mode, p0], dt)
                gp, cp = gpu.transform(71, x, ii, pi, e_pool), cpu.transform(71, x, ii, pi, e_pool)
                if mode == 2:
                    assert np.allclose(gp.astype(np.float64), cp.astype(np.float64), rtol=1e-2 if dt == np.float16 else 1e-5), ("pooling", dt, iH, iW, mode)
                else:
                    assert np.array_equal(gp, cp, equal_nan=True), ("pooling", dt, iH, iW, mode, p0)


def test_whole_array_transforms_strided_form_and_errors(gpu, cpu):
    # the strided entry point runs the ops' per-element op(): identity, and softplus for the softmax family
    x = np.linspace(-3, 3, 257).astype(np.float32)
    for op in (36, 37, 48, 70, 71):
        assert np.array_equal(gpu.transform_strided(op, x, 1, 1, None, x.size), x), op
    for op in (38, 39, 40, 41):
        assert ulp_distance(gpu.transform_strided(op, x, 1, 1, None, x.size), cpu.transform_strided(op, x, 1, 1, None, x.size)).max() <= 2, op
    # arguments the whole-array routines cannot take are reported, not ignored
    vi = shape_info_np([1, 257])
    for op in (36, 37, 71):
        with pytest.raises(Exception):
            gpu.transform(op, x, vi, vi, np.zeros(11, np.float32))


def test_choice(gpu, cpu):
    checks.check_choice(gpu, cpu)
    # more results than probabilities without element-wise strides: the reference reads outside the probabilities;
    # the device refuses
    zi = harness.shape_info([5, 6], "c", strides=[1, 7])
    vi = shape_info_np([1, 4])
    g = gpu.rng(1, 64)
    with pytest.raises(Exception, match="Choice"):
        g.choice(np.arange(4, dtype=np.float32), vi, np.full(4, 0.25, np.float32), vi, zi)
    g.destroy()


def test_dropout_transforms(gpu):
    # DropOut 43 / DropOutInverted 44: the reference draws from an unseeded generator (rand() / the clock), so only the
    # distribution can be held to it: survivors keep x (or x / p), the rest is zero, about p of the elements survive,
    # and two calls do not drop the same elements
    n, p = 1 << 20, 0.3
    x = np.random.RandomState(3).uniform(1, 2, n).astype(np.float32)
    vi = shape_info_np([1, n])
    e = np.array([p, 0], np.float32)
    a, b = gpu.transform(43, x, vi, vi, e), gpu.transform(43, x, vi, vi, e)
    for z in (a, b):
        kept = z != 0
        assert np.array_equal(z[kept], x[kept])
        assert abs(kept.mean() - p) < 5 * np.sqrt(p * (1 - p) / n)
    both = ((a != 0) & (b != 0)).mean()
    assert abs(both - p * p) < 0.01, both
    inv = gpu.transform(44, x, vi, vi, e)
    kept = inv != 0
    assert np.array_equal(inv[kept], (x[kept] / np.float32(p)).astype(np.float32))
    assert abs(kept.mean() - p) < 5 * np.sqrt(p * (1 - p) / n)
    # a strided view: nothing outside it is written, and the strided entry point takes the same ops
    xi = harness.shape_info([64, 50], "c", strides=[100, 2])
    xs = np.ones(harness.span_of(xi), np.float32)
    z = gpu.transform(43, xs, xi, xi, e)
    sel = harness.element_offsets(xi)
    assert np.all(np.delete(z, sel) == 0) and 0.2 < (z[sel] != 0).mean() < 0.4
    z = gpu.transform_strided(44, xs, 2, 3, e, 1000)
    assert np.all(np.delete(z, np.arange(1000) * 3) == 0) and 0.2 < (z[::3] != 0).mean() < 0.4


def test_debug_and_verbose_mode_print_the_launches(gpu, capfd):
    x = np.linspace(-1, 1, 1000).astype(np.float32)
    vi = shape_info_np([1, 1000])
    gpu.ops.enableDebugMode(True)
    gpu.ops.enableVerboseMode(True)
    try:
        got = gpu.transform(0, x, vi, vi)
        total = gpu.reduce_scalar(1, np.ones(1000, np.float32), vi)
    finally:
        gpu.ops.enableDebugMode(False)
        gpu.ops.enableVerboseMode(False)
    out = capfd.readouterr().out
    assert np.array_equal(got, np.abs(x)) and float(total) == 1000.0
    assert "Launch:" in out and "ewVecKernel" in out and "flatKernel" in out and "gridSize" in out
    gpu.transform(0, x, vi, vi)
    assert "Launch:" not in capfd.readouterr().out


def test_softmax_of_long_rows_cooperating_blocks(gpu, cpu):
    # contiguous, 16-byte aligned rows too long for one block's registers: the blocks that hold the slices of a row
    # exchange maxima and sums.  Checked against float64 and the CPU checker, out of place and in place, for the three
    # ops and types; then again with the blocks' patience set to zero from the host, so that every row whose slices are
    # not all there at the first look is aborted and computed by the repair kernel - same results.
    rs = np.random.RandomState(37)

    def run(limit):
        gpu.ops.amd_setCooperativeWaitLimit(limit)
        for shape, dt in (([6, 40000], np.float32), ([1, 300001], np.float32), ([700, 8192 + 4 * 7], np.float32),
                          ([3, 16384 * 3 + 8], np.float16), ([5, 20002], np.float64), ([40, 262144], np.float32),
                          # rows of odd length: every row starts at another distance from a 16-byte boundary
                          ([33, 50257], np.float32), ([7, 20001], np.float16), ([9, 9001], np.float64)):
            n = shape[0] * shape[1]
            info = harness.shape_info(shape, "c")
            x = rs.uniform(-6, 6, n).astype(dt)
            rows = x.astype(np.float64).reshape(shape)
            truth = np.exp(rows - rows.max(axis=1, keepdims=True))
            truth /= truth.sum(axis=1, keepdims=True)
            rtol = {np.float32: 2e-5, np.float16: 1e-2, np.float64: 1e-12}[dt]
            atol = {np.float32: 1e-7, np.float16: 1e-4, np.float64: 1e-300}[dt]
            for op, f in ((38, lambda v: v), (39, lambda v: v * (1 - v)), (40, np.log)):
                got = gpu.transform(op, x, info, info).astype(np.float64).reshape(shape)
                assert np.all(np.abs(got - f(truth)) <= rtol * np.abs(f(truth)) + atol), (shape, dt, op, limit)
                inplace = gpu.transform_inplace(op, x, info).astype(np.float64).reshape(shape)
                if limit > 0:
                    assert np.array_equal(inplace, got), (shape, dt, op, limit, "in place")
                else:
                    # with no patience, which rows the slow kernel redoes (it sums in another order) is a matter of timing
                    assert np.all(np.abs(inplace - f(truth)) <= rtol * np.abs(f(truth)) + atol), (shape, dt, op, limit, "in place")
            if dt == np.float32 and n <= 300001:
                c = cpu.transform(38, x, info, info)
                assert np.all(np.abs(gpu.transform(38, x, info, info).astype(np.float64) - c) <= 1e-5 * np.abs(c) + 1e-7)

    try:
        run(5000)
        run(0)
    finally:
        gpu.ops.amd_setCooperativeWaitLimit(5000)


def test_softmax_of_f_order_matrices_cooperating_blocks(gpu, cpu):
    # f-order matrices with more columns than one block keeps of a group of rows: the blocks that share a group's columns
    # exchange the rows' maxima and sums.  Against float64, out of place and in place, the three ops and types, ragged
    # last groups and last slices; then with no patience, so that the repair kernel does what was not there at once.
    rs = np.random.RandomState(41)

    def run(limit):
        gpu.ops.amd_setCooperativeWaitLimit(limit)
        for shape, dt in (([512, 2048], np.float32), ([260, 1500], np.float32), ([1024, 5001], np.float32),
                          ([512, 1100], np.float16), ([264, 3000], np.float64), ([4100, 1025], np.float32)):
            info = harness.shape_info(shape, "f")
            a = rs.uniform(-6, 6, shape).astype(dt)
            x = np.ascontiguousarray(a.flatten(order="F"))
            rows = a.astype(np.float64)
            truth = np.exp(rows - rows.max(axis=1, keepdims=True))
            truth /= truth.sum(axis=1, keepdims=True)
            rtol = {np.float32: 2e-5, np.float16: 1e-2, np.float64: 1e-12}[dt]
            atol = {np.float32: 1e-7, np.float16: 1e-4, np.float64: 1e-300}[dt]
            for op, f in ((38, lambda v: v), (39, lambda v: v * (1 - v)), (40, np.log)):
                got = gpu.transform(op, x, info, info).astype(np.float64).reshape(shape, order="F")
                assert np.all(np.abs(got - f(truth)) <= rtol * np.abs(f(truth)) + atol), (shape, dt, op, limit)
                inplace = gpu.transform_inplace(op, x, info).astype(np.float64).reshape(shape, order="F")
                if limit > 0:
                    assert np.array_equal(inplace, got), (shape, dt, op, limit, "in place")
                else:
                    assert np.all(np.abs(inplace - f(truth)) <= rtol * np.abs(f(truth)) + atol), (shape, dt, op, limit, "in place")
            if dt == np.float32 and shape[0] * shape[1] <= 1 << 20:
                c = cpu.transform(38, x, info, info)
                assert np.all(np.abs(gpu.transform(38, x, info, info).astype(np.float64) - c) <= 1e-5 * np.abs(c) + 1e-7)

    try:
        run(5000)
        run(0)
    finally:
        gpu.ops.amd_setCooperativeWaitLimit(5000)


def test_reductions_over_generated_shapes(gpu):
    # Sum / Mean / Max, IndexMax, bias-corrected variance and the scalar-returning calls over generated matrices whose
    # extents sit on and around the sizes where the reduction kernels change (lanes per TAD, slices of long TADs, vector
    # widths, the whole-array grid), both orders, three types, along either dimension or both, with and without the
    # caller's TAD tables: against float64.
    rs = np.random.RandomState(59)
    sizes = [1, 2, 3, 7, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1000, 1023, 1024, 1025, 2048, 4095, 4096,
             4100, 8192, 16383, 16384, 16385, 20000, 65536, 100003, 262144, 1 << 20, (1 << 20) + 3]
    for it in range(200):
        rows, cols = int(rs.choice(sizes)), int(rs.choice(sizes))
        while rows * cols > (4 << 20):
            if rows > cols:
                rows = int(rs.choice([v for v in sizes if v < rows]))
            else:
                cols = int(rs.choice([v for v in sizes if v < cols]))
        order = "c" if rs.rand() < 0.5 else "f"
        dt = [np.float32, np.float32, np.float64, np.float16][int(rs.randint(0, 4))]
        shape = [rows, cols]
        info = harness.shape_info(shape, order)
        a = rs.uniform(-1, 1, shape).astype(dt) if dt == np.float16 else rs.uniform(-3, 3, shape).astype(dt)
        memory_order = "F" if order == "f" else "C"
        x = np.ascontiguousarray(a.flatten(order=memory_order))
        a64 = a.astype(np.float64)
        which = int(rs.randint(0, 4))
        dims = [[0], [1], [0, 1]][int(rs.randint(0, 3))]
        pass_tads = bool(rs.randint(0, 2))
        axis = tuple(dims)
        out_len = int(np.prod([shape[d] for d in range(2) if d not in dims])) if len(dims) < 2 else 1
        rtol = {np.float32: 2e-5, np.float64: 1e-12, np.float16: 2e-2}[dt]
        tag = (shape, order, dt.__name__, which, dims, pass_tads)
        if which == 0:
            op = int(rs.choice([0, 1, 3]))
            got = gpu.reduce(op, x, info, None, dims, out_len, pass_tads=pass_tads).astype(np.float64)
            want = {0: a64.mean(axis=axis), 1: a64.sum(axis=axis), 3: a64.max(axis=axis)}[op].reshape(-1)
            scale = np.abs(a64).sum(axis=axis).reshape(-1) if op != 3 else np.abs(want)
            if op == 0:
                scale = scale / np.prod([shape[d] for d in dims])
            if dt == np.float16 and op != 3 and np.abs(want).max() > 60000:
                continue
            assert np.all(np.abs(got - want) <= rtol * scale + 1e-30), tag
        elif which == 1:
            if (dt == np.float16 and rows * cols > 2000) or len(dims) == 2 and order == "f":
                continue
            perm = rs.permutation(rows * cols).astype(dt)  # distinct values: no ties to resolve
            got = gpu.indexreduce(0, perm, info, None, dims, out_len, pass_tads=pass_tads).astype(np.int64)
            p2 = perm.reshape(shape, order=memory_order).astype(np.float64)
            want = np.array([int(np.argmax(p2.reshape(-1)))]) if len(dims) == 2 else p2.argmax(axis=dims[0]).reshape(-1)
            assert np.array_equal(got, want), tag
        elif which == 2:
            if dt == np.float16 or int(np.prod([shape[d] for d in dims])) < 2:
                continue
            got = gpu.summarystats(0, True, x, info, dims, out_len, pass_tads=pass_tads).astype(np.float64)
            want = a64.var(axis=axis, ddof=1).reshape(-1)
            assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-12), tag
        else:
            op = int(rs.choice([0, 1, 3]))
            got = float(gpu.reduce_scalar(op, x, info))
            want = {0: a64.mean(), 1: a64.sum(), 3: a64.max()}[op]
            scale = np.abs(a64).sum() if op == 1 else (np.abs(a64).mean() if op == 0 else abs(want))
            if dt == np.float16 and op == 1 and abs(want) > 60000:
                continue
            assert abs(got - want) <= rtol * scale + 1e-30, tag


def test_softmax_family_over_generated_shapes(gpu):
    # SoftMax / SoftMaxDerivative / LogSoftMax over generated matrices whose row lengths sit on and around the sizes where
    # the kernels change (16, 64, 256, 1024, 2048, 8192, 16384, 65536 columns; few and many rows), both orders, three types,
    # in place or not, now and then with the cooperative kernels' patience at zero: against float64.
    rs = np.random.RandomState(53)
    col_choices = [2, 3, 15, 16, 17, 63, 64, 65, 255, 256, 257, 1000, 1023, 1024, 1025, 1026, 1500, 2047, 2048, 2049, 2052, 3000, 4096,
                   4100, 5001, 8191, 8192, 8193, 8200, 10000, 16383, 16384, 16388, 20000, 32768, 50257, 65536, 65540, 100003, 300001]
    row_choices = [1, 2, 3, 4, 7, 8, 31, 32, 33, 64, 100, 255, 256, 257, 260, 264, 300, 512, 1000, 1024, 2048, 4100]
    try:
        for it in range(160):
            cols = int(rs.choice(col_choices))
            rows = min(int(rs.choice(row_choices)), max(1, (4 << 20) // cols))
            order = "c" if rs.rand() < 0.5 else "f"
            dt = [np.float32, np.float32, np.float16, np.float64][int(rs.randint(0, 4))]
            op = int(rs.choice([38, 39, 40]))
            limit = 5000 if rs.rand() < 0.8 else 0
            gpu.ops.amd_setCooperativeWaitLimit(limit)
            shape = [rows, cols]
            info = harness.shape_info(shape, order)
            a = rs.uniform(-6, 6, shape).astype(dt)
            memory_order = "F" if order == "f" else "C"
            x = np.ascontiguousarray(a.flatten(order=memory_order))
            r64 = a.astype(np.float64)
            truth = np.exp(r64 - r64.max(axis=1, keepdims=True))
            truth /= truth.sum(axis=1, keepdims=True)
            want = {38: lambda v: v, 39: lambda v: v * (1 - v), 40: np.log}[op](truth)
            rtol = {np.float32: 3e-5, np.float16: 2e-2, np.float64: 1e-11}[dt]
            atol = {np.float32: 2e-7, np.float16: 2e-4, np.float64: 1e-300}[dt]
            in_place = rs.rand() < 0.4
            got = gpu.transform_inplace(op, x, info) if in_place else gpu.transform(op, x, info, info)
            got = got.astype(np.float64).reshape(shape, order=memory_order)
            assert np.all(np.abs(got - want) <= rtol * np.abs(want) + atol), (shape, order, dt, op, limit, in_place)
    finally:
        gpu.ops.amd_setCooperativeWaitLimit(5000)


def test_half_families(gpu, cpu):
    rs = np.random.RandomState(28)
    h = np.float16
    R, C = 64, 96
    x = rs.randn(R * C).astype(h)
    y = rs.randn(R * C).astype(h)
    xi = shape_info_np([R, C])

    def close(g, c, what):
        g64, c64 = g.astype(np.float64), c.astype(np.float64)
        assert np.all(np.abs(g64 - c64) <= 1e-2 * np.maximum(np.abs(c64), 1e-2)), what

    for op in (0, 6, 9):
        close(gpu.pairwise(op, x, xi, y, xi, xi), cpu.pairwise(op, x, xi, y, xi, xi), "half pairwise %d" % op)
    for op in (15, 3, 10):
        close(gpu.transform(op, x, xi, xi), cpu.transform(op, x, xi, xi), "half transform %d" % op)
    row = rs.randn(C).astype(h)
    close(gpu.broadcast(0, x, xi, row, shape_info_np([1, C]), xi, [1]), cpu.broadcast(0, x, xi, row, shape_info_np([1, C]), xi, [1]), "half broadcast")
    # reductions: the reference accumulates in fp16, this path in fp32; compare with the exact value instead
    exact = x.astype(np.float64).reshape(R, C)
    g = gpu.reduce(1, x, xi, None, [1], R).astype(np.float64)
    assert np.all(np.abs(g - exact.sum(axis=1)) <= 1e-2 * np.maximum(np.abs(exact.sum(axis=1)), 1.0))
    assert np.array_equal(gpu.reduce(3, x, xi, None, [0], C), exact.max(axis=0).astype(h))
    assert np.array_equal(gpu.indexreduce(0, x, xi, None, [1], R), np.argmax(exact, axis=1).astype(h))
    g = gpu.summarystats(0, 1, x, xi, [0], C).astype(np.float64)
    assert np.all(np.abs(g - exact.var(axis=0, ddof=1)) <= 1e-2 * exact.var(axis=0, ddof=1))
    # wide enough for the kernel that gives each lane eight adjacent strided TADs
    R2, C2 = 200, 2056
    x2 = rs.randn(R2 * C2).astype(h)
    e2 = x2.astype(np.float64).reshape(R2, C2)
    xi2 = shape_info_np([R2, C2])
    assert np.array_equal(gpu.reduce(3, x2, xi2, None, [0], C2), e2.max(axis=0).astype(h))
    assert np.array_equal(gpu.indexreduce(1, x2, xi2, None, [0], C2), np.argmin(e2, axis=0).astype(h))
    g = gpu.reduce(1, x2, xi2, None, [0], C2).astype(np.float64)
    assert np.all(np.abs(g - e2.sum(axis=0)) <= 1e-2 * np.maximum(np.abs(e2.sum(axis=0)), 1.0))
    # NaN is stored as 0x7fff
    nan_in = np.array([np.nan, 1.0], h)
    out = gpu.transform(6, nan_in, shape_info_np([1, 2]), shape_info_np([1, 2]))
    assert out.view(np.uint16)[0] == 0x7fff


def test_half_reductions_against_the_reference_loops(gpu, cpu):
    """The reference's float16 reductions accumulate in fp16; this path in fp32.  On TADs short enough for the fp16
    accumulation to stay inside the bar the two are compared directly, 1e-2, over several shapes and dimensions."""
    rs = np.random.RandomState(29)
    h = np.float16
    for shape, dims in (([40, 16], [1]), ([16, 40], [0]), ([6, 12, 5], [1]), ([8, 3, 6], [0, 2]), ([5, 24], [1])):
        n = int(np.prod(shape))
        x = (0.5 + rs.rand(n)).astype(h)
        info = shape_info_np(shape)
        out_len = n // int(np.prod([shape[d] for d in dims]))
        for op in (0, 1, 3, 5, 6):
            g = gpu.reduce(op, x, info, None, dims, out_len).astype(np.float64)
            c = cpu.reduce(op, x, info, None, dims, out_len).astype(np.float64)
            assert np.all(np.abs(g - c) <= 1e-2 * np.abs(c)), (shape, dims, op, np.abs(g - c).max())
        assert np.array_equal(gpu.indexreduce(0, x, info, None, dims, out_len), cpu.indexreduce(0, x, info, None, dims, out_len)), (shape, dims)
        for op in (0, 1):
            g = gpu.summarystats(op, 1, x, info, dims, out_len).astype(np.float64)
            c = cpu.summarystats(op, 1, x, info, dims, out_len).astype(np.float64)
            assert np.all(np.abs(g - c) <= 1e-2 * np.abs(c)), (shape, dims, op, "stats")


def test_slot_tickets_across_the_points_where_the_slots_are_cleared(gpu):
    """Whole-array reductions, strided reductions that finish in one launch, the whole-array reduce3 and the cooperative
    softmax kernels tag what their blocks exchange with a per-stream launch ticket (30 bits of it for the softmax), and the exchange area is not cleared between launches.
    Data set A is run on the tickets just behind a multiple of 2^30; then the counter is put back to just before that
    multiple - where a long-running process arrives 2^30 launches later - and data set B is run: it draws the same tickets
    again, and must not see what A left behind (the library clears the area when the counter nears the boundary)."""
    rs = np.random.RandomState(41)
    n = 1 << 20
    xi = shape_info_np([1, n])
    rows = shape_info_np([4, 40000])
    square = shape_info_np([1024, 1024])
    ex = gpu.dev.extra(xi)

    def data():
        x, y = rs.randn(n).astype(np.float32), rs.randn(n).astype(np.float32)
        xr = rs.uniform(-5, 5, 4 * 40000).astype(np.float32)
        r64 = xr.astype(np.float64).reshape(4, 40000)
        soft = np.exp(r64 - r64.max(axis=1, keepdims=True))
        return x, y, xr, soft / soft.sum(axis=1, keepdims=True)

    def run(d, what):
        x, y, xr, soft = d
        total, dot = x.astype(np.float64).sum(), (x.astype(np.float64) * y).sum()
        scale = np.abs(x).astype(np.float64).sum() / np.sqrt(n)
        columns = x.astype(np.float64).reshape(1024, 1024).sum(axis=0)
        column_scale = np.abs(x).astype(np.float64).reshape(1024, 1024).sum(axis=0)
        for k in range(6):
            got = gpu.reduce(1, x, square, None, [0], 1024).astype(np.float64)
            assert np.all(np.abs(got - columns) <= 1e-5 * column_scale), (what, k)
            assert abs(float(gpu.reduce_scalar(1, x, xi)) - total) <= 1e-5 * max(abs(total), scale), (what, k)
            assert float(gpu.indexreduce_scalar(0, x, xi)) == float(np.argmax(x)), (what, k)
            assert abs(float(gpu.reduce3_scalar(3, x, xi, y, xi)) - dot) <= 1e-4 * np.sqrt(n), (what, k)
            got = gpu.transform(38, xr, rows, rows).astype(np.float64).reshape(4, 40000)
            assert np.all(np.abs(got - soft) <= 2e-5 * soft + 1e-30), (what, k)

    a, b = data(), data()
    try:
        for boundary in (0x40000000, 0x80000000, 0):
            gpu.ops.amd_setSlotTicket(ex, boundary)
            run(a, ("A", hex(boundary)))
            gpu.ops.amd_setSlotTicket(ex, (boundary - 16) & 0xffffffff)
            run(b, ("B", hex(boundary)))
    finally:
        gpu.ops.amd_setSlotTicket(ex, 5)


def test_elementwise_calls_in_a_captured_graph(gpu):
    """A pairwise add, an exp transform and a row broadcast are captured into a HIP graph on the caller's stream (after one
    eager pass, which lets the stream allocate what it keeps) and replayed three times with new operand values, eager
    work and synchronisations in between; every replay must give the bits of the same three calls made eagerly."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    dev, ops = gpu.dev, gpu.dev.ops
    rs = np.random.RandomState(91)
    rows, cols = 300, 1024
    n = rows * cols
    xi, bi = shape_info_np([rows, cols]), shape_info_np([1, cols])
    tad = dev.tad(xi, [1])
    X = harness.Operand(dev, rs.uniform(-2, 2, n).astype(np.float32), xi)
    Y = harness.Operand(dev, rs.uniform(-2, 2, n).astype(np.float32), xi)
    B = harness.Operand(dev, rs.uniform(-2, 2, cols).astype(np.float32), bi)
    outs = [[harness.Operand(dev, np.zeros(n, np.float32), xi) for _ in range(3)] for _ in range(2)]  # graph, eager
    dim = dev.upload(np.array([1], np.int32))
    ex = dev.extra(xi, xi, xi)
    exb = dev.extra(xi, bi, xi, tad=tad, tad_z=tad)

    def calls(o):
        ops.execPairwiseTransformFloat(ex, 0, X.ptr, X.info_ptr, Y.ptr, Y.info_ptr, o[0].ptr, o[0].info_ptr, None)
        ops.execTransformFloat(ex, 3, o[0].ptr, o[0].info_ptr, o[1].ptr, o[1].info_ptr, None)
        ops.execBroadcastFloat(exb, 0, o[1].ptr, o[1].info_ptr, B.ptr, B.info_ptr, o[2].ptr, o[2].info_ptr, dim.ptr, 1)

    calls(outs[1])
    dev.sync()
    stream = ctypes.c_void_p(dev.stream)
    graph, executable = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 1) == 0  # 1: thread-local capture mode
    try:
        calls(outs[0])
    finally:
        status = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
    assert status == 0 and graph.value
    assert hip.hipGraphInstantiate(ctypes.byref(executable), graph, None, None, ctypes.c_size_t(0)) == 0
    try:
        for replay in range(3):
            fresh = rs.uniform(-2, 2, n).astype(np.float32)
            ops.memcpy(X.ptr, fresh.ctypes.data, fresh.nbytes, 1, None)
            dev.sync()
            assert hip.hipGraphLaunch(executable, stream) == 0
            dev.sync()
            calls(outs[1])
            dev.sync()
            e = np.exp((fresh + Y.get()).astype(np.float64)).reshape(rows, cols)
            b = B.get().astype(np.float64)
            for k in range(3):
                assert np.array_equal(outs[0][k].get(), outs[1][k].get()), (replay, k)
            assert np.all(np.abs(outs[0][2].get().reshape(rows, cols) - (e + b)) <= 1e-5 * (e + np.abs(b))), replay
    finally:
        hip.hipGraphExecDestroy(executable)
        hip.hipGraphDestroy(graph)
        for o in [X, Y, B] + outs[0] + outs[1]:
            o.free()
        dim.free()


def test_reductions_in_a_captured_graph(gpu):
    """Calls whose blocks exchange partial results (sums along the strided dimension, the whole-array sum left on the
    device, argmax along dimension 0, SoftMax over long rows) keep their launches apart by tickets drawn on the host, which a
    graph would replay; on a stream under capture they take their two-launch forms instead.  Captured after one eager pass,
    replayed three times with new values: every replay against float64 numpy (1e-5; indices exactly)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    dev, ops = gpu.dev, gpu.dev.ops
    rs = np.random.RandomState(92)
    rows, cols = 4096, 512
    n = rows * cols
    xi = shape_info_np([rows, cols])
    li = shape_info_np([8, n // 8])  # the same buffer as eight long rows
    X = harness.Operand(dev, rs.uniform(0.5, 1.5, n).astype(np.float32), xi)
    XL = harness.Operand(dev, np.zeros(n, np.float32), li)
    ci, ri, si = shape_info_np([1, cols]), shape_info_np([1, rows]), shape_info_np([1, 1])
    S0, M1, A0 = (harness.Operand(dev, np.zeros(cols, np.float32), ci), harness.Operand(dev, np.zeros(rows, np.float32), ri),
                  harness.Operand(dev, np.zeros(cols, np.float32), ci))
    F = harness.Operand(dev, np.zeros(1, np.float32), si)
    P = harness.Operand(dev, np.zeros(n, np.float32), li)
    d0, d1 = dev.upload(np.array([0], np.int32)), dev.upload(np.array([1], np.int32))
    ex0 = dev.extra(xi, z_info=ci, tad=dev.tad(xi, [0]))
    ex1 = dev.extra(xi, z_info=ri, tad=dev.tad(xi, [1]))
    exf = dev.extra(xi, z_info=si)
    exl = dev.extra(li, z_info=li, tad=dev.tad(li, [1]))  # (with the row tables a host passes: building them would allocate)

    def calls():
        ops.execReduceFloat(ex0, 1, X.ptr, X.info_ptr, None, S0.ptr, S0.info_ptr, d0.ptr, 1)
        ops.execReduceFloat(ex1, 3, X.ptr, X.info_ptr, None, M1.ptr, M1.info_ptr, d1.ptr, 1)
        ops.execIndexReduceFloat(ex0, 0, X.ptr, X.info_ptr, None, A0.ptr, A0.info_ptr, d0.ptr, 1)
        ops.execReduceFloatFull(exf, 1, X.ptr, X.info_ptr, None, F.ptr, F.info_ptr)
        ops.execTransformFloat(exl, 38, X.ptr, XL.info_ptr, P.ptr, P.info_ptr, None)

    def check(values, what):
        v = values.astype(np.float64).reshape(rows, cols)
        close = lambda g, e: np.all(np.abs(g.astype(np.float64) - e) <= 1e-5 * np.abs(e) + 1e-12)
        assert close(S0.get(), v.sum(axis=0)), (what, "sum along dimension 0")
        assert np.array_equal(M1.get(), values.reshape(rows, cols).max(axis=1)), (what, "max along dimension 1")
        assert np.array_equal(A0.get(), np.argmax(v, axis=0).astype(np.float32)), (what, "argmax along dimension 0")
        assert close(F.get(), np.array([v.sum()])), (what, "whole-array sum")
        long = values.astype(np.float64).reshape(8, n // 8)
        e = np.exp(long - long.max(axis=1, keepdims=True))
        assert np.all(np.abs(P.get().reshape(8, n // 8) - e / e.sum(axis=1, keepdims=True)) <= 1e-5 * e / e.sum(axis=1, keepdims=True) + 1e-12), (what, "softmax")

    first = X.get().copy()
    calls()
    dev.sync()
    check(first, "eager")
    stream = ctypes.c_void_p(dev.stream)
    graph, executable = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 1) == 0  # 1: thread-local capture mode
    try:
        calls()
    finally:
        status = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
    assert status == 0 and graph.value
    assert hip.hipGraphInstantiate(ctypes.byref(executable), graph, None, None, ctypes.c_size_t(0)) == 0
    try:
        for replay in range(3):
            fresh = rs.uniform(0.5, 1.5, n).astype(np.float32)
            ops.memcpy(X.ptr, fresh.ctypes.data, fresh.nbytes, 1, None)
            for o in (S0, M1, A0, F):
                ops.memset(o.ptr, 0, 4, 0, None)
            dev.sync()
            assert hip.hipGraphLaunch(executable, stream) == 0
            dev.sync()
            check(fresh, ("replay", replay))
            calls()  # eager work between the replays, on its one-launch paths
            dev.sync()
            check(fresh, ("eager after replay", replay))
    finally:
        hip.hipGraphExecDestroy(executable)
        hip.hipGraphDestroy(graph)
        for o in (X, XL, S0, M1, A0, F, P, d0, d1):
            o.free()


def test_releasing_a_streams_resources(gpu):
    """A stream's workspace, exchange slots and pinned scalar block are freed on request and come back at the next call."""
    rs = np.random.RandomState(43)
    x = rs.randn(1 << 18).astype(np.float32)
    xi = shape_info_np([512, 512])
    want = x.astype(np.float64).reshape(512, 512)
    for _ in range(3):
        assert abs(float(gpu.reduce_scalar(1, x, xi)) - want.sum()) <= 1e-5 * np.abs(want).sum()
        assert np.array_equal(gpu.reduce(3, x, xi, None, [0], 512), want.max(axis=0).astype(np.float32))
        gpu.ops.amd_releaseStream(gpu.dev.stream)
    gpu.ops.amd_releaseStream(gpu.dev.stream)  # nothing left to free: a no-op


def test_double_family_smoke(gpu, cpu):
    rs = np.random.RandomState(29)
    x = rs.randn(1000).astype(np.float64)
    xi = shape_info_np([10, 100])
    g, c = gpu.transform(15, x, xi, xi), cpu.transform(15, x, xi, xi)
    assert np.allclose(g, c, rtol=1e-14, atol=0)
    assert np.allclose(gpu.reduce(1, x, xi, None, [1], 10), cpu.reduce(1, x, xi, None, [1], 10), rtol=1e-13)
    assert float(gpu.indexreduce_scalar(0, x, xi)) == float(cpu.indexreduce_scalar(0, x, xi))
    x = rs.randn(300 * 600).astype(np.float64)
    xi = shape_info_np([300, 600])
    assert np.allclose(gpu.reduce(1, x, xi, None, [0], 600), cpu.reduce(1, x, xi, None, [0], 600), rtol=1e-13)
    assert np.array_equal(gpu.indexreduce(0, x, xi, None, [0], 600), cpu.indexreduce(0, x, xi, None, [0], 600))
    assert np.allclose(gpu.summarystats(0, 1, x, xi, [0], 600), cpu.summarystats(0, 1, x, xi, [0], 600), rtol=1e-12)


def test_random_ops_against_cpu(gpu, cpu):
    for seed, size, pre in ((119, 1 << 12, 0), (3, 777, 5000), (-11, 64, 63)):
        a, b = gpu.rng(seed, size), cpu.rng(seed, size)
        a.rewind(pre)
        b.rewind(pre)
        assert a.state() == b.state()
        assert np.array_equal(a.elements(0, 5000), b.elements(0, 5000))
        a.reseed(424242)
        b.reseed(424242)
        assert np.array_equal(a.elements(100, 3000), b.elements(100, 3000))
        for op, args in ((0, [0, 1]), (0, [-1, 3]), (7, [0.4]), (4, [2, 5]), (13, [0.7])):
            assert ulp_distance(a.random_z(op, 1001, args), b.random_z(op, 1001, args)).max() <= (2 if op == 13 else 0), op
            assert a.state() == b.state()
        x = np.linspace(-2, 2, 999).astype(np.float32)
        for op, args in ((1, [0.5]), (2, [0.3]), (7, [0]), (12, [0.5, 1.1, 0.2, -1.7]), (13, [2.0])):
            assert ulp_distance(a.random_xz(op, x, args), b.random_xz(op, x, args)).max() <= (2 if op == 13 else 0), op
        for op, args in ((6, [1.5, 2.0]), (10, [0.1, 0.3]), (11, [0.0, 1.0]), (8, [3, 0.5]), (9, [2, 0.7])):
            g = a.random_xyz(op, None, None, args, mode="inplace_all", n=777)
            c = b.random_xyz(op, None, None, args, mode="inplace_all", n=777)
            assert ulp_distance(g, c).max() <= 2, op
            assert a.state() == b.state(), op
        y = np.linspace(0, 1, 999).astype(np.float32)
        assert np.array_equal(a.random_xyz(3, x, y, [0.5]), b.random_xyz(3, x, y, [0.5]))
        assert ulp_distance(a.random_xyz(6, x, y, [0, 0.5]), b.random_xyz(6, x, y, [0, 0.5])).max() <= 2
        a.refresh(99)
        b.refresh(99)
        assert a.state() == b.state() and np.array_equal(a.elements(0, 300), b.elements(0, 300))
        a.destroy()
        b.destroy()


def test_random_blocks_across_the_ends_of_the_buffer(gpu, cpu):
    # Draws far longer than the buffer, whose size is no multiple of what a block takes: blocks straddle the buffer's end,
    # where the generation (and with it the divisor of the first shift) changes inside a block; started at several
    # positions, after a reseed too.  Uniform and dropout bit for bit, Gaussian within 2 ULP.
    n = 50000
    x = np.linspace(-2, 2, n).astype(np.float32)
    for seed, size, pre in ((7, 1000, 0), (8, 4099, 123456), (9, 10000, 9999), (10, 300, 77)):
        a, b = gpu.rng(seed, size), cpu.rng(seed, size)
        a.rewind(pre)
        b.rewind(pre)
        for round_ in range(2):
            assert np.array_equal(a.random_z(0, n, [-1, 3]), b.random_z(0, n, [-1, 3])), (size, pre, round_)
            assert np.array_equal(a.random_xz(1, x, [0.5]), b.random_xz(1, x, [0.5])), (size, pre, round_)
            g = a.random_xyz(6, None, None, [0.5, 2.0], mode="inplace_all", n=n - 1)
            c = b.random_xyz(6, None, None, [0.5, 2.0], mode="inplace_all", n=n - 1)
            assert ulp_distance(g, c).max() <= 2, (size, pre, round_)
            assert a.state() == b.state()
            a.reseed(31337)
            b.reseed(31337)
        a.destroy()
        b.destroy()


def test_random_on_strided_output(gpu, cpu):
    # a non-EWS output is filled in Fortran order of its shape (the reference's ind2sub branch)
    zi = harness.shape_info([7, 9], "f")  # EWS -1
    a, b = gpu.rng(5, 128), cpu.rng(5, 128)
    assert np.array_equal(a.random_z(0, zi, [0, 1]), b.random_z(0, zi, [0, 1]))
    assert a.state() == b.state()
    a.destroy()
    b.destroy()


def test_concurrent_callers_on_their_own_streams():
    """The reference's entry points are re-entrant: nd4j calls them from many threads, each with its own stream and
    scratch (blas/cuda/NativeOps.cu:1609-1624).  Four threads with a stream each hammer the calls that touch the
    library's shared state - the TAD cache (no caller tables), the per-stream workspace (which has to grow for the
    long rows) and the pinned scalar slot - and every result is checked."""
    import threading

    errors = []

    def worker(seed):
        try:
            be = backends.GpuBackend()
            rs = np.random.RandomState(seed)
            rows, cols = 48 + seed, 96
            info = shape_info_np([rows, cols])
            long_info = shape_info_np([3, 40000])
            for it in range(12):
                x = rs.randn(rows * cols).astype(np.float32)
                m = x.reshape(rows, cols).astype(np.float64)
                got = be.reduce(1, x, info, None, [1], rows, pass_tads=False)
                assert np.allclose(got, m.sum(axis=1), rtol=1e-5, atol=1e-5), "sum dim1"
                got = be.reduce(3, x, info, None, [0], cols, pass_tads=False)
                assert np.array_equal(got, x.reshape(rows, cols).max(axis=0)), "max dim0"
                assert abs(float(be.reduce_scalar(1, x, info)) - m.sum()) <= 1e-4 * np.abs(m).sum(), "sum"
                assert float(be.indexreduce_scalar(0, x, info)) == float(np.argmax(x)), "argmax"
                y = rs.randn(3 * 40000).astype(np.float32)
                sm = be.transform(38, y, long_info, long_info).astype(np.float64).reshape(3, 40000)
                rows64 = y.astype(np.float64).reshape(3, 40000)
                truth = np.exp(rows64 - rows64.max(axis=1, keepdims=True))
                truth /= truth.sum(axis=1, keepdims=True)
                assert np.all(np.abs(sm - truth) <= 2e-5 * truth + 1e-30), "softmax"
                assert np.array_equal(be.pairwise(0, x, info, x, info, info), x + x), "add"
        except BaseException as e:  # noqa: B036 - reported by the main thread
            errors.append((seed, repr(e)))

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a caller did not finish"
    assert errors == []


def test_random_views_against_the_cpu_checker(gpu, cpu):
    """Generated shapes, strides and dimensions through every loop family (tests/checks.py: check_random_views), with and
    without the caller's TAD tables.  Fixed seed: the same few thousand calls every run."""
    done = checks.check_random_views(gpu, cpu, seed=7, cases=4000)
    assert len(done) == 8 and min(done.values()) > 200
    # the other two storage types: vectors of two and of eight elements through the same kernels
    done = checks.check_random_views(gpu, cpu, seed=8, cases=1200, dtype=np.float64)
    assert len(done) == 8 and min(done.values()) > 50
    done = checks.check_random_views(gpu, cpu, seed=9, cases=1200, dtype=np.float16)
    assert len(done) == 5 and min(done.values()) > 50


def test_dense_matrices_in_mixed_orders(gpu):
    """z = op(x, y) over dense matrices whose orders differ (a + b.transpose()): every combination of c and f for x, y
    and z, shapes that allow 16-byte accesses and shapes that do not, all three data types.  Add and Abs are single IEEE
    operations, so numpy gives the expected bits."""
    rs = np.random.RandomState(77)
    for dt in (np.float32, np.float16, np.float64):
        for shape in ([128, 256], [96, 40], [33, 65], [64, 7]):
            n = shape[0] * shape[1]
            a, b = rs.randn(*shape).astype(dt), rs.randn(*shape).astype(dt)
            for ox, oy, oz in itertools.product("cf", repeat=3):
                if ox == oy == oz:
                    continue
                xi, yi, zi = (harness.shape_info(shape, o) for o in (ox, oy, oz))
                x = np.ascontiguousarray(a if ox == "c" else a.T).ravel()
                y = np.ascontiguousarray(b if oy == "c" else b.T).ravel()
                got = gpu.pairwise(0, x, xi, y, yi, zi).reshape(shape, order="F" if oz == "f" else "C")
                assert np.array_equal(got, a + b), (np.dtype(dt).name, shape, ox, oy, oz)
            for ox, oz in (("c", "f"), ("f", "c")):
                xi, zi = harness.shape_info(shape, ox), harness.shape_info(shape, oz)
                x = np.ascontiguousarray(a if ox == "c" else a.T).ravel()
                got = gpu.transform(0, x, xi, zi).reshape(shape, order="F" if oz == "f" else "C")
                assert np.array_equal(got, np.abs(a)), (np.dtype(dt).name, shape, ox, oz)
                got = gpu.scalar(0, x, xi, zi, 2.0).reshape(shape, order="F" if oz == "f" else "C")
                assert np.array_equal(got, (a.astype(np.float32) + np.float32(2.0)).astype(dt) if dt == np.float16 else a + dt(2.0)), (
                    "scalar", np.dtype(dt).name, shape, ox, oz)
