"""The benchmark configurations at their full sizes: HIP path through the C ABI against the CPU checker on the
same seeded inputs, plus properties that do not depend on a second implementation (exact IEEE results from
numpy where the op is a single rounding, float64 ground truth for reductions, softmax rows summing to one,
dropout keeping survivors unchanged).

Tolerances (the ones the benchmark definition states): index reductions and the RNG integer stream bit-exact;
fp32 elementwise <= 2 ULP; fp32 reductions relative 1e-5; fp16 1e-2.
"""
import numpy as np
import pytest

from golden_inputs import shape_info_np, ulp_distance
from libnd4j_amd import harness, workloads

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib(cpu_checker):
    return cpu_checker


def _run(case):
    case.gpu(0)
    return case.result(0)


def test_config0_tanh(gpu, lib):
    w = workloads.transform_tanh(gpu.dev, copies=1)
    try:
        c = w.case("transform_tanh")
        got, want = _run(c), c.cpu(lib)
        assert got.shape == want.shape == (1 << 24,)
        assert ulp_distance(got, want).max() <= 2
        # odd function, bounded by one, monotone on a sorted sample
        x = w.host["x"]
        assert np.all(np.abs(got) <= 1.0)
        assert np.array_equal(np.sign(got), np.sign(x))
        order = np.argsort(x[: 1 << 16])
        assert np.all(np.diff(got[: 1 << 16][order]) >= 0)
    finally:
        w.free()


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_config1_pairwise_and_broadcast(gpu, lib, dtype):
    w = workloads.pairwise_broadcast(gpu.dev, dtype=dtype, copies=1)
    try:
        x, y, bias = w.host["x"], w.host["y"], w.host["bias"]
        tag = "" if dtype == "float32" else "_float16"
        rows, cols = 65536, 1024
        # one rounding per element: numpy's IEEE result is the expected value, bit for bit
        expect = {"pairwise_add": x + y, "pairwise_multiply": x * y,
                  "broadcast_add_row": (x.reshape(rows, cols) + bias[None, :]).reshape(-1)}
        for name, e in expect.items():
            c = w.case(name + tag)
            got = _run(c)
            assert got.dtype == np.dtype(dtype)
            assert np.array_equal(got, e.astype(dtype)), name
            if dtype == "float32":
                assert np.array_equal(got, c.cpu(lib)), name
    finally:
        w.free()


def test_config2_reductions(gpu, lib):
    w = workloads.reductions(gpu.dev, copies=1)
    try:
        rows, cols = 16384, 4096
        x = w.host["x"]
        x64 = x.astype(np.float64).reshape(rows, cols)
        absx = np.abs(x64)
        for dim, axis_len in ((1, cols), (0, rows)):
            truth_sum = x64.sum(axis=dim)
            # a sum of n rounded terms is only defined up to the rounding of its partial sums: scale of a
            # row's terms, as in tests/checks.py
            scale = absx.sum(axis=dim) / np.sqrt(axis_len)
            got = _run(w.case("sum_dim%d" % dim)).astype(np.float64)
            assert np.all(np.abs(got - truth_sum) <= 1e-5 * np.maximum(np.abs(truth_sum), scale)), dim
            # against the CPU loop: its own fp32 running sum drifts from the exact value (16384 sequential
            # roundings along dimension 0), so the two may differ by that drift plus the bound above
            cpu = w.case("sum_dim%d" % dim).cpu(lib).astype(np.float64)
            assert np.all(np.abs(got - cpu) <= np.abs(cpu - truth_sum) + 1e-5 * np.maximum(np.abs(truth_sum), scale)), dim
            got = _run(w.case("mean_dim%d" % dim)).astype(np.float64)
            assert np.all(np.abs(got - truth_sum / axis_len) <= 1e-5 * np.maximum(np.abs(truth_sum), scale) / axis_len), dim
            assert np.array_equal(_run(w.case("max_dim%d" % dim)), x.reshape(rows, cols).max(axis=dim)), dim
            got = _run(w.case("argmax_dim%d" % dim))
            assert np.array_equal(got, np.argmax(x.reshape(rows, cols), axis=dim).astype(np.float32)), dim
            assert np.array_equal(got, w.case("argmax_dim%d" % dim).cpu(lib)), dim
        total = x64.sum()
        scale = absx.sum() / np.sqrt(x.size)
        got = float(_run(w.case("sum_full"))[0])
        assert abs(got - total) <= 1e-5 * max(abs(total), scale)
        assert abs(float(_run(w.case("mean_full"))[0]) - total / x.size) <= 1e-5 * max(abs(total), scale) / x.size
        assert float(_run(w.case("max_full"))[0]) == float(x.max())
        assert float(_run(w.case("argmax_full"))[0]) == float(np.float32(np.argmax(x)))
        assert float(_run(w.case("argmax_full"))[0]) == float(w.case("argmax_full").cpu(lib))
    finally:
        w.free()


def test_config3_summary_stats_and_softmax_chain(gpu, lib):
    w = workloads.stats_softmax(gpu.dev, copies=1)
    try:
        rows, cols = 32768, 2048
        x = w.host["x"]
        m = x.astype(np.float64).reshape(cols, rows).T  # the f-order matrix as [rows, cols]
        for dim in (1, 0):
            var = m.var(axis=dim, ddof=1)
            got = _run(w.case("variance_dim%d" % dim)).astype(np.float64)
            assert np.all(np.abs(got - var) <= 1e-5 * var), dim
            got = _run(w.case("std_dim%d" % dim)).astype(np.float64)
            assert np.all(np.abs(got - np.sqrt(var)) <= 1e-5 * np.sqrt(var)), dim
            cpu = w.case("variance_dim%d" % dim).cpu(lib).astype(np.float64)
            got = _run(w.case("variance_dim%d" % dim)).astype(np.float64)
            assert np.all(np.abs(got - cpu) <= 1e-5 * np.abs(cpu)), dim
        chain = w.case("softmax_chain")
        got = _run(chain)
        want = chain.cpu(lib)
        sm = got.astype(np.float64).reshape(cols, rows).T
        assert np.all(got >= 0) and np.all(got <= 1)
        assert np.all(np.abs(sm.sum(axis=1) - 1.0) <= 1e-5)
        # exp and the row sums differ by rounding only: 2 ULP on the exponential (2.4e-7), 1e-5 on the row sum and half
        # an ULP on the quotient add up to 1.03e-5; the measured maxima are printed (pytest -s shows them)
        bar = 1.0e-5 + 3 * 2.0 ** -23
        denom = np.maximum(np.abs(want.astype(np.float64)), 1e-30)
        worst = {"chain vs reference": (np.abs(got.astype(np.float64) - want) / denom).max()}
        assert worst["chain vs reference"] <= bar
        truth = np.exp(m - m.max(axis=1, keepdims=True))
        truth /= truth.sum(axis=1, keepdims=True)
        worst["chain vs float64"] = (np.abs(sm - truth) / np.maximum(truth, 1e-30)).max()
        assert worst["chain vs float64"] <= bar
        # the same softmax as one call, on the f-order matrix and on the same memory read as a c-order matrix
        fused = _run(w.case("softmax_fused_forder")).astype(np.float64).reshape(cols, rows).T
        worst["fused f-order vs float64"] = (np.abs(fused - truth) / np.maximum(truth, 1e-30)).max()
        assert worst["fused f-order vs float64"] <= bar
        assert np.all(np.abs(fused.sum(axis=1) - 1.0) <= 1e-5)
        mc = x.astype(np.float64).reshape(rows, cols)
        truth_c = np.exp(mc - mc.max(axis=1, keepdims=True))
        truth_c /= truth_c.sum(axis=1, keepdims=True)
        fused = _run(w.case("softmax_fused_corder")).astype(np.float64).reshape(rows, cols)
        worst["fused c-order vs float64"] = (np.abs(fused - truth_c) / np.maximum(truth_c, 1e-30)).max()
        assert worst["fused c-order vs float64"] <= bar
        want = w.case("softmax_fused_corder").cpu(lib).astype(np.float64).reshape(rows, cols)
        worst["fused c-order vs reference"] = (np.abs(fused - want) / np.maximum(want, 1e-30)).max()
        assert worst["fused c-order vs reference"] <= bar
        logsm = _run(w.case("logsoftmax_fused_corder")).astype(np.float64).reshape(rows, cols)
        # (a logarithm near zero has no relative accuracy to speak of: 1e-5 relative plus 1e-6 absolute)
        assert np.all(np.abs(logsm - np.log(truth_c)) <= 1e-5 * np.abs(np.log(truth_c)) + 1e-6)
        # few long rows: the same memory read as [rows / 64, cols * 64]
        ml = x.astype(np.float64).reshape(rows // 64, cols * 64)
        truth_l = np.exp(ml - ml.max(axis=1, keepdims=True))
        truth_l /= truth_l.sum(axis=1, keepdims=True)
        fused = _run(w.case("softmax_fused_long_rows")).astype(np.float64).reshape(rows // 64, cols * 64)
        worst["fused long rows vs float64"] = (np.abs(fused - truth_l) / np.maximum(truth_l, 1e-30)).max()
        assert worst["fused long rows vs float64"] <= bar
        print("softmax, largest relative differences:", ", ".join("%s %.3g" % kv for kv in sorted(worst.items())))
        assert np.all(np.abs(fused.sum(axis=1) - 1.0) <= 1e-5)
        # the copy that serves as the f-order kernel's yardstick moves every element
        assert np.array_equal(_run(w.case("yardstick_copy_forder_tiles")), x)
        # IsMax: one-hot of the first maximum, whole array and per row; bit-exact
        xf = x.reshape(rows, cols)
        # (the winning index travels as a value of the data type, in the reference too - execIndexReduceScalarFloat
        # returns a float - so beyond 2^24 elements the one lands on the index rounded to float)
        got = _run(w.case("ismax_whole"))
        assert got.sum() == 1 and got[int(np.float32(np.argmax(x)))] == 1
        got = _run(w.case("ismax_dim1")).reshape(rows, cols)
        assert np.all(got.sum(axis=1) == 1)
        assert np.array_equal(np.argmax(got, axis=1), np.argmax(xf, axis=1))
    finally:
        w.free()


def test_general_views_at_benchmark_size(gpu, lib):
    """TADs over several dimensions, broadcasts of sub-arrays and rows with a pitch: against the compiled reference and
    against numpy on the same inputs."""
    w = workloads.general_views(gpu.dev, copies=1)
    try:
        h = w.host
        x1 = h["x1"].reshape(128, 128, 56, 56)
        x64 = x1.astype(np.float64)
        truth = x64.sum(axis=(0, 2, 3))
        scale = np.abs(x64).sum(axis=(0, 2, 3)) / np.sqrt(x1.size // 128)
        c = w.case("sum_nchw_dims023")
        got, cpu = _run(c).astype(np.float64), c.cpu(lib).astype(np.float64)
        assert np.all(np.abs(got - truth) <= 1e-5 * np.maximum(np.abs(truth), scale))
        assert np.all(np.abs(got - cpu) <= np.abs(cpu - truth) + 1e-5 * np.maximum(np.abs(truth), scale))
        c = w.case("sum_nchw_dims02")
        truth2 = x64.sum(axis=(0, 2)).ravel()
        scale2 = np.abs(x64).sum(axis=(0, 2)).ravel() / np.sqrt(128 * 56)
        got, cpu = _run(c).astype(np.float64), c.cpu(lib).astype(np.float64)
        assert np.all(np.abs(got - truth2) <= 1e-5 * np.maximum(np.abs(truth2), scale2))
        assert np.all(np.abs(got - cpu) <= np.abs(cpu - truth2) + 1e-5 * np.maximum(np.abs(truth2), scale2))
        c = w.case("variance_nchw_dims023")
        var = x64.var(axis=(0, 2, 3), ddof=1)
        got, cpu = _run(c).astype(np.float64), c.cpu(lib).astype(np.float64)
        assert np.all(np.abs(got - var) <= 1e-5 * var)
        assert np.all(np.abs(got - cpu) <= 1e-5 * np.abs(cpu))
        c = w.case("broadcast_add_nchw_dims23")
        got = _run(c)
        assert np.array_equal(got, (x1 + h["plane"].reshape(1, 1, 56, 56)).ravel())
        assert np.array_equal(got, c.cpu(lib))
        c = w.case("argmax_cube_dims12")
        got = _run(c)
        assert np.array_equal(got, np.argmax(h["x2"].reshape(4096, -1), axis=1).astype(np.float32))
        assert np.array_equal(got, c.cpu(lib))
        c = w.case("broadcast_add_slab_dims02")
        got = _run(c)
        assert np.array_equal(got, (h["x3"].reshape(256, 1024, 256) + h["mat"].reshape(256, 1, 256)).ravel())
        assert np.array_equal(got, c.cpu(lib))
        # the view's rows: 1024 of every 1032 elements; the 8 between two rows are never written
        rows, cols, pitch = 65536, 1024, 1032

        def view(a):
            return np.lib.stride_tricks.as_strided(a, (rows, cols), (4 * pitch, 4))

        def gaps(a):
            return np.lib.stride_tricks.as_strided(a[cols:], (rows - 1, pitch - cols), (4 * pitch, 4))

        c = w.case("pairwise_add_padded_rows")
        got = _run(c)
        assert np.array_equal(view(got), view(h["xv"]) + view(h["yv"]))
        assert np.array_equal(view(got), view(c.cpu(lib)))
        assert not gaps(got).any()
        c = w.case("broadcast_add_row_padded_rows")
        got = _run(c)
        assert np.array_equal(view(got), view(h["xv"]) + h["bias_v"][None, :])
        assert np.array_equal(view(got), view(c.cpu(lib)))
        assert not gaps(got).any()
        c = w.case("transform_exp_padded_rows")
        got = _run(c)
        assert ulp_distance(view(got), view(c.cpu(lib))).max() <= 2
        assert not gaps(got).any()
    finally:
        w.free()


def test_data_movement_at_benchmark_size(gpu, lib):
    w = workloads.data_movement(gpu.dev, copies=1)
    try:
        rows, cols = 65536, 1024
        x, perm, smap = w.host["x"], w.host["perm"], w.host["smap"]
        m = x.reshape(rows, cols)
        assert np.array_equal(_run(w.case("pullrows_permute")).reshape(rows, cols), m[perm])
        assert np.array_equal(_run(w.case("concat_dim0")), x)      # row blocks of x put back together
        assert np.array_equal(_run(w.case("concat_dim1")), x)      # column blocks of x put back together
        assert np.array_equal(_run(w.case("concat_dim1")), w.case("concat_dim1").cpu(lib))
        assert np.array_equal(_run(w.case("flatten_same_order")), x)
        # the buffer read as an f-order [rows, cols] matrix, flattened in C order
        assert np.array_equal(_run(w.case("flatten_f_to_c")), x.reshape(cols, rows).T.ravel())
        assert np.array_equal(_run(w.case("tear_rows")), x.reshape(1024, -1)[5])
        want = m.copy()
        a = np.nonzero(smap >= 0)[0]
        want[a], want[smap[a]] = m[smap[a]], m[a]
        assert np.array_equal(_run(w.case("shuffle_rows")).reshape(rows, cols), want)
        half = _run(w.case("convert_float_to_half"))
        assert np.array_equal(half.view(np.uint16), x.astype(np.float16).view(np.uint16))
        assert np.array_equal(_run(w.case("convert_half_to_float")), x.astype(np.float16).astype(np.float32))
    finally:
        w.free()


def test_config4_random(gpu, lib):
    w = workloads.random_fills(gpu.dev, copies=1)
    try:
        n = 1 << 26
        # the integer stream, at the start, across the first buffer wrap and at the far end
        a = gpu.rng(w.host["seed"], w.host["buffer_longs"])
        b = lib.rng_init(w.host["seed"], w.host["buffer_longs"])
        for start, count in ((0, 4096), ((1 << 20) - 100, 4096), (n - 4096, 4096), (3 * n + 12345, 4096)):
            assert np.array_equal(a.elements(start, count), b.elements(start, count)), start
        a.destroy()
        b.destroy()
        uni = w.case("uniform_fill")
        got, want = _run(uni), uni.cpu(lib)
        assert np.array_equal(got, want)
        assert got.min() >= 0.0 and got.max() <= 1.0
        assert abs(float(got.astype(np.float64).mean()) - 0.5) < 1e-3
        gau = w.case("gaussian_fill")
        got, want = _run(gau), gau.cpu(lib)
        assert ulp_distance(got, want).max() <= 2
        g64 = got.astype(np.float64)
        assert abs(g64.mean()) < 5e-3 and abs(g64.std() - 1.0) < 5e-3
        drop = w.case("dropout_inplace")
        before = w.host["dropout_x"]
        got, want = _run(drop), drop.cpu(lib)
        assert np.array_equal(got, want)
        kept = got != 0
        assert np.array_equal(got[kept], before[kept])
        assert abs(float(kept.mean()) - 0.5) < 1e-3
    finally:
        w.free()


def test_array_result_calls_need_no_read_back_from_the_device(gpu):
    """Every benchmark case passes what the CUDA convention provides (host copies of the shapeInfos, TAD tables); with
    that, no call may have to read a shapeInfo or a dimension array back from the device, because each read-back
    synchronises the stream.  Small shapes: the host paths are the same as at full size."""
    ops = gpu.dev.ops
    builders = (lambda d: workloads.transform_tanh(d, n=1 << 12, copies=1),
                lambda d: workloads.pairwise_broadcast(d, rows=64, cols=128, copies=1),
                lambda d: workloads.pairwise_broadcast(d, rows=64, cols=128, dtype="float16", copies=1),
                lambda d: workloads.reductions(d, rows=64, cols=128, copies=1),
                lambda d: workloads.reduce3_pairs(d, rows=64, cols=128, copies=1),
                lambda d: workloads.stats_softmax(d, rows=128, cols=64, copies=1),
                lambda d: workloads.data_movement(d, rows=2048, cols=64, copies=1),
                lambda d: workloads.random_fills(d, n=1 << 12, side=64, buffer_longs=1 << 10, copies=1))
    for build in builders:
        w = build(gpu.dev)
        try:
            for c in w.cases:
                before = ops.amd_hostFetchCount()
                c.gpu(0)
                gpu.dev.sync()
                assert ops.amd_hostFetchCount() == before, (w.name, c.name)
        finally:
            w.free()


def test_arrays_of_more_than_2_to_the_31_elements(gpu):
    """Lengths are Nd4jLong in the reference's entry points (blas/NativeOps.h): element indexes, vector counts and
    reduction positions must not pass through 32 bits anywhere.  Half arrays keep the transfers to a few GB; the data are a
    short pattern repeated, so that the expected results are known without a second pass of numpy arithmetic."""
    n = (1 << 31) + 65539  # odd: the 16-byte vector path ends in a scalar tail
    L = 4099
    rs = np.random.RandomState(77)
    px = rs.randint(-200, 200, L).astype(np.float16)
    py = rs.randint(-200, 200, L).astype(np.float16)
    reps = n // L + 1
    x, y = np.tile(px, reps)[:n], np.tile(py, reps)[:n]
    info = harness.shape_info([1, n])

    def matches(out, pattern):
        k = n // L
        body = out[:k * L].view(np.uint16).reshape(k, L)
        return bool(np.all(body == pattern.view(np.uint16))) and np.array_equal(out[k * L:].view(np.uint16),
                                                                                 pattern[:n - k * L].view(np.uint16))

    print("pairwise add over %d halves" % n, flush=True)
    assert matches(gpu.pairwise(0, x, info, y, info, info), px + py)
    del y
    print("scalar multiply", flush=True)
    assert matches(gpu.scalar(2, x, info, info, 0.5), (px.astype(np.float32) * np.float32(0.5)).astype(np.float16))
    print("mean, max, argmax", flush=True)
    tail = px[:n - (n // L) * L].astype(np.float64)
    total = px.astype(np.float64).sum() * (n // L) + tail.sum()
    # Mean divides by the length cast to int (include/ops/ops.h:2147), which wraps beyond 2^31 - 1: the reference's own
    # result for this length, and so this library's
    mean = total / (n - (1 << 32))
    assert abs(gpu.reduce_scalar(0, x, info) - mean) <= 1e-2 * abs(mean) + 1e-3
    where = (1 << 31) + 1000
    x[where] = 300
    assert gpu.reduce_scalar(3, x, info) == 300.0
    # the position passes through the data type on its way back (the CUDA back end stores it in a half buffer before
    # widening it, blas/cuda/NativeOps.cu execIndexReduceScalarHalf): beyond 65504 that is infinity
    assert gpu.indexreduce_scalar(0, x, info, raw=True) == float("inf")
    x[where] = px[where % L]
    # in fp32 the position survives, rounded to the 24 bits of a float
    print("argmax over %d floats" % n, flush=True)
    xf = x.astype(np.float32)
    xf[where] = 300
    assert gpu.indexreduce_scalar(0, xf, info, raw=True) == float(np.float32(where))
    del xf
    # a view that is not element-wise strided and spans more than 2^32 positions of a c-order walk
    print("transform over a padded [65537, 65536] view", flush=True)
    rows, cols, pitch = 65537, 65536, 65544
    del x
    xv = np.tile(px, (rows * pitch) // L + 1)[:rows * pitch]
    vinfo = harness.shape_info([rows, cols], strides=[pitch, 1], ews=0)
    out = gpu.transform(0, xv, vinfo, vinfo)  # Abs
    got = out[:(rows - 1) * pitch + cols]
    want = np.abs(xv[:got.size]).view(np.uint16).reshape(-1)
    grid_got = np.lib.stride_tricks.as_strided(got.view(np.uint16), (rows, cols), (pitch * 2, 2))
    grid_want = np.lib.stride_tricks.as_strided(want, (rows, cols), (pitch * 2, 2))
    assert np.array_equal(grid_got, grid_want)
    # the padding between the rows is not touched
    pad = np.lib.stride_tricks.as_strided(got.view(np.uint16)[cols:], (rows - 1, pitch - cols), (pitch * 2, 2))
    assert not pad.any()


def test_tanh_within_two_ulp_of_the_reference_over_the_float_range(gpu, lib):
    import backends
    cpu = backends.CpuBackend(lib)
    # The device does not replay the C library's tanhf: a polynomial below 1, an exp2-based form from 1 on.  Every one of
    # the 2^32 float bit patterns has been compared with the compiled reference: 4176995678 identical, 117188678 at
    # 1 ULP, 782940 at 2 ULP (all of those below 1, where the library itself is up to 2 ULP off), none further.  This is
    # the same comparison on every 61st pattern, plus whole stretches around the points where the routine changes its
    # course (|x| = 1, 22, the denormals, infinity and the NaNs) and the signed zeros, bit for bit.
    parts = [np.arange(0, 1 << 32, 61, dtype=np.uint64)]
    for centre in (0x3f800000, 0x41b00000, 0x00800000, 0x7f800000, 0x39800000, 0x3c7b9000):
        for sign in (0, 0x80000000):
            parts.append(np.arange(centre - 70000, centre + 70000, dtype=np.uint64) + sign)
    x = np.concatenate(parts).astype(np.uint32).view(np.float32)
    xi = shape_info_np([1, x.size])
    g, c = gpu.transform(15, x, xi, xi), cpu.transform(15, x, xi, xi)
    assert np.array_equal(np.isnan(g), np.isnan(c))
    assert ulp_distance(g, c).max() <= 2
    zeros = np.array([0.0, -0.0, 1e-45, -1e-45], np.float32)
    zi = shape_info_np([1, 4])
    assert np.array_equal(gpu.transform(15, zeros, zi, zi).view(np.uint32), cpu.transform(15, zeros, zi, zi).view(np.uint32))
    # odd lengths and misaligned starts take the scalar edges of the kernel; half goes through the same routine
    for n, off in ((1, 0), (7, 1), (4099, 3), (100001, 2)):
        xs = np.linspace(-5, 5, n + off).astype(np.float32)
        vi = shape_info_np([1, n + off])
        assert ulp_distance(gpu.transform(15, xs, vi, vi), cpu.transform(15, xs, vi, vi)).max() <= 2
    xh = np.arange(0, 1 << 16, dtype=np.uint16).view(np.float16)
    hi = shape_info_np([1, xh.size])
    gh, ch = gpu.transform(15, xh, hi, hi), cpu.transform(15, xh, hi, hi)
    assert np.array_equal(np.isnan(gh), np.isnan(ch)) and ulp_distance(gh, ch).max() <= 1
