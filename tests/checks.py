"""Parity checks that take a backend (tests/backends.py), so the CPU oracle and the HIP path are held to the
same known answers:

  * the golden values of the reference's own unit tests (tests/golden/reference_fixtures.json);
  * vectors produced by the compiled reference (tests/golden/ref_vectors.json);
  * closed forms that do not come from the code under test (numpy / brute force).

Tolerances (from the task statement): bit-exact for indices and the generator's integer stream, at most 2 ULP
for fp32 elementwise results, relative error 1e-5 for fp32 reductions, 1e-2 for fp16.
"""
import json
import os

import numpy as np

from golden_inputs import (BROADCAST_OPS, INDEX_OPS, PAIRWISE_OPS, REDUCE_OPS, SCALAR_OPS, SCALAR_VALUES, TRANSFORM_OPS, from_hexbits, op_extra,
                           pairwise_inputs, reduce_input, shape_info_np, transform_input, ulp_distance)

HERE = os.path.dirname(os.path.abspath(__file__))
ELEMENTWISE_ULP = 2
REDUCE_RTOL = 1e-5
HALF_RTOL = 1e-2


def load_json(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


def assert_ulp(got, want, max_ulp, what):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, got.shape, want.shape)
    d = ulp_distance(got, want)
    nan_mismatch = np.isnan(got) != np.isnan(want)
    assert not nan_mismatch.any(), "%s: NaN pattern differs at %s" % (what, np.nonzero(nan_mismatch)[0][:5])
    worst = int(d.max()) if d.size else 0
    assert worst <= max_ulp, "%s: %d ULP at index %d (got %r, want %r)" % (
        what, worst, int(d.argmax()), got.flat[int(d.argmax())], want.flat[int(d.argmax())])


def assert_reduction_close(got, want, scale, what, rtol=REDUCE_RTOL):
    """|got - want| <= rtol * max(|want|, scale).  `scale` is the natural magnitude of the accumulation (for a
    sum: the sum of magnitudes over sqrt(n)), which keeps the bound meaningful where a sum cancels to ~0."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want)), "%s: NaN pattern differs" % what
    bound = rtol * np.maximum(np.abs(want), scale)
    with np.errstate(invalid="ignore"):  # equal infinities subtract to NaN; `got == want` accepts them below
        err = np.abs(got - want)
    ok = (err <= bound) | (np.isnan(want)) | (got == want)
    assert ok.all(), "%s: |err| %g > bound %g at %d (got %r want %r)" % (
        what, err[~ok].max(), bound[~ok][0], int(np.nonzero(~ok)[0][0]), got[~ok][0], want[~ok][0])


# ---------------------------------------------------------------------------------------------------------
# fixtures of the reference's own tests

def check_reference_fixtures(be):
    fx = load_json("reference_fixtures.json")
    f32 = np.float32
    for c in fx["transform"]:
        shape = c["shape"]
        n = int(np.prod(shape))
        x = np.array(c["x"], f32) if "x" in c else np.full(n, c["fill"], f32)
        want = np.array(c["expected"], f32) if "expected" in c else np.full(n, c["expected_fill"], f32)
        extra = np.array(c["extra"], f32) if "extra" in c else None
        info = shape_info_np(shape)
        got = be.transform(c["opNum"], x, info, info, extra)
        assert np.array_equal(got, want), c["source"]
    for c in fx["pairwise"]:
        n = int(np.prod(c["shape"]))
        info = shape_info_np(c["shape"])
        got = be.pairwise(c["opNum"], np.full(n, c["x_fill"], f32), info, np.full(n, c["y_fill"], f32), info, info)
        assert np.array_equal(got, np.full(n, c["expected_fill"], f32)), c["source"]
    for c in fx["broadcast"]:
        xi = np.array(c["x_info"], np.int64)
        got = be.broadcast(c["opNum"], np.array(c["x"], f32), xi, np.array(c["y"], f32), np.array(c["y_info"], np.int64),
                           xi, c["dims"])
        assert np.array_equal(got, np.array(c["expected"], f32)), c["source"]
    for c in fx["reduce"]:
        shape = c["shape"]
        if "row_pattern" in c:
            k = np.arange(1, shape[0] + 1, dtype=f32)[:, None]
            x = (k * np.array(c["row_pattern"], f32)[None, :]).reshape(-1)
        else:
            x = np.array(c["x"], f32)
        got = be.reduce(c["opNum"], x, shape_info_np(shape), None, c["dims"], len(c["expected"]))
        assert np.array_equal(got, np.array(c["expected"], f32)), c["source"]
    for c in fx["reduce_scalar"]:
        got = be.reduce_scalar(c["opNum"], np.array(c["x"], f32), shape_info_np(c["shape"]))
        assert float(got) == c["expected"], c["source"]
    for c in fx["index_reduce"]:
        xi = np.array(c["x_info"], np.int64)
        x = np.array(c["x"], f32) if "x" in c else np.linspace(c["linspace"][0], c["linspace"][1], int(np.prod(xi[1:1 + xi[0]]))).astype(f32)
        got = be.indexreduce(c["opNum"], x, xi, None, c["dims"], len(c["expected"]))
        assert np.array_equal(got, np.array(c["expected"], f32)), c["source"]
    for c in fx["index_reduce_scalar"]:
        xi = np.array(c["x_info"], np.int64)
        x = np.linspace(c["linspace"][0], c["linspace"][1], 25).astype(f32)
        assert float(be.indexreduce_scalar(c["opNum"], x, xi)) == c["expected"], c["source"]
    for c in fx["reduce3"]:
        x, y = np.array(c["x"], f32), np.array(c["y"], f32)
        xi = shape_info_np(c["shape"])
        yi = shape_info_np(c.get("y_shape", c["shape"]))
        if c["kind"] == "scalar":
            got = np.array([be.reduce3_scalar(c["opNum"], x, xi, y, yi)], f32)
        elif c["kind"] == "all":
            got = be.reduce3_all(c["opNum"], x, xi, y, yi, None, c["dims"], len(c["expected"]))
        else:
            got = be.reduce3(c["opNum"], x, xi, y, yi, np.zeros(1, f32), c["dims"], len(c["expected"]))
        assert np.allclose(got, c["expected"], atol=c["tol"] + 1e-6 * (c["tol"] > 0), rtol=0), "%s: %r" % (c["source"], got)
    for c in fx["summary_stats"]:
        got = be.summarystats(c["opNum"], c["bias"], np.array(c["x"], f32), shape_info_np(c["shape"]), c["dims"],
                              len(c["expected"]))
        assert np.allclose(got, c["expected"], atol=c["tol"], rtol=0), c["source"]
    for c in fx["summary_stats_scalar"]:
        if "x" in c:
            x = np.array(c["x"], f32)
            shape = c["shape"]
        else:
            n = c["n"]
            base, amp = c["alternating"]
            x = (f32(base) + np.where(np.arange(n) % 2 == 1, f32(amp), -f32(amp))).astype(f32)
            shape = [1, n]
        got = be.summarystats_scalar(c["opNum"], c["bias"], x, shape_info_np(shape))
        assert abs(float(got) - c["expected"]) <= c["tol"], "%s: %r" % (c["source"], got)


def check_tad_fixtures(tad_fn):
    """tad_fn(x_info, dims) -> (tadShapeInfo, offsets)."""
    fx = load_json("reference_fixtures.json")
    for c in fx["tad_shape_info"]:
        ti, _ = tad_fn(np.array(c["x_info"], np.int64), c["dims"])
        assert [int(v) for v in ti] == c["tad_info"], "%s: %s" % (c["source"], list(ti))
    for c in fx["tad_offsets"]:
        _, off = tad_fn(np.array(c["x_info"], np.int64), c["dims"])
        assert [int(v) for v in off] == c["offsets"], c["source"]
    for c in fx["tad_ews"]:
        info = shape_info_np(c["shape"], c["order"])
        ti, off = tad_fn(info, c["dims"])
        r = int(ti[0])
        assert int(ti[2 * r + 2]) == c["ews"], c["source"]
        assert len(off) == c["result_length"], c["source"]
    for c in fx["shape_info"]:
        info = shape_info_np(c["shape"], c["order"])
        r = len(c["shape"])
        assert [int(v) for v in info[1 + r:1 + 2 * r]] == c["strides"], c["source"]
    vec = load_json("ref_vectors.json")
    for c in vec["tad"]:
        info = shape_info_np(c["shape"], c["order"])
        assert [int(v) for v in info] == c["x_info"], "shapeInfo of %s %s" % (c["shape"], c["order"])
        ti, off = tad_fn(info, c["dims"])
        assert [int(v) for v in ti] == c["tad_info"], "TAD shapeInfo %s %s %s" % (c["shape"], c["order"], c["dims"])
        assert len(off) == c["num_tads"]
        assert [int(v) for v in off[:8]] == c["offsets_head"] and [int(v) for v in off[-3:]] == c["offsets_tail"]
        assert int(np.sum(off)) == c["offsets_sum"]


# ---------------------------------------------------------------------------------------------------------
# vectors of the compiled reference

# Composite ops whose float expression the reference's -fassociative-math / -freciprocal-math build is free to
# reorder, and which amplify a last-place difference of an intermediate (1 - 1/(1+a), five-term sums): the
# compiled reference's vectors are reproduced to a few ULP only.  Everything else is held to ELEMENTWISE_ULP.
LOOSE_TRANSFORM_ULP = {53: 4, 54: 16}
LOOSE_PAIRWISE_ULP = {94: 8}


def check_op_vectors(be, max_ulp=ELEMENTWISE_ULP, exact_composites=False):
    vec = load_json("ref_vectors.json")["ops"]
    f32 = np.float32
    failures = []

    def run(fn, what):
        try:
            fn()
        except AssertionError as e:
            failures.append("%s: %s" % (what, str(e).splitlines()[0]))

    x = transform_input()
    xi = shape_info_np([1, x.size])
    for op in TRANSFORM_OPS:
        want = from_hexbits(vec["transform_f32"][str(op)], f32)
        tol = max_ulp if exact_composites else max(max_ulp, LOOSE_TRANSFORM_ULP.get(op, 0))
        run(lambda: assert_ulp(be.transform(op, x, xi, xi, op_extra("transform", op)), want, tol, "transform op %d" % op), "transform %d" % op)
    a, b = pairwise_inputs()
    ai = shape_info_np([1, a.size])
    for op in PAIRWISE_OPS:
        want = from_hexbits(vec["pairwise_f32"][str(op)], f32)
        tol = max(max_ulp, LOOSE_PAIRWISE_ULP.get(op, 0))
        run(lambda: assert_ulp(be.pairwise(op, a, ai, b, ai, ai, op_extra("pairwise", op)), want, tol, "pairwise op %d" % op), "pairwise %d" % op)
    bxi = shape_info_np([12, 8])
    for op in BROADCAST_OPS:
        want1 = from_hexbits(vec["broadcast_f32_12x8"][str(op)]["dim1"], f32)
        run(lambda: assert_ulp(be.broadcast(op, a, bxi, b[:8].copy(), shape_info_np([1, 8]), bxi, [1]), want1, max_ulp, "broadcast op %d dim 1" % op), "broadcast %d/1" % op)
        want0 = from_hexbits(vec["broadcast_f32_12x8"][str(op)]["dim0"], f32)
        run(lambda: assert_ulp(be.broadcast(op, a, bxi, b[8:20].copy(), shape_info_np([12, 1]), bxi, [0]), want0, max_ulp, "broadcast op %d dim 0" % op), "broadcast %d/0" % op)
    for op in SCALAR_OPS:
        w = vec["scalar_f32"][str(op)]
        for k, value in enumerate(SCALAR_VALUES):
            run(lambda: assert_ulp(be.scalar(op, a, ai, ai, value), from_hexbits(w["value%d" % k], f32), max_ulp, "scalar op %d value %g" % (op, value)), "scalar %d" % op)
        run(lambda: assert_ulp(be.scalar_tad(op, a, bxi, b[:12].copy(), None, [1]), from_hexbits(w["tad_dim1"], f32), max_ulp, "scalar op %d per row" % op), "scalar %d/1" % op)
        run(lambda: assert_ulp(be.scalar_tad(op, a, bxi, b[:8].copy(), None, [0]), from_hexbits(w["tad_dim0"], f32), max_ulp, "scalar op %d per column" % op), "scalar %d/0" % op)
    m = reduce_input()
    mi = shape_info_np([12, 10])
    scale = float(np.abs(m).sum())
    for op in REDUCE_OPS:
        e = op_extra("reduce", op)
        w = vec["reduce_f32_12x10"][str(op)]
        run(lambda: assert_reduction_close(be.reduce(op, m, mi, e, [1], 12), from_hexbits(w["dim1"], f32), scale * 1e-2, "reduce op %d dim 1" % op), "reduce %d/1" % op)
        run(lambda: assert_reduction_close(be.reduce(op, m, mi, e, [0], 10), from_hexbits(w["dim0"], f32), scale * 1e-2, "reduce op %d dim 0" % op), "reduce %d/0" % op)
        run(lambda: assert_reduction_close([be.reduce_scalar(op, m, mi, e)], from_hexbits(w["scalar"], f32), scale * 1e-2, "reduce op %d scalar" % op), "reduce %d/s" % op)
    for op in INDEX_OPS:
        e = op_extra("indexreduce", op)
        w = vec["indexreduce_f32_12x10"][str(op)]

        def idx():
            assert np.array_equal(be.indexreduce(op, m, mi, e, [1], 12), from_hexbits(w["dim1"], f32)), "index op %d dim 1" % op
            assert np.array_equal(be.indexreduce(op, m, mi, e, [0], 10), from_hexbits(w["dim0"], f32)), "index op %d dim 0" % op
            assert f32(be.indexreduce_scalar(op, m, mi, e)) == from_hexbits(w["scalar"], f32)[0], "index op %d scalar" % op
        run(idx, "indexreduce %d" % op)
    for op in (0, 1):
        for bias in (0, 1):
            w = vec["summarystats_f32_12x10"]["%d_%d" % (op, bias)]
            run(lambda: assert_reduction_close(be.summarystats(op, bias, m, mi, [1], 12), from_hexbits(w["dim1"], f32), 0, "stats %d/%d dim 1" % (op, bias)), "stats")
            run(lambda: assert_reduction_close(be.summarystats(op, bias, m, mi, [0], 10), from_hexbits(w["dim0"], f32), 0, "stats %d/%d dim 0" % (op, bias)), "stats")
            run(lambda: assert_reduction_close([be.summarystats_scalar(op, bias, m, mi)], from_hexbits(w["scalar"], f32), 0, "stats %d/%d scalar" % (op, bias)), "stats")
    assert not failures, "%d op vector mismatches:\n  %s" % (len(failures), "\n  ".join(failures))


def check_half_vectors(be, exact):
    """fp16 known answers of the reference's float16 loops.  `exact`: the CPU checkers reproduce them bit for
    bit (same per-operation rounding); the HIP path computes in fp32 and rounds once, so it is held to 1e-2."""
    vec = load_json("ref_vectors.json")["ops"]["f16_2x4"]
    h = np.float16
    xh = (0.1 * (np.arange(8, dtype=np.float32) + 1)).astype(h)
    yh = (1000 + np.arange(8, dtype=np.float32)).astype(h)
    hi = shape_info_np([2, 4])
    rowh = (0.333 * np.arange(4, dtype=np.float32)).astype(h)

    def cmp(got, key):
        want = from_hexbits(vec[key], h)
        if exact:
            assert np.array_equal(np.asarray(got).view(np.uint16), want.view(np.uint16)), key
        else:
            g, w = np.asarray(got, np.float64), want.astype(np.float64)
            assert np.all(np.abs(g - w) <= HALF_RTOL * np.abs(w)), key

    cmp(be.pairwise(0, xh, hi, yh, hi, hi), "pairwise_add")
    cmp(be.pairwise(6, xh, hi, yh, hi, hi), "pairwise_multiply")
    cmp(be.transform(15, xh, hi, hi), "transform_tanh")
    cmp(be.broadcast(0, xh, hi, rowh, shape_info_np([1, 4]), hi, [1]), "broadcast_add_row")
    cmp(np.array([be.reduce_scalar(1, yh, hi)], h), "reduce_sum_y")


def check_half_reduction_vectors(be, exact):
    """fp16 reductions, index reductions and summary statistics against what the reference's own float16 loops return
    (they accumulate in fp16, cpu/reduce.cpp:150-156 with T = float16).  `exact`: the CPU checkers reproduce them bit for
    bit; the HIP path accumulates in fp32 (statistics in double) and rounds once, and is held to the 1e-2 of fp16 -
    index reductions bit for bit."""
    from golden_inputs import half_reduction_input
    vec = load_json("ref_vectors.json")["ops"]["f16_reductions_12x16"]
    h = np.float16
    x = half_reduction_input()
    assert np.array_equal(x.view(np.uint16), from_hexbits(vec["x"], h).view(np.uint16))
    info = shape_info_np([12, 16])

    def cmp(got, want_hex, what, bitwise):
        want = from_hexbits(want_hex, h)
        got = np.asarray(got, h).reshape(want.shape)
        if bitwise:
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), what
        else:
            g, w = got.astype(np.float64), want.astype(np.float64)
            assert np.all(np.abs(g - w) <= HALF_RTOL * np.abs(w)), (what, np.abs(g - w).max())

    for op in (0, 1, 3, 4, 5, 6):
        v = vec["reduce_%d" % op]
        cmp(be.reduce(op, x, info, None, [1], 12), v["dim1"], ("reduce", op, 1), exact)
        cmp(be.reduce(op, x, info, None, [0], 16), v["dim0"], ("reduce", op, 0), exact)
        cmp([be.reduce_scalar(op, x, info)], v["scalar"], ("reduce", op, "scalar"), exact)
    for op in (0, 1):
        v = vec["indexreduce_%d" % op]
        cmp(be.indexreduce(op, x, info, None, [1], 12), v["dim1"], ("indexreduce", op, 1), True)
        cmp(be.indexreduce(op, x, info, None, [0], 16), v["dim0"], ("indexreduce", op, 0), True)
        cmp([be.indexreduce_scalar(op, x, info)], v["scalar"], ("indexreduce", op, "scalar"), True)
    for op in (0, 1):
        for bias in (0, 1):
            v = vec["summarystats_%d_%d" % (op, bias)]
            cmp(be.summarystats(op, bias, x, info, [1], 12), v["dim1"], ("summarystats", op, bias, 1), exact)
            cmp(be.summarystats(op, bias, x, info, [0], 16), v["dim0"], ("summarystats", op, bias, 0), exact)
            cmp([be.summarystats_scalar(op, bias, x, info)], v["scalar"], ("summarystats", op, bias, "scalar"), exact)


def check_rng_vectors(be, float_ulp=ELEMENTWISE_ULP, big=True):
    vec = load_json("ref_vectors.json")["rng"]
    u64 = np.uint64
    for c in vec["small"]:
        g = be.rng(c["seed"], c["size"])
        for kind, v in c["ops"]:
            if kind == "rewind":
                g.rewind(v)
            elif kind == "reseed":
                g.reseed(v)
        assert list(g.state()) == c["state"], "state %s" % c
        got = g.elements(0, 400)
        assert np.array_equal(got, np.array(c["elements_0_400"], u64)), "stream seed %d size %d ops %s" % (c["seed"], c["size"], c["ops"])
        g.destroy()
    if big:
        c = vec["seed119_size2p20"]
        g = be.rng(119, 1 << 20)
        assert [int(v) for v in g.buffer[:8]] == c["buffer_head"] and [int(v) for v in g.buffer[-2:]] == c["buffer_tail"]
        probe = c["probe_index"]
        assert [int(g.elements(i, 1)[0]) for i in probe] == c["fresh"]
        g.destroy()
    seq = vec["float_sequence_seed119_size4096"]
    g = be.rng(119, 4096)
    f32 = np.float32
    for s in seq:
        n = s["n"]
        want = from_hexbits(s["out"], f32)
        x = np.arange(n, dtype=f32) + 1
        if s["overload"] == "z":
            got = g.random_z(s["op"], n, s["args"])
        elif s["overload"] == "xz_inplace":
            got = g.random_xz(s["op"], x, s["args"], inplace=True)
        elif s["overload"] == "xz":
            got = g.random_xz(s["op"], x, s["args"], inplace=False)
        elif s["overload"] == "xyz_inplace":
            got = g.random_xyz(s["op"], None, None, s["args"], mode="inplace_all", n=n)
        else:
            got = g.random_xyz(s["op"], x, -np.arange(n, dtype=f32), s["args"])
        exact_ops = (1, 2, 3, 4, 7, 8, 12)  # selections, integer counts, plain arithmetic
        assert_ulp(got, want, 0 if s["op"] in exact_ops else float_ulp, "random op %d (%s)" % (s["op"], s["overload"]))
        assert list(g.state()) == s["state"], "state after random op %d: %s vs %s" % (s["op"], g.state(), s["state"])
    g.destroy()


# ---------------------------------------------------------------------------------------------------------
# closed forms independent of the code under test

def check_closed_forms(be):
    f32 = np.float32
    rs = np.random.RandomState(5)
    # elementwise: the mathematical function evaluated in float64 and rounded once; the C library's float
    # routines are within 2 ULP of that
    x = rs.uniform(-4, 4, 4099).astype(f32)
    xi = shape_info_np([1, x.size])
    for op, fn in ((15, np.tanh), (3, np.exp), (0, np.abs), (12, np.sin), (2, np.cos), (6, np.negative), (4, np.floor)):
        assert_ulp(be.transform(op, x, xi, xi), fn(x.astype(np.float64)).astype(f32), 2, "transform %d vs float64" % op)
    pos = np.abs(x) + f32(0.01)
    assert_ulp(be.transform(5, pos, xi, xi), np.log(pos.astype(np.float64)).astype(f32), 2, "log vs float64")
    assert_ulp(be.transform(14, pos, xi, xi), np.sqrt(pos), 0, "sqrt vs numpy")
    y = rs.randn(4099).astype(f32)
    for op, fn in ((0, np.add), (6, np.multiply), (9, np.subtract), (2, np.divide)):
        assert np.array_equal(be.pairwise(op, x, xi, y, xi, xi), fn(x, y)), "pairwise %d vs numpy" % op
    # broadcast of a row / a column
    R, C = 37, 53
    m = rs.randn(R * C).astype(f32)
    mi = shape_info_np([R, C])
    row = rs.randn(C).astype(f32)
    col = rs.randn(R).astype(f32)
    assert np.array_equal(be.broadcast(0, m, mi, row, shape_info_np([1, C]), mi, [1]).reshape(R, C), m.reshape(R, C) + row[None, :])
    assert np.array_equal(be.broadcast(1, m, mi, col, shape_info_np([R, 1]), mi, [0]).reshape(R, C), m.reshape(R, C) - col[:, None])
    # reductions against float64 ground truth
    M = m.reshape(R, C).astype(np.float64)
    scale1 = np.abs(M).sum(axis=1) / np.sqrt(C)
    scale0 = np.abs(M).sum(axis=0) / np.sqrt(R)
    assert_reduction_close(be.reduce(1, m, mi, None, [1], R), M.sum(axis=1), scale1, "sum dim1")
    assert_reduction_close(be.reduce(1, m, mi, None, [0], C), M.sum(axis=0), scale0, "sum dim0")
    assert_reduction_close(be.reduce(0, m, mi, None, [1], R), M.mean(axis=1), scale1 / C, "mean dim1")
    assert np.array_equal(be.reduce(3, m, mi, None, [1], R), m.reshape(R, C).max(axis=1))
    assert np.array_equal(be.reduce(3, m, mi, None, [0], C), m.reshape(R, C).max(axis=0))
    assert np.array_equal(be.reduce(4, m, mi, None, [0], C), m.reshape(R, C).min(axis=0))
    assert_reduction_close([be.reduce_scalar(1, m, mi)], [M.sum()], np.abs(M).sum() / np.sqrt(M.size), "sum all")
    assert f32(be.reduce_scalar(3, m, mi)) == m.max()
    ones = np.ones(R * C, f32)
    assert float(be.reduce_scalar(1, ones, mi)) == R * C
    # argmax with ties: first maximum wins
    t = np.array([1, 7, 7, 3, 7, 0], f32)
    assert float(be.indexreduce_scalar(0, t, shape_info_np([1, 6]))) == 1.0
    tie = m.reshape(R, C).copy()
    tie[:, 10] = 50
    tie[:, 20] = 50
    tie[3, :] = 60
    assert np.array_equal(be.indexreduce(0, tie.reshape(-1), mi, None, [1], R), np.argmax(tie, axis=1).astype(f32))
    assert np.array_equal(be.indexreduce(0, tie.reshape(-1), mi, None, [0], C), np.argmax(tie, axis=0).astype(f32))
    assert np.array_equal(be.indexreduce(1, tie.reshape(-1), mi, None, [1], R), np.argmin(tie, axis=1).astype(f32))
    assert float(be.indexreduce_scalar(0, tie.reshape(-1), mi)) == float(np.argmax(tie))
    # all values below the start value -1e37: index 0 (the reference starts from -1e37, not -inf)
    low = np.full(8, -np.inf, f32)
    assert float(be.indexreduce_scalar(0, low, shape_info_np([1, 8]))) == 0.0
    # variance / standard deviation: two-pass float64
    for bias in (0, 1):
        assert_reduction_close(be.summarystats(0, bias, m, mi, [1], R), M.var(axis=1, ddof=bias), 0, "var dim1 bias %d" % bias)
        assert_reduction_close(be.summarystats(1, bias, m, mi, [0], C), M.std(axis=0, ddof=bias), 0, "std dim0 bias %d" % bias)
        assert_reduction_close([be.summarystats_scalar(0, bias, m, mi)], [M.var(ddof=bias)], 0, "var all bias %d" % bias)
    shifted = (m + f32(1000)).astype(f32)
    assert_reduction_close(be.summarystats(0, 0, shifted, mi, [1], R), shifted.reshape(R, C).astype(np.float64).var(axis=1), 0,
                           "var of shifted data")


def check_rng_closed_forms(be):
    """The buffer fill is textbook xoroshiro128+ seeded through splitmix64: recomputed here from the published
    recurrences; and the first `size` draws of a fresh generator are the buffer itself."""
    mask = (1 << 64) - 1

    def splitmix(x):
        x = (x + 0x9E3779B97F4A7C15) & mask
        z = x
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        return z ^ (z >> 31)

    def rotl(x, k):
        return ((x << k) | (x >> (64 - k))) & mask

    for seed, size in ((119, 64), (1, 33), (-7, 20)):
        s0 = splitmix(seed & mask)
        s1 = splitmix((seed * 119 + 3) & mask)
        want = []
        for _ in range(size):
            want.append((s0 + s1) & mask)
            s1 ^= s0
            s0 = rotl(s0, 55) ^ s1 ^ ((s1 << 14) & mask)
            s1 = rotl(s1, 36)
        g = be.rng(seed, size)
        assert [int(v) for v in g.buffer] == want, "buffer fill seed %d" % seed
        assert [int(v) for v in g.elements(0, size)] == want, "fresh draws are the buffer"
        # uniform [0,1): float(u64) / 2^64
        u = g.random_z(0, size, [0, 1])
        assert np.array_equal(u, (np.array(want, np.uint64).astype(np.float32) * np.float32(2.0 ** -64)))
        assert g.state()[1] == 0 and g.state()[3] == 2  # offset wrapped exactly once: generation 1 -> 2
        g.destroy()


# ---- data-movement specials: flatten, concat, pullRows, tear, shuffle, convertTypes ----------------------------
def _view(shape, order="c", strides=None):
    """(flat buffer of distinct values, shapeInfo, logical array) of a dense array or a strided view."""
    from libnd4j_amd.harness import element_offsets, shape_info, span_of
    info = shape_info(shape, order, strides)
    buf = np.arange(1, span_of(info) + 1, dtype=np.float64)
    logical = buf[element_offsets(info)].reshape(shape)
    return buf, info, logical


def _logical(buf, info):
    from libnd4j_amd.harness import element_offsets, info_shape
    return np.asarray(buf)[element_offsets(info)].reshape(info_shape(info))


def _cast(a, dt):
    """Values as the data type under test; for half they are folded into the range it holds exactly."""
    a = np.asarray(a)
    if np.dtype(dt) == np.float16:
        a = np.mod(a, 2039.0)
    return a.astype(dt)


def check_data_movement(be, dtypes=(np.float32, np.float64, np.float16), big=False, exact_sums=True):
    """Every result is compared bit for bit with what numpy says the operation means."""
    from libnd4j_amd.harness import shape_info, span_of
    rs = np.random.RandomState(77)
    for dt in dtypes:
        # flatten: the input read in the requested order, written from `offset` on
        cases = [([3, 4], "c", None), ([3, 4], "f", None), ([2, 3, 4], "c", None), ([2, 3, 4], "f", None),
                 ([5, 7], "c", [14, 1]), ([5, 7], "c", [1, 5]), ([4, 3, 5], "c", [40, 10, 2]), ([1, 9], "c", None)]
        if big:
            cases += [([700, 300], "c", None), ([700, 300], "f", None), ([64, 33, 17], "f", None)]
        for shape, order, strides in cases:
            buf, info, logical = _view(shape, order, strides)
            x = _cast(buf, dt)
            n = logical.size
            for want_order in "cf":
                got = be.flatten(3, want_order, x, info, n + 5)
                want = np.zeros(n + 5, dt)
                want[3:3 + n] = _cast(logical.ravel(order=want_order.upper()), dt)
                assert np.array_equal(got, want), ("flatten", shape, order, strides, want_order, np.dtype(dt).name)

        # concat along every dimension, equal and unequal extents, c- and f-order inputs and results
        ccases = [(0, [[2, 5], [3, 5], [1, 5]], "c", "c"), (1, [[4, 2], [4, 3]], "c", "c"), (1, [[4, 2], [4, 3]], "f", "c"),
                  (0, [[2, 3, 4], [5, 3, 4]], "c", "c"), (1, [[2, 3, 4], [2, 1, 4]], "c", "f"), (2, [[2, 3, 4], [2, 3, 2]], "f", "f"),
                  (1, [[1, 6], [1, 4], [1, 8]], "c", "c"), (0, [[1, 8]] * 9, "c", "c"), (1, [[1, 1]] * 5, "c", "c")]
        if big:
            ccases += [(0, [[200, 96]] * 12, "c", "c"), (1, [[300, 64], [300, 32], [300, 128]], "c", "c"),
                       (0, [[1, 4096]] * 300, "c", "c")]
        for dim, shapes, in_order, out_order in ccases:
            arrays, infos, logicals = [], [], []
            base = 0
            for shp in shapes:
                buf, info, logical = _view(shp, in_order)
                arrays.append(_cast(buf + base, dt))
                infos.append(info)
                logicals.append(_cast(logical + base, dt))
                base += buf.size
            want = np.concatenate(logicals, axis=dim)
            z_info = shape_info(list(want.shape), out_order)
            got = be.concat(dim, arrays, infos, z_info)
            assert np.array_equal(_logical(got, z_info), want), ("concat", dim, shapes, in_order, out_order, np.dtype(dt).name)

        # pullRows: z row i <- x row indexes[i]; rows of a c-order matrix (contiguous) and of an f-order one (strided),
        # and "rows" that are 2-D slices of a rank-3 array
        pcases = [([9, 6], "c", [1], "c"), ([9, 6], "f", [1], "c"), ([9, 6], "c", [1], "f"), ([7, 3, 4], "c", [1, 2], "c"),
                  ([7, 3, 4], "f", [1, 2], "f")]
        if big:
            pcases += [([500, 1024], "c", [1], "c"), ([300, 2052], "c", [1], "c"), ([400, 130], "f", [1], "c"),
                       ([6, 9000], "c", [1], "c"), ([5, 9001], "c", [1], "c")]  # long rows go in pieces
        for shape, order, dims, z_order in pcases:
            buf, info, logical = _view(shape, order)
            x = _cast(buf, dt)
            idx = rs.randint(0, shape[0], size=shape[0] + 3)
            z_shape = [len(idx)] + shape[1:]
            z_info = shape_info(z_shape, z_order)
            tad, z_tad = be.tad(info, dims), be.tad(z_info, dims)
            got = be.pullrows(x, info, z_info, idx, tad, z_tad)
            assert np.array_equal(_logical(got, z_info), _cast(logical[idx], dt)), ("pullRows", shape, order, dims, z_order)

        # tear: target r <- TAD r
        tcases = [([5, 8], "c", [1], [1, 8], "c"), ([5, 8], "f", [1], [1, 8], "c"), ([4, 3, 6], "c", [1, 2], [3, 6], "c"),
                  ([4, 3, 6], "c", [1, 2], [3, 6], "f"), ([4, 3, 6], "f", [1, 2], [3, 6], "f")]
        if big:
            tcases += [([40, 2048], "c", [1], [1, 2048], "c"), ([33, 20, 30], "c", [1, 2], [20, 30], "c"),
                       ([6, 9000], "c", [1], [1, 9000], "c"), ([5, 9001], "c", [1], [1, 9001], "c")]  # long TADs go in pieces
        for shape, order, dims, t_shape, t_order in tcases:
            buf, info, logical = _view(shape, order)
            x = _cast(buf, dt)
            z_info = shape_info(t_shape, t_order)
            tad = be.tad(info, dims)
            got = be.tear(x, info, z_info, tad)
            assert len(got) == shape[0]
            for r in range(shape[0]):
                assert np.array_equal(_logical(got[r], z_info), _cast(logical[r].reshape(t_shape), dt)), ("tear", shape, order, r)

        # shuffle: disjoint pairs of rows trade places in every array of the set
        scases = [[([8, 5], "c"), ([8, 3], "c")], [([8, 5], "f"), ([8, 2, 3], "c")]]
        if big:
            scases += [[([256, 1024], "c"), ([256, 10], "c"), ([256, 7], "f")]]
        for group in scases:
            rows = group[0][0][0]
            perm = rs.permutation(rows)
            smap = -np.ones(rows, np.int32)
            for a, b in zip(perm[0::2], perm[1::2]):
                smap[a] = b  # one entry per pair, the partner stays -1
            arrays, infos, tads, wants = [], [], [], []
            for shape, order in group:
                buf, info, logical = _view(shape, order)
                arrays.append(_cast(buf, dt))
                infos.append(info)
                tads.append(be.tad(info, list(range(1, len(shape)))))
                want = logical.copy()
                for a in range(rows):
                    if smap[a] >= 0:
                        want[[a, smap[a]]] = want[[smap[a], a]]
                wants.append(_cast(want, dt))
            got = be.shuffle(arrays, infos, smap, tads)
            for g, info, want in zip(got, infos, wants):
                assert np.array_equal(_logical(g, info), want), ("shuffle", group)

    # accumulate / average of n buffers: a running sum from zero in table order (one IEEE addition per term, which numpy
    # reproduces exactly for float and double), divided by n for the average; `exact_sums` is off for a checker that
    # orders or scales the terms differently (the reference's CPU loops) and for half, which the path sums in float
    for dt in dtypes:
        for n_arrays, length in ((3, 37), (8, 1024), (5, 4099)) + (((16, 300001),) if big else ()):
            arrays = [(rs.randn(length) * 3).astype(dt) for _ in range(n_arrays)]
            acc = np.zeros(length, np.float32 if dt == np.float16 else dt)
            for a in arrays:
                acc = acc + a.astype(acc.dtype)
            exact = exact_sums and dt != np.float16
            tol = 1e-2 if dt == np.float16 else (1e-5 if dt == np.float32 else 1e-12)
            # a running sum in half (the reference's kernels) loses up to 2^-11 of the partial sum per term
            scale = np.sum([np.abs(a.astype(np.float64)) for a in arrays], axis=0) + 1

            def same(got, want, what, div=1):
                if exact:
                    assert np.array_equal(got, want.astype(dt)), what
                else:
                    g, w = got.astype(np.float64), want.astype(np.float64)
                    assert np.all(np.abs(g - w) <= tol * scale / div), what

            same(be.accumulate(arrays), acc, ("accumulate", np.dtype(dt).name, n_arrays, length))
            mean = acc / acc.dtype.type(n_arrays)
            z, after = be.average(arrays, propagate=False)
            same(z, mean, ("average", np.dtype(dt).name, n_arrays, length), n_arrays)
            if exact_sums:  # the reference's CPU loop copies the average into every input whatever `propagate` says
                assert all(np.array_equal(a, b) for a, b in zip(after, arrays)), "average without propagate changed an input"
            z, after = be.average(arrays, propagate=True)
            same(z, mean, "average + propagate", n_arrays)
            assert all(np.array_equal(a, z) for a in after), "propagate"
            z, after = be.average(arrays, propagate=True, with_z=False)
            assert z is None
            for a in after:
                same(a, mean, "average into the inputs only", n_arrays)

    # conversions: z = (dst)(float)x
    codes = {np.dtype(np.float16): 3, np.dtype(np.float32): 6, np.dtype(np.float64): 7}
    vals = np.concatenate([rs.randn(1001) * 100, [0.0, -0.0, 1e-8, 65504.0, 70000.0, -1e10, 1e-40, np.inf, -np.inf, 3.14159265358979],
                           rs.randn(40) * 1e-6])
    if big:
        vals = np.concatenate([vals, rs.randn(200003)])
    for src in codes:
        for dst in codes:
            if src == dst:
                continue
            with np.errstate(over="ignore"):
                x = vals.astype(src)
                want = x.astype(np.float32).astype(dst)
            got = be.convert(codes[src], x, codes[dst])
            assert np.array_equal(got.view(np.dtype("u%d" % np.dtype(dst).itemsize)),
                                  want.view(np.dtype("u%d" % np.dtype(dst).itemsize))), ("convert", src, dst)


# ---- random views: every family on generated shapes, strides and dimensions, one implementation against another ------
def random_view(rs, shape=None):
    """A shapeInfo for `shape` (or for a random shape of rank 1-4): dense c, dense f, permuted dense strides, or permuted
    strides with padding between the dimensions.  A given shape is kept as it is.  Unit dimensions only appear in the
    dense kinds: the EWS field of a vector-shaped view is the stride of its last dimension whatever that dimension's
    extent (shape.h:1467), so an [n,1] view with arbitrary strides would describe memory its buffer does not have."""
    from libnd4j_amd import harness
    fixed = shape is not None
    if shape is None:
        rank = rs.randint(1, 5)
        shape = [int(rs.choice([1, 2, 3, 4, 5, 7, 8, 16, 33, 64, 100])) for _ in range(rank)]
        if rank == 1:
            shape = [1] + shape
    shape = [int(v) for v in shape]
    rank = len(shape)
    kind = rs.randint(0, 4)
    if fixed and any(v == 1 for v in shape):
        kind = rs.randint(0, 2)
    if kind < 2:
        return harness.shape_info(shape, "c" if kind == 0 else "f")
    shape = [max(2, v) for v in shape]
    strides = [0] * rank
    run = 1 if kind == 2 else int(rs.choice([1, 2, 3]))
    for d in rs.permutation(rank):
        strides[d] = run
        run *= shape[d] + (int(rs.randint(0, 3)) if kind == 3 else 0)
    info = harness.shape_info(shape, "c" if rs.rand() < 0.5 else "f", strides=strides)
    offsets = harness.element_offsets(info)
    assert 0 <= offsets.min() and offsets.max() < harness.span_of(info)
    return info


def check_random_views(be, ref, seed, cases, dtype=np.float32):
    """`be` against `ref` (two backends of tests/backends.py) on `cases` generated calls.  Elementwise results within
    ELEMENTWISE_ULP (pairwise and scalar arithmetic exactly), nothing written outside the result's view; reductions
    within REDUCE_RTOL of the result plus the rounding of the summed magnitudes; index reductions (on distinct values)
    exactly.  `dtype` float16: the reductions and statistics are left out (the reference accumulates them in half), and
    so are the index reductions (a half does not hold a few thousand distinct integers)."""
    from libnd4j_amd import harness
    rs = np.random.RandomState(seed)
    done = {}

    def kw(**k):  # the GPU backend can be told to withhold the caller's TAD tables; the CPU ones have no such switch
        return k if getattr(be, "kind", "") == "hip" else {}

    for _ in range(cases):
        xi = random_view(rs)
        shape = [int(v) for v in harness.info_shape(xi)]
        n, rank = int(np.prod(shape)), len(shape)
        x = rs.uniform(-3, 3, harness.span_of(xi)).astype(dtype)
        what = int(rs.randint(0, 8))
        if dtype == np.float16 and what in (2, 3, 4):
            continue
        if what == 7:
            # broadcast of a dense sub-array along several dimensions
            if rank < 3:
                continue
            k = int(rs.randint(2, rank))
            dims = sorted(int(d) for d in rs.choice(rank, size=k, replace=False))
            yshape = [shape[d] for d in dims]
            yi = harness.shape_info(yshape, "c")
            y = rs.uniform(-3, 3, int(np.prod(yshape))).astype(dtype)
            op = int(rs.choice([0, 1, 2, 3]))
            g = be.broadcast(op, x, xi, y, yi, xi, dims, **kw(pass_tads=bool(rs.randint(0, 2))))
            c = ref.broadcast(op, x, xi, y, yi, xi, dims)
            sel = harness.element_offsets(xi)
            assert ulp_distance(g[sel], c[sel]).max() <= 1, ("broadcast", op, dims, list(xi))
            assert np.array_equal(np.delete(g, sel), np.delete(c, sel)), ("broadcast wrote outside its view", dims, list(xi))
        elif what == 0:
            # (double and half: single IEEE operations only - Abs, Ceiling, Floor, Neg; the library functions are held to
            # their bars where the op vectors test them)
            zi, op = random_view(rs, shape), int(rs.choice([0, 3, 15, 6, 10, 23, 42] if dtype == np.float32 else [0, 1, 4, 6]))
            g, c = be.transform(op, x, xi, zi), ref.transform(op, x, xi, zi)
            sel = harness.element_offsets(zi)
            assert ulp_distance(g[sel], c[sel]).max() <= ELEMENTWISE_ULP, ("transform", op, list(xi), list(zi))
            assert np.all(np.delete(g, sel) == 0), ("transform wrote outside its view", list(zi))
        elif what == 1:
            yi, zi, op = random_view(rs, shape), random_view(rs, shape), int(rs.choice([0, 1, 2, 6, 13]))
            y = rs.uniform(-3, 3, harness.span_of(yi)).astype(dtype)
            g, c = be.pairwise(op, x, xi, y, yi, zi), ref.pairwise(op, x, xi, y, yi, zi)
            sel = harness.element_offsets(zi)
            assert np.array_equal(g[sel], c[sel]), ("pairwise", op, list(xi), list(yi), list(zi))
            assert np.all(np.delete(g, sel) == 0), ("pairwise wrote outside its view", list(zi))
        elif what in (2, 3, 4):
            k = int(rs.randint(1, rank + 1)) if rank > 1 else 1
            dims = sorted(int(d) for d in rs.choice(rank, size=min(k, rank), replace=False))
            out_len = n // int(np.prod([shape[d] for d in dims]))
            if what == 2:
                op = int(rs.choice([0, 1, 3, 4, 5]))
                g = be.reduce(op, x, xi, None, dims, out_len, **kw(pass_tads=bool(rs.randint(0, 2))))
                c = ref.reduce(op, x, xi, None, dims, out_len)
                scale = np.abs(x).sum() / max(1, out_len)
                # (the reference adds a TAD up in float, one element after the other: over millions of elements its own
                # result is off by some sqrt(length) roundings - 4e-5 was seen on 2.9 M elements where the device's sum was
                # within 5e-8 of the float64 one - so the bar widens with the TAD's length)
                drift = 2.0 * np.sqrt(n / max(1, out_len)) * 6e-8
                assert np.all(np.abs(g.astype(np.float64) - c) <= (2 * REDUCE_RTOL + drift) * np.abs(c) + (2e-6 + drift) * scale), ("reduce", op, dims, list(xi))
            elif what == 3:
                xu = rs.permutation(harness.span_of(xi)).astype(dtype)  # distinct values: no ties to resolve
                op = int(rs.choice([0, 1]))
                assert np.array_equal(be.indexreduce(op, xu, xi, None, dims, out_len), ref.indexreduce(op, xu, xi, None, dims, out_len)), (
                    "indexreduce", op, dims, list(xi))
            else:
                if len(dims) != 1 and out_len > 1:
                    continue  # the reference's summary statistics take one dimension (or all of them)
                g, c = be.summarystats(0, True, x, xi, dims, out_len), ref.summarystats(0, True, x, xi, dims, out_len)
                assert np.allclose(g, c, rtol=2 * REDUCE_RTOL, atol=1e-6), ("summarystats", dims, list(xi))
        elif what == 5:
            if rank < 2:
                continue
            d = int(rs.randint(0, rank))
            yi = harness.shape_info([1, shape[d]])
            y = rs.uniform(-3, 3, shape[d]).astype(dtype)
            op = int(rs.choice([0, 1, 2, 3]))
            g = be.broadcast(op, x, xi, y, yi, xi, [d], **kw(pass_tads=bool(rs.randint(0, 2))))
            c = ref.broadcast(op, x, xi, y, yi, xi, [d])
            sel = harness.element_offsets(xi)
            assert ulp_distance(g[sel], c[sel]).max() <= 1, ("broadcast", op, d, list(xi))
        else:
            zi, op = random_view(rs, shape), int(rs.choice([0, 1, 2]))
            g, c = be.scalar(op, x, xi, zi, 1.5), ref.scalar(op, x, xi, zi, 1.5)
            sel = harness.element_offsets(zi)
            assert np.array_equal(g[sel], c[sel]), ("scalar", op, list(xi), list(zi))
        done[what] = done.get(what, 0) + 1
    return done


# ---- whole-array transforms: Col2Im 36, Im2col 37, Histogram 48, Reverse 70, Pooling2D 71 ------------------------------
def _strided_info(rs, shape, kind):
    """dense c (0), dense f (1), permuted dense strides (2) or permuted strides with padding (3) for `shape`."""
    from libnd4j_amd import harness
    shape = [int(v) for v in shape]
    if kind < 2 or any(v == 1 for v in shape):
        return harness.shape_info(shape, "c" if kind != 1 else "f")
    strides = [0] * len(shape)
    run = 1
    for d in rs.permutation(len(shape)):
        strides[d] = run
        run *= shape[d] + (int(rs.randint(0, 3)) if kind == 3 else 0)
    return harness.shape_info(shape, "c" if rs.rand() < 0.5 else "f", strides=strides)


def _conv_geometry(rs):
    kH, kW = int(rs.randint(1, 4)), int(rs.randint(1, 4))
    sH, sW = int(rs.randint(1, 3)), int(rs.randint(1, 3))
    dH, dW = int(rs.randint(1, 3)), int(rs.randint(1, 3))
    pH, pW = int(rs.randint(0, 3)), int(rs.randint(0, 3))
    kHe, kWe = kH + (kH - 1) * (dH - 1), kW + (kW - 1) * (dW - 1)
    iH, iW = int(rs.randint(kHe, kHe + 9)), int(rs.randint(kWe, kWe + 9))
    oH, oW = (iH + 2 * pH - kHe) // sH + 1, (iW + 2 * pW - kWe) // sW + 1
    return kH, kW, sH, sW, pH, pW, dH, dW, iH, iW, oH, oW


def check_whole_array_transforms(be, ref, seed, cases, dtypes=(np.float32, np.float64)):
    """`be` against `ref` on generated calls of the five whole-array transforms.  Reverse, Im2col and Col2Im (sums in
    the reference's order) exactly, over the whole result buffer; Histogram counts exactly; Pooling2D: max exactly,
    average and p-norm within REDUCE_RTOL (the reference's window sums are re-associated by its build)."""
    from libnd4j_amd import harness
    rs = np.random.RandomState(seed)
    done = {}
    for it in range(cases):
        dt = dtypes[it % len(dtypes)]
        what = int(rs.randint(0, 5))
        if what == 0:  # Reverse
            shape = [int(rs.choice([1, 2, 3, 4, 5, 7, 8, 16, 33, 64])) for _ in range(int(rs.randint(1, 4)))]
            if len(shape) == 1:
                shape = [1] + shape
            xi = _strided_info(rs, shape, int(rs.randint(0, 4)))
            x = rs.uniform(-3, 3, harness.span_of(xi)).astype(dt)
            if rs.rand() < 0.4:
                g, c = be.transform_inplace(70, x, xi), ref.transform_inplace(70, x, xi)
            else:
                zi = _strided_info(rs, shape, int(rs.randint(0, 4)))
                g, c = be.transform(70, x, xi, zi), ref.transform(70, x, xi, zi)
            assert np.array_equal(g, c), ("reverse", list(xi), it)
        elif what == 1:  # Histogram
            # half holds counts up to 2048 exactly; beyond that the reference's result depends on which of its two
            # threads adds its share first
            n = int(rs.choice([1, 5, 64, 1000, 4099, 70001] if np.dtype(dt) != np.float16 else [1, 5, 64, 1000, 2000]))
            bins = int(rs.choice([1, 2, 7, 64, 1000, 5000]))
            x = rs.uniform(-3, 3, n).astype(dt)
            lo, hi = (float(x.min()), float(x.max())) if rs.rand() < 0.5 else (-2.0, 2.5)
            if lo == hi:
                hi = lo + 1.0
            extra = np.array([bins, lo, hi], dtype=dt)
            z0 = np.floor(rs.uniform(0, 4, bins)).astype(dt)
            xi, zi = harness.shape_info([1, n]), harness.shape_info([1, bins])
            g, c = be.transform(48, x, xi, zi, extra, z=z0), ref.transform(48, x, xi, zi, extra, z=z0)
            assert np.array_equal(g, c), ("histogram", n, bins, lo, hi, np.dtype(dt).name, it, np.nonzero(g != c)[0][:4])
        else:
            kH, kW, sH, sW, pH, pW, dH, dW, iH, iW, oH, oW = _conv_geometry(rs)
            bS, iC = int(rs.randint(1, 4)), int(rs.randint(1, 5))
            img, col, pooled = [bS, iC, iH, iW], [bS, iC, kH, kW, oH, oW], [bS, iC, oH, oW]
            if what == 2:  # Im2col
                xi, zi = _strided_info(rs, img, int(rs.randint(0, 4))), _strided_info(rs, col, int(rs.randint(0, 4)))
                x = rs.uniform(-3, 3, harness.span_of(xi)).astype(dt)
                extra = np.array([kH, kW, sH, sW, pH, pW, dH, dW, 0, 0], dtype=dt)
                z0 = np.full(harness.span_of(zi), 9, dt)
                g, c = be.transform(37, x, xi, zi, extra, z=z0), ref.transform(37, x, xi, zi, extra, z=z0)
                assert np.array_equal(g, c), ("im2col", list(xi), list(zi), list(extra), it)
            elif what == 3:  # Col2Im
                xi, zi = _strided_info(rs, col, int(rs.randint(0, 4))), _strided_info(rs, img, int(rs.randint(0, 4)))
                x = rs.uniform(-3, 3, harness.span_of(xi)).astype(dt)
                extra = np.array([sH, sW, pH, pW, iH, iW, dH, dW], dtype=dt)
                z0 = np.full(harness.span_of(zi), 9, dt)
                g, c = be.transform(36, x, xi, zi, extra, z=z0), ref.transform(36, x, xi, zi, extra, z=z0)
                assert np.array_equal(g, c), ("col2im", list(xi), list(zi), list(extra), it)
            else:  # Pooling2D
                mode = int(rs.randint(0, 3))
                p0 = float(rs.randint(0, 2)) if mode == 1 else float(rs.choice([1.0, 2.0, 3.0]))
                xi = _strided_info(rs, img, int(rs.randint(0, 4)))
                zi = harness.shape_info(pooled, "c" if rs.rand() < 0.6 else "f")
                x = rs.uniform(-3, 3, harness.span_of(xi)).astype(dt)
                extra = np.array([kH, kW, sH, sW, pH, pW, dH, dW, 0, mode, p0], dtype=dt)
                g, c = be.transform(71, x, xi, zi, extra), ref.transform(71, x, xi, zi, extra)
                if mode == 0:
                    assert np.array_equal(g, c), ("maxpool", list(xi), list(zi), list(extra), it)
                else:
                    ok = np.isclose(g, c, rtol=REDUCE_RTOL if np.dtype(dt) != np.float16 else HALF_RTOL, atol=1e-6, equal_nan=True)
                    assert ok.all(), ("pool", mode, list(xi), list(zi), list(extra), it, g[~ok][:3], c[~ok][:3])
        done[what] = done.get(what, 0) + 1
    return done


def check_whole_array_vectors(be):
    """The fixed calls of golden_inputs.whole_array_cases against what the compiled reference wrote for them."""
    from golden_inputs import whole_array_cases
    vec = load_json("ref_vectors.json")["ops"]["whole_array_f32"]
    for name, op, x, x_info, z_info, extra, z0 in whole_array_cases():
        want = from_hexbits(vec[name], np.float32)
        got = be.transform(op, x, x_info, z_info, extra, z=z0)
        if name.startswith("pool_") and name != "pool_max":
            assert np.allclose(got, want, rtol=REDUCE_RTOL, atol=0), name
        else:
            assert np.array_equal(got, want), name


def check_whole_array_closed_forms(be):
    """The whole-array transforms against plain numpy on integer-valued data (so that no sum depends on its order)."""
    rs = np.random.RandomState(77)
    f = np.float32
    # Reverse
    x = rs.randint(-50, 50, 24).astype(f)
    vi, mi = shape_info_np([1, 24]), shape_info_np([4, 6])
    assert np.array_equal(be.transform(70, x, vi, vi), x[::-1])
    assert np.array_equal(be.transform(70, x, mi, mi), x[::-1])
    assert np.array_equal(be.transform_inplace(70, x, vi), x[::-1])
    assert np.array_equal(be.transform_inplace(70, x[:23].copy(), shape_info_np([1, 23])), x[:23][::-1])
    # Histogram: values in the middle of their bins, two outliers clamped into the outer bins, counts added onto z
    bins, lo, hi = 8, -4.0, 4.0
    idx = rs.randint(0, bins, 500)
    x = (lo + (idx + 0.5) * (hi - lo) / bins).astype(f)
    x[:2] = [-100.0, 100.0]
    idx[:2] = [0, bins - 1]
    z0 = np.arange(bins, dtype=f)
    got = be.transform(48, x, shape_info_np([1, 500]), shape_info_np([1, bins]), np.array([bins, lo, hi], f), z=z0)
    assert np.array_equal(got, z0 + np.bincount(idx, minlength=bins)), "histogram"
    # Im2col / Col2Im / Pooling2D
    bS, iC, iH, iW, kH, kW, sH, sW, pH, pW, dH, dW = 2, 3, 8, 7, 3, 2, 2, 1, 1, 1, 1, 2
    kHe, kWe = kH + (kH - 1) * (dH - 1), kW + (kW - 1) * (dW - 1)
    oH, oW = (iH + 2 * pH - kHe) // sH + 1, (iW + 2 * pW - kWe) // sW + 1
    img = rs.randint(-9, 10, (bS, iC, iH, iW)).astype(f)
    padded = np.zeros((bS, iC, iH + 2 * pH + sH * oH + kHe, iW + 2 * pW + sW * oW + kWe), f)
    padded[:, :, pH:pH + iH, pW:pW + iW] = img
    col = np.zeros((bS, iC, kH, kW, oH, oW), f)
    for kr in range(kH):
        for kc in range(kW):
            for r in range(oH):
                for q in range(oW):
                    col[:, :, kr, kc, r, q] = padded[:, :, kr * dH + r * sH, kc * dW + q * sW]
    ii, ci = shape_info_np([bS, iC, iH, iW]), shape_info_np([bS, iC, kH, kW, oH, oW])
    e = np.array([kH, kW, sH, sW, pH, pW, dH, dW, 0, 0], f)
    assert np.array_equal(be.transform(37, img.ravel(), ii, ci, e), col.ravel()), "im2col"
    cols = rs.randint(-9, 10, col.shape).astype(f)
    back = np.zeros_like(padded)
    for kr in range(kH):
        for kc in range(kW):
            for r in range(oH):
                for q in range(oW):
                    back[:, :, kr * dH + r * sH, kc * dW + q * sW] += cols[:, :, kr, kc, r, q]
    e = np.array([sH, sW, pH, pW, iH, iW, dH, dW], f)
    assert np.array_equal(be.transform(36, cols.ravel(), ci, ii, e, z=np.full(img.size, 5, f)),
                          back[:, :, pH:pH + iH, pW:pW + iW].ravel()), "col2im"
    pi = shape_info_np([bS, iC, oH, oW])
    inside = np.zeros_like(padded)
    inside[:, :, pH:pH + iH, pW:pW + iW] = 1
    mx = np.full((bS, iC, oH, oW), -1e37, f)
    sm = np.zeros((bS, iC, oH, oW), np.float64)
    sq = np.zeros((bS, iC, oH, oW), np.float64)
    cnt = np.zeros((bS, iC, oH, oW), np.float64)
    for kr in range(kH):
        for kc in range(kW):
            for r in range(oH):
                for q in range(oW):
                    v, ok = padded[:, :, kr * dH + r * sH, kc * dW + q * sW], inside[:, :, kr * dH + r * sH, kc * dW + q * sW]
                    mx[:, :, r, q] = np.where(ok > 0, np.maximum(mx[:, :, r, q], v), mx[:, :, r, q])
                    sm[:, :, r, q] += v
                    sq[:, :, r, q] += v.astype(np.float64) ** 2
                    cnt[:, :, r, q] += ok

    def pool(mode, p0):
        return be.transform(71, img.ravel(), ii, pi, np.array([kH, kW, sH, sW, pH, pW, dH, dW, 0, mode, p0], f))
    assert np.array_equal(pool(0, 0), mx.ravel()), "max pooling"
    assert np.allclose(pool(1, 0), (sm / cnt).ravel(), rtol=1e-6, atol=0), "average over the cells inside the image"
    assert np.allclose(pool(1, 1), (sm / (kH * kW)).ravel(), rtol=1e-6, atol=0), "average over the kernel"
    assert np.allclose(pool(2, 2), np.sqrt(sq).ravel(), rtol=1e-6, atol=0), "2-norm pooling"


# ---- Choice (random op 5) ---------------------------------------------------------------------------------------------
def check_choice(be, ref, seed=5):
    """Choice on `be` against `ref`: the element-wise-stride branch on dense and strided vectors, and the coordinate
    branch (which indexes the probabilities with the result's index, so it is only defined while there are no more
    results than probabilities).  Results and generator state exactly."""
    from libnd4j_amd import harness
    rs = np.random.RandomState(seed)
    for dt in (np.float32, np.float64, np.float16):
        a, b = be.rng(119, 1 << 12), ref.rng(119, 1 << 12)
        for n_vals, n_out in ((4, 500), (1, 17), (37, 4099), (256, 70001)):
            probs = rs.uniform(0.1, 1, n_vals)
            probs = (probs / probs.sum()).astype(dt)
            vals = (np.arange(n_vals) * 3 + 10).astype(dt)
            vi, zi = harness.shape_info([1, n_vals]), harness.shape_info([1, n_out])
            assert np.array_equal(a.choice(vals, vi, probs, vi, zi), b.choice(vals, vi, probs, vi, zi)), ("choice", n_vals, n_out, dt)
            assert a.state() == b.state()
        # strided vectors: values and probabilities every third / second element, results every second
        n_vals, n_out = 9, 301
        vi = harness.shape_info([1, n_vals], strides=[1, 3], ews=3)
        pi = harness.shape_info([1, n_vals], strides=[1, 2], ews=2)
        zi = harness.shape_info([1, n_out], strides=[1, 2], ews=2)
        vals = rs.uniform(-5, 5, harness.span_of(vi)).astype(dt)
        probs = np.full(harness.span_of(pi), 1.0 / n_vals, dt)
        assert np.array_equal(a.choice(vals, vi, probs, pi, zi), b.choice(vals, vi, probs, pi, zi)), ("choice strided", dt)
        # no element-wise stride on the result: the coordinate branch
        zi = harness.shape_info([3, 4], "c", strides=[1, 5])
        vi = harness.shape_info([4, 5], "f")
        vals = rs.uniform(-5, 5, 20).astype(dt)
        probs = rs.uniform(0.02, 0.2, 20).astype(dt)
        assert harness.info_numel(zi) <= 20
        assert np.array_equal(a.choice(vals, vi, probs, vi, zi), b.choice(vals, vi, probs, vi, zi)), ("choice by coordinates", dt)
        assert a.state() == b.state()
        a.destroy()
        b.destroy()
