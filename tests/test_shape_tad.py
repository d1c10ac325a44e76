"""Host-side shapeInfo / TAD logic of the product (NativeOps::tadOnlyShapeInfo through the C ABI; no GPU is
touched) against the reference's TAD / shape test fixtures, vectors of the compiled reference and - when it was
built - the compiled reference on random shapes."""
import itertools
import random

import numpy as np

import checks
from libnd4j_amd import harness
from libnd4j_amd.native import NativeOps


def _product_tad(x_info, dims):
    ops = NativeOps()
    x_info = np.ascontiguousarray(x_info, np.int64)
    d = np.array(list(dims), np.int32)
    rank = int(x_info[0])
    n = harness.info_numel(x_info)
    tl = 1
    for k in dims:
        tl *= int(x_info[1 + k])
    num = n // tl if tl else 0
    target = np.full(2 * max(rank, 2) + 8, -12345, np.int64)
    off = np.zeros(max(num, 1), np.int64)
    ops.tadOnlyShapeInfo(x_info.ctypes.data, d.ctypes.data, len(dims), target.ctypes.data, off.ctypes.data)
    r = int(target[0])
    assert np.all(target[2 * r + 4:] == -12345), "wrote past the shapeInfo"
    return target[:2 * r + 4].copy(), off[:num].copy()


def test_fixtures_and_vectors():
    checks.check_tad_fixtures(_product_tad)


def test_shape_info_builder_matches_reference(reference_lib):
    rnd = random.Random(3)
    for _ in range(300):
        rank = rnd.randint(1, 5)
        shape = [rnd.choice([1, 2, 3, 4, 7]) for _ in range(rank)]
        order = rnd.choice("cf")
        assert np.array_equal(harness.shape_info(shape, order), reference_lib.shape_buffer(shape, order)), (shape, order)


def test_ews_matches_reference(reference_lib):
    rnd = random.Random(4)
    for _ in range(500):
        rank = rnd.randint(1, 4)
        shape = [rnd.choice([1, 2, 3, 5]) for _ in range(rank)]
        strides = [rnd.choice([1, 2, 3, 5, 6, 10, 15, 30]) for _ in range(rank)]
        for f in (False, True):
            assert harness.compute_ews(shape, strides, f) == reference_lib.compute_ews(shape, strides, f), (shape, strides, f)


def test_random_tads_match_reference(reference_lib):
    rnd = random.Random(1)
    for _ in range(1500):
        rank = rnd.randint(1, 5)
        shape = [rnd.choice([1, 2, 3, 4, 5]) for _ in range(rank)]
        order = rnd.choice("cf")
        dims = sorted(rnd.sample(range(rank), rnd.randint(1, rank)))
        info = harness.shape_info(shape, order)
        a = reference_lib.tad(info, dims)
        b = _product_tad(info, dims)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), (shape, order, dims, a[0], b[0])


def test_views_match_reference(reference_lib):
    # permuted and strided views, as ND4J hands them over (EWS -1 or a plain stride)
    rnd = random.Random(2)
    for _ in range(600):
        rank = rnd.randint(2, 4)
        shape = [rnd.choice([2, 3, 4]) for _ in range(rank)]
        base = harness.dense_strides(shape, "c")
        perm = list(range(rank))
        rnd.shuffle(perm)
        shp = [shape[p] for p in perm]
        st = [base[p] * rnd.choice([1, 1, 2]) for p in perm]
        info = harness.shape_info(shp, "c", strides=st)
        dims = sorted(rnd.sample(range(rank), rnd.randint(1, rank - 1)))
        a = reference_lib.tad(info, dims)
        b = _product_tad(info, dims)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), (shp, st, dims, a[0], b[0])
