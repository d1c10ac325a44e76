"""Deterministic inputs and op lists shared by tests/golden/make_vectors.py and the tests that replay its
vectors.  Everything is generated arithmetically (no RNG library), so the same values come out anywhere."""
import numpy as np

# opNum tables (reference: include/loops/legacy_ops.h); ops without a scalar functor are left out of the
# transform list: 36-41 (col2im, im2col, softmax family, IsMax), 43/44 (unseeded dropout), 48, 70, 71
TRANSFORM_OPS = [o for o in range(0, 97) if o not in (36, 37, 38, 39, 40, 41, 43, 44, 48, 56, 57, 58, 60, 69, 70, 71)]
PAIRWISE_OPS = list(range(0, 29)) + [45, 46, 56, 57, 58, 59, 60, 69, 92, 93, 94]
BROADCAST_OPS = list(range(0, 24))
SCALAR_OPS = list(range(0, 24))
SCALAR_VALUES = [1.7, -2.25]
REDUCE_OPS = [0, 1] + list(range(3, 27))
INDEX_OPS = list(range(0, 6))
RANDOM_PLAIN_OPS = [0, 1, 2, 3, 4, 7, 12, 13]

DEFAULT_EXTRA = [0.5, 0.25, 2.0, 3.0]


def op_extra(family, op, dtype=np.float32):
    """extraParams used for every op of a family: [0.5, 0.25, 2.0, 3.0] gives each parameterised op something
    sensible (compare 0.5 / eps 0.25 / mode 2 for MatchCondition; compare 0.5, set 0.25, eps 2, mode 3 for the
    CompareAndSet family; exponent 0.5 for NormP ...).  Pow and LogX get their own so results stay finite."""
    e = list(DEFAULT_EXTRA)
    if family == "transform":
        if op == 7:
            e = [2.0, 0, 0, 0]
        elif op == 55:
            e = [3.0, 0, 0, 0]
        elif op == 73:
            e = [-1.0, 1.5, 0, 0]
        elif op == 9:
            e = [-0.5, 1.5, 0, 0]
        elif op == 92:
            e = [3.0, 0, 0, 0]
    return np.array(e, dtype=dtype)


def shape_info_np(shape, order="c"):
    """Dense shapeInfo; mirrors libnd4j_amd.harness.shape_info without importing the package."""
    shape = [int(s) for s in shape]
    rank = len(shape)
    vec = rank == 1 or (rank == 2 and (shape[0] == 1 or shape[1] == 1))
    if vec:
        strides = [1] * rank
    else:
        strides = [0] * rank
        acc = 1
        for i in (range(rank) if order == "f" else range(rank - 1, -1, -1)):
            strides[i] = acc
            acc *= shape[i]
    if vec:
        ews = strides[-1]
    else:
        dims = [(s, t) for s, t in zip(shape, strides) if s != 1]
        ews = dims[-1][1] if dims else strides[-1]
        for k in range(len(dims) - 1):
            if dims[k][1] != dims[k + 1][0] * dims[k + 1][1]:
                ews = -1
    return np.array([rank] + shape + strides + [0, ews, ord(order)], dtype=np.int64)


def transform_input():
    """120 float32 values: a sweep over [-4, 4], small magnitudes, exact integers and halves, a few large."""
    v = [(-4.0 + 8.0 * k / 63.0) for k in range(64)]
    v += [0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 2.5, -2.5, 1.5, -1.5, 0.25, 3.0, -3.0, 6.5]
    v += [1e-3, -1e-3, 1e-6, -1e-6, 1e-12, 3.3e-5, 0.999, 1.001, -0.999, 0.7071, 0.1, 0.2, 0.3, 0.9, -0.9, 0.01]
    v += [10.0, -10.0, 20.5, -20.5, 50.0, 87.0, -87.0, 100.0, 0.4999, 0.5001, 7.25, -7.75, 12.0, 15.0, 33.3, -44.4]
    v += [1.25, 1.75, 2.25, 2.75, 3.25, 3.75, 0.75, 0.125]
    return np.array(v, dtype=np.float32)


def pairwise_inputs():
    """Two float32 vectors of 96 values with magnitudes >= 1.2 (integer casts never hit zero) and mixed signs."""
    k = np.arange(96, dtype=np.float64)
    a = (1.25 + (k * 0.37) % 7.5) * np.where(k % 3 == 0, -1.0, 1.0)
    b = (1.5 + (k * 0.61) % 4.25) * np.where(k % 5 == 0, -1.0, 1.0)
    a[10] = b[10]
    a[20] = b[20]
    a[30] = -b[30]
    return a.astype(np.float32), b.astype(np.float32)


def reduce_input():
    """12 x 10 float32 matrix (flattened, c order) in about [-3, 3] with repeated maxima, zeros and 0.5s."""
    k = np.arange(120, dtype=np.float64)
    m = ((k * 0.7919) % 6.0) - 3.0
    m[::17] = 0.0
    m[5] = m[3]
    m[25] = 2.9
    m[27] = 2.9
    m[61] = 0.5
    m[99] = -2.95
    m[109] = -2.95
    return m.astype(np.float32)


def hexbits(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float32:
        return "".join("%08x" % int(v) for v in a.view(np.uint32))
    if a.dtype == np.float16:
        return "".join("%04x" % int(v) for v in a.view(np.uint16))
    if a.dtype == np.float64:
        return "".join("%016x" % int(v) for v in a.view(np.uint64))
    raise TypeError(a.dtype)


def from_hexbits(s, dtype):
    dtype = np.dtype(dtype)
    w = dtype.itemsize * 2
    ints = [int(s[i:i + w], 16) for i in range(0, len(s), w)]
    u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[dtype.itemsize]
    return np.array(ints, dtype=u).view(dtype)


def ulp_distance(a, b):
    """Element-wise distance in units in the last place between two float32/float16 arrays; NaN vs NaN is 0,
    +0 vs -0 is 0."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    if a.dtype == np.float32:
        ia, ib, sign = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64), 0x7fffffff
    elif a.dtype == np.float16:
        ia, ib, sign = a.view(np.int16).astype(np.int64), b.view(np.int16).astype(np.int64), 0x7fff
    else:
        ia, ib, sign = a.view(np.int64), b.view(np.int64), 0x7fffffffffffffff
    ia = np.where(ia < 0, -(ia & sign), ia)
    ib = np.where(ib < 0, -(ib & sign), ib)
    d = np.abs(ia - ib)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


def whole_array_cases():
    """Fixed calls of the whole-array transforms (Col2Im 36, Im2col 37, Histogram 48, Reverse 70, Pooling2D 71):
    (name, opNum, x, x_info, z_info, extraParams, initial z).  Dense c-order float32 arrays, values from the same
    arithmetic sweep as the other inputs."""
    def values(n, scale=6.0):
        k = np.arange(n, dtype=np.float64)
        return (((k * 0.7919) % scale) - scale / 2).astype(np.float32)

    f = np.float32
    cases = []
    img, col, pooled = [2, 3, 7, 6], [2, 3, 3, 2, 4, 3], [2, 3, 4, 3]
    ii, ci, pi = shape_info_np(img), shape_info_np(col), shape_info_np(pooled)
    n_img, n_col, n_pool = int(np.prod(img)), int(np.prod(col)), int(np.prod(pooled))
    # kH 3, kW 2, stride 2 x 2, padding 1 x 1, dilation 1 x 2: oH = (7 + 2 - 3) / 2 + 1 = 4, oW = (6 + 2 - 3) / 2 + 1 = 3
    cases.append(("im2col", 37, values(n_img), ii, ci, np.array([3, 2, 2, 2, 1, 1, 1, 2, 0, 0], f), np.full(n_col, 9, f)))
    cases.append(("col2im", 36, values(n_col), ci, ii, np.array([2, 2, 1, 1, 7, 6, 1, 2], f), np.full(n_img, 9, f)))
    for name, mode, p0 in (("pool_max", 0, 0), ("pool_avg_inside", 1, 0), ("pool_avg_kernel", 1, 1), ("pool_pnorm2", 2, 2)):
        cases.append((name, 71, values(n_img), ii, pi, np.array([3, 2, 2, 2, 1, 1, 1, 2, 0, mode, p0], f), np.zeros(n_pool, f)))
    x = values(1000)
    cases.append(("histogram", 48, x, shape_info_np([1, 1000]), shape_info_np([1, 16]), np.array([16, -2.5, 2.75], f),
                  np.arange(16, dtype=f)))
    cases.append(("reverse_vector", 70, values(37), shape_info_np([1, 37]), shape_info_np([1, 37]), None, np.zeros(37, f)))
    cases.append(("reverse_matrix_c_to_f", 70, values(35), shape_info_np([5, 7]), shape_info_np([5, 7], "f"), None, np.zeros(35, f)))
    return cases


def half_reduction_input():
    """192 fp16 values in [0.5, 1.5) (a [12, 16] matrix): short enough that sums accumulated in fp16, as the reference's
    float16 loops accumulate them, stay within a few 1e-3 of the exact ones."""
    return (0.5 + np.random.RandomState(5).rand(192)).astype(np.float16)
