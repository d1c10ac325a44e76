"""The whole-array reduce that allocates nothing (nd4j_amd_execReduceFloatNoAlloc) against the entry point it is a
variant of (nd4j_execReduceFloatFull, i.e. execReduceFloat without dimensions), through the C ABI: the same bits in
result[0], on two calls in a row of which the second has the smaller input (the scratch array keeps the first call's
partial results), for several ops and layouts; and the inputs it must refuse."""
import numpy as np
import pytest

from libnd4j_amd import harness
from libnd4j_amd.native import Nd4jError

pytestmark = pytest.mark.gpu

SUM, MAX, NORM2, LOGSUMEXP = 1, 3, 6, 19


def _both(dev, op, x, info):
    """(result of the existing entry point, result of the no-allocation one) as raw 32-bit patterns"""
    X = harness.Operand(dev, x, info)
    zi = harness.shape_info([1, 1])
    out = []
    for member in ("execReduceFloatFull", "amd_execReduceFloatNoAlloc"):
        Z = harness.Operand(dev, np.full(1, np.float32(-777.0)), zi)
        extra = dev.extra(info, z_info=zi)
        if member == "execReduceFloatFull":
            dev.ops.execReduceFloatFull(extra, op, X.ptr, X.info_ptr, None, Z.ptr, Z.info_ptr)
        else:
            dev.ops.amd_execReduceFloatNoAlloc(extra, op, X.ptr, X.info_ptr, None, Z.ptr)
        out.append(Z.get().view(np.uint32)[0])
        Z.free()
    X.free()
    dev.release()
    return out


def test_no_alloc_reduce_matches_the_allocating_entry_point():
    dev = harness.Device()
    rs = np.random.RandomState(5)
    # (elements of the first call, elements of the second, smaller, call)
    for big, small in (((1 << 22) + 3, 70001), (1 << 20, 1000), (300000, 17)):
        for op in (SUM, MAX, NORM2, LOGSUMEXP):
            for n in (big, small):
                x = rs.uniform(-3, 3, n).astype(np.float32)
                want, got = _both(dev, op, x, harness.shape_info([1, n]))
                assert want == got, (op, n, hex(want), hex(got))
                assert want != np.float32(-777.0).view(np.uint32)
    # a dense f-order matrix (no element-wise stride) and a strided view, large then small
    for shape, order in (([700, 900], "f"), ([33, 65], "f")):
        x = rs.randn(shape[0] * shape[1]).astype(np.float32)
        want, got = _both(dev, SUM, x, harness.shape_info(shape, order))
        assert want == got
    for n in (50000, 129):
        x = rs.randn(3 * n).astype(np.float32)
        want, got = _both(dev, MAX, x, harness.shape_info([1, n], strides=[3, 3], ews=3))
        assert want == got
    # agreement with float64 numpy on top of agreement with the other entry point (which shares the kernels)
    x = rs.uniform(-1, 1, 123457).astype(np.float32)
    x64 = x.astype(np.float64)
    truth = {SUM: x64.sum(), MAX: x64.max(), NORM2: np.sqrt((x64 * x64).sum()), LOGSUMEXP: np.log(np.exp(x64 - x64.max()).sum()) + x64.max()}
    for op, want in truth.items():
        _, got = _both(dev, op, x, harness.shape_info([1, x.size]))
        value = float(np.uint32(got).view(np.float32))
        bound = 1e-5 * (np.abs(x64).sum() if op == SUM else abs(want))
        assert value == want if op == MAX else abs(value - want) <= bound, (op, value, want)


def test_no_alloc_reduce_refuses_what_it_cannot_do():
    dev = harness.Device()
    x = np.arange(8, dtype=np.float32)
    info = harness.shape_info([1, 8])
    X = harness.Operand(dev, x, info)
    Z = harness.Operand(dev, np.full(1, np.float32(-777.0)), harness.shape_info([1, 1]))
    # more elements than the stated maximum (only the shapeInfo says so: nothing is launched)
    huge = harness.shape_info([1 << 20, 1 << 17])
    with pytest.raises(Nd4jError, match="2\\^36"):
        dev.ops.amd_execReduceFloatNoAlloc(dev.extra(huge), SUM, X.ptr, X.info_ptr, None, Z.ptr)
    # no host shapeInfo: a device one would have to be read back
    with pytest.raises(Nd4jError, match="host copy"):
        dev.ops.amd_execReduceFloatNoAlloc(dev.extra(None), SUM, X.ptr, X.info_ptr, None, Z.ptr)
    with pytest.raises(Nd4jError, match="opNum"):
        dev.ops.amd_execReduceFloatNoAlloc(dev.extra(info), 2, X.ptr, X.info_ptr, None, Z.ptr)
    assert Z.get()[0] == np.float32(-777.0)
    # and still works afterwards
    dev.ops.amd_execReduceFloatNoAlloc(dev.extra(info), SUM, X.ptr, X.info_ptr, None, Z.ptr)
    assert Z.get()[0] == np.float32(28.0)
    X.free()
    Z.free()
    dev.release()
