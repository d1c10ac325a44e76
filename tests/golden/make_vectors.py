"""Writes tests/golden/ref_vectors.json: input/output vectors produced by the reference's own loop code,
compiled as it is into oracle/_ref/libnd4j_ref.so (see oracle/Makefile).  Run in a container that has the
reference tree and the built library:

    make -C oracle ref && python tests/golden/make_vectors.py

Only data is written (inputs as seeds/values, outputs as IEEE bit patterns in hex).  The reference's own unit
tests hold no absolute vectors for the RandomBuffer stream and only a handful of per-op known answers, so these
vectors are what pins those parts when the compiled reference is not at hand.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import cpu_ref  # noqa: E402
from golden_inputs import (BROADCAST_OPS, INDEX_OPS, PAIRWISE_OPS, REDUCE_OPS, SCALAR_OPS, SCALAR_VALUES, TRANSFORM_OPS,  # noqa: E402
                           half_reduction_input, hexbits, op_extra, pairwise_inputs, reduce_input, shape_info_np, transform_input, whole_array_cases)


def main():
    ref = cpu_ref.load_reference()
    if ref is None:
        raise SystemExit("oracle/_ref/libnd4j_ref.so is missing: run `make -C oracle ref` first")
    ref.set_threads(1)
    out = {"_about": "vectors produced by the compiled reference (oracle/_ref); see make_vectors.py"}

    # ---- RandomBuffer stream -------------------------------------------------------------------
    rng = {}
    g = ref.rng_init(119, 1 << 20)
    n26 = 1 << 26
    probe = [0, 1, 2, 3, (1 << 20) - 1, 1 << 20, (1 << 20) + 1, 2 * (1 << 20) + 5, 12345678, n26 - 1]
    rng["seed119_size2p20"] = {
        "buffer_head": [int(v) for v in g.buffer[:8]], "buffer_tail": [int(v) for v in g.buffer[-2:]],
        "probe_index": probe,
        "fresh": [int(g.elements(i, 1)[0]) for i in probe]}
    g.rewind(n26)
    rng["seed119_size2p20"]["state_after_rewind_2p26"] = list(g.get_state())
    rng["seed119_size2p20"]["after_rewind_2p26"] = [int(g.elements(i, 1)[0]) for i in probe]
    g.rewind(n26)
    rng["seed119_size2p20"]["state_after_2nd_rewind"] = list(g.get_state())
    rng["seed119_size2p20"]["after_2nd_rewind"] = [int(g.elements(i, 1)[0]) for i in probe]
    g.destroy()

    # small buffer: dense stream over several wraps, offsets, reseeding, negative seed
    small = []
    for seed, size, ops in ((7, 100, [("none", 0)]), (7, 100, [("rewind", 37)]), (7, 100, [("rewind", 100)]),
                            (7, 100, [("rewind", 1234)]), (7, 100, [("reseed", 99)]), (7, 100, [("reseed", -5)]),
                            (-3, 64, [("rewind", 200), ("reseed", 12345678901)]), (0, 50, [("rewind", 49)]),
                            (2 ** 40 + 17, 33, [("rewind", 5000)])):
        g = ref.rng_init(seed, size)
        for kind, v in ops:
            if kind == "rewind":
                g.rewind(v)
            elif kind == "reseed":
                g.reseed(v)
        small.append({"seed": seed, "size": size, "ops": ops, "state": list(g.get_state()),
                      "elements_0_400": [int(v) for v in g.elements(0, 400)]})
        g.destroy()
    rng["small"] = small

    # float outputs of the random ops on a fresh seed-119 generator of 4096 words, in sequence
    g = ref.rng_init(119, 4096)
    seq = []
    n = 1000
    zi = shape_info_np([1, n])
    z = np.zeros(n, np.float32)
    g.random_z(0, z, zi, np.array([0, 1], np.float32))
    seq.append({"op": 0, "overload": "z", "args": [0, 1], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    g.random_z(0, z, zi, np.array([-2.5, 7], np.float32))
    seq.append({"op": 0, "overload": "z", "args": [-2.5, 7], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    g.random_xyz(6, z, zi, z, zi, z, zi, np.array([0, 1], np.float32))
    seq.append({"op": 6, "overload": "xyz_inplace", "args": [0, 1], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    x = (np.arange(n, dtype=np.float32) + 1)
    zz = x.copy()
    g.random_xz(1, zz, zi, zz, zi, np.array([0.5], np.float32))
    seq.append({"op": 1, "overload": "xz_inplace", "x": "arange+1", "args": [0.5], "n": n, "out": hexbits(zz),
                "state": list(g.get_state())})
    zz = x.copy()
    g.random_xz(2, zz, zi, zz, zi, np.array([0.25], np.float32))
    seq.append({"op": 2, "overload": "xz_inplace", "x": "arange+1", "args": [0.25], "n": n, "out": hexbits(zz),
                "state": list(g.get_state())})
    g.random_z(7, z, zi, np.array([0.3], np.float32))
    seq.append({"op": 7, "overload": "z", "args": [0.3], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    g.random_z(4, z, zi, np.array([1, 2], np.float32))
    seq.append({"op": 4, "overload": "z", "args": [1, 2], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    g.random_xyz(10, z, zi, z, zi, z, zi, np.array([0.5, 0.25], np.float32))
    seq.append({"op": 10, "overload": "xyz_inplace", "args": [0.5, 0.25], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    g.random_xyz(11, z, zi, z, zi, z, zi, np.array([1.0, 2.0], np.float32))
    seq.append({"op": 11, "overload": "xyz_inplace", "args": [1.0, 2.0], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    g.random_xyz(8, z, zi, z, zi, z, zi, np.array([5, 0.4], np.float32))
    seq.append({"op": 8, "overload": "xyz_inplace", "args": [5, 0.4], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    zodd = np.zeros(n - 1, np.float32)
    zio = shape_info_np([1, n - 1])
    g.random_xyz(6, zodd, zio, zodd, zio, zodd, zio, np.array([3, 0.5], np.float32))
    seq.append({"op": 6, "overload": "xyz_inplace", "args": [3, 0.5], "n": n - 1, "out": hexbits(zodd), "state": list(g.get_state())})
    g.random_xz(12, x.copy(), zi, z, zi, np.array([0.6, 1.5, -0.5, 2.0], np.float32))
    seq.append({"op": 12, "overload": "xz", "x": "arange+1", "args": [0.6, 1.5, -0.5, 2.0], "n": n, "out": hexbits(z),
                "state": list(g.get_state())})
    g.random_z(13, z, zi, np.array([1.5], np.float32))
    seq.append({"op": 13, "overload": "z", "args": [1.5], "n": n, "out": hexbits(z), "state": list(g.get_state())})
    yv = (np.arange(n, dtype=np.float32) * -1)
    g.random_xyz(3, x.copy(), zi, yv, zi, z, zi, np.array([0.35], np.float32))
    seq.append({"op": 3, "overload": "xyz", "x": "arange+1", "y": "-arange", "args": [0.35], "n": n, "out": hexbits(z),
                "state": list(g.get_state())})
    g.destroy()
    rng["float_sequence_seed119_size4096"] = seq
    out["rng"] = rng

    # ---- TAD tables ----------------------------------------------------------------------------------
    tads = []
    cases = [([16384, 4096], "c", [1]), ([16384, 4096], "c", [0]), ([32768, 2048], "f", [0]), ([32768, 2048], "f", [1]),
             ([2, 3, 4], "c", [0]), ([2, 3, 4], "c", [1]), ([2, 3, 4], "c", [2]), ([2, 3, 4], "f", [1]), ([2, 3, 4], "c", [0, 2]),
             ([2, 3, 4], "c", [1, 2]), ([2, 3, 4, 5], "c", [1, 3]), ([2, 3, 4, 5], "f", [0, 2]), ([2, 3, 4, 5], "c", [0, 1, 2]),
             ([1, 7], "c", [1]), ([7, 1], "c", [0]), ([7], "c", [0]), ([3, 1, 4], "c", [1]), ([3, 1, 4], "c", [0, 1]),
             ([1, 1, 5], "f", [2]), ([2, 2, 2, 2, 3], "c", [2, 4]), ([4, 5], "c", [0, 1]), ([5, 5], "f", [1])]
    for shape, order, dims in cases:
        info = ref.shape_buffer(shape, order)
        ti, off = ref.tad(info, dims)
        tads.append({"shape": shape, "order": order, "dims": dims, "x_info": [int(v) for v in info],
                     "tad_info": [int(v) for v in ti], "num_tads": int(len(off)),
                     "offsets_head": [int(v) for v in off[:8]], "offsets_tail": [int(v) for v in off[-3:]],
                     "offsets_sum": int(off.sum())})
    out["tad"] = tads

    # ---- per-op outputs ------------------------------------------------------------------------------
    ops = {}
    x = transform_input()
    xi = shape_info_np([1, x.size])
    tr = {}
    for op in TRANSFORM_OPS:
        z = np.zeros_like(x)
        ref.transform(op, x, xi, z, xi, op_extra("transform", op))
        tr[str(op)] = hexbits(z)
    ops["transform_f32"] = tr
    a, b = pairwise_inputs()
    ai = shape_info_np([1, a.size])
    pw = {}
    for op in PAIRWISE_OPS:
        z = np.zeros_like(a)
        ref.pairwise(op, a, ai, b, ai, z, ai, op_extra("pairwise", op))
        pw[str(op)] = hexbits(z)
    ops["pairwise_f32"] = pw
    # broadcast: x = the first pairwise vector as a 12 x 8 matrix, y = the first 8 values of the second one
    bxi = shape_info_np([12, 8])
    row = b[:8].copy()
    col = b[8:20].copy()
    bc = {}
    for op in BROADCAST_OPS:
        z = np.zeros(a.size, np.float32)
        ref.broadcast(op, a, bxi, row, shape_info_np([1, 8]), z, bxi, [1])
        z0 = np.zeros(a.size, np.float32)
        ref.broadcast(op, a, bxi, col, shape_info_np([12, 1]), z0, bxi, [0])
        bc[str(op)] = {"dim1": hexbits(z), "dim0": hexbits(z0)}
    ops["broadcast_f32_12x8"] = bc
    # scalar family: the first pairwise vector against a by-value scalar, and as a 12 x 8 matrix against one
    # scalar per TAD (rows: the first 12 values of the second vector; columns: its first 8)
    sc = {}
    for op in SCALAR_OPS:
        entry = {}
        for k, value in enumerate(SCALAR_VALUES):
            z = np.zeros_like(a)
            ref.scalar(op, a, ai, z, ai, value, None)
            entry["value%d" % k] = hexbits(z)
        z = np.zeros_like(a)
        ref.scalar_tad(op, a, bxi, z, bxi, b[:12].copy(), None, [1])
        entry["tad_dim1"] = hexbits(z)
        z = np.zeros_like(a)
        ref.scalar_tad(op, a, bxi, z, bxi, b[:8].copy(), None, [0])
        entry["tad_dim0"] = hexbits(z)
        sc[str(op)] = entry
    ops["scalar_f32"] = sc
    m = reduce_input()  # [12, 10]
    mi = shape_info_np([12, 10])
    rd = {}
    for op in REDUCE_OPS:
        e = op_extra("reduce", op)
        z1 = np.zeros(12, np.float32)
        ref.reduce(op, m, mi, e, z1, shape_info_np([1, 12]), [1])
        z0 = np.zeros(10, np.float32)
        ref.reduce(op, m, mi, e, z0, shape_info_np([1, 10]), [0])
        s = ref.reduce_scalar(op, m, mi, e)
        rd[str(op)] = {"dim1": hexbits(z1), "dim0": hexbits(z0), "scalar": hexbits(np.array([s], np.float32))}
    ops["reduce_f32_12x10"] = rd
    ir = {}
    for op in INDEX_OPS:
        e = op_extra("indexreduce", op)
        z1 = np.zeros(12, np.float32)
        ref.indexreduce(op, m, mi, e, z1, shape_info_np([1, 12]), [1])
        z0 = np.zeros(10, np.float32)
        ref.indexreduce(op, m, mi, e, z0, shape_info_np([1, 10]), [0])
        s = ref.indexreduce_scalar(op, m, mi, e)
        ir[str(op)] = {"dim1": hexbits(z1), "dim0": hexbits(z0), "scalar": hexbits(np.array([s], np.float32))}
    ops["indexreduce_f32_12x10"] = ir
    st = {}
    for op in (0, 1):
        for bias in (0, 1):
            z1 = np.zeros(12, np.float32)
            ref.summarystats(op, bias, m, mi, z1, shape_info_np([1, 12]), [1])
            z0 = np.zeros(10, np.float32)
            ref.summarystats(op, bias, m, mi, z0, shape_info_np([1, 10]), [0])
            s = ref.summarystats_scalar(op, bias, m, mi)
            st["%d_%d" % (op, bias)] = {"dim1": hexbits(z1), "dim0": hexbits(z0), "scalar": hexbits(np.array([s], np.float32))}
    ops["summarystats_f32_12x10"] = st

    # fp16: reached through functions::*<float16> (the NativeOps Half entry points are empty on the CPU back end)
    xh = (0.1 * (np.arange(8, dtype=np.float32) + 1)).astype(np.float16)
    yh = (1000 + np.arange(8, dtype=np.float32)).astype(np.float16)
    hi = shape_info_np([2, 4])
    h = {}
    for name, op in (("add", 0), ("multiply", 6)):
        z = np.zeros(8, np.float16)
        ref.pairwise(op, xh, hi, yh, hi, z, hi, None)
        h["pairwise_" + name] = hexbits(z)
    z = np.zeros(8, np.float16)
    ref.transform(15, xh, hi, z, hi, None)
    h["transform_tanh"] = hexbits(z)
    rowh = (0.333 * np.arange(4, dtype=np.float32)).astype(np.float16)
    ref.broadcast(0, xh, hi, rowh, shape_info_np([1, 4]), z, hi, [1])
    h["broadcast_add_row"] = hexbits(z)
    h["reduce_sum_y"] = hexbits(np.array([ref.reduce_scalar(1, yh, hi, None)], np.float16))
    ops["f16_2x4"] = h
    # fp16 reductions at a size where the reference's accumulation in fp16 (every update rounds to half,
    # cpu/reduce.cpp:150-156, types/float16.h:391-394) is still within a few 1e-3 of the exact value: rows of 16, columns
    # of 12, 192 elements in all, values in [0.5, 1.5)
    xr = half_reduction_input()
    ri = shape_info_np([12, 16])
    hr = {"x": hexbits(xr)}
    for op in (0, 1, 3, 4, 5, 6):
        z1, z0 = np.zeros(12, np.float16), np.zeros(16, np.float16)
        ref.reduce(op, xr, ri, None, z1, shape_info_np([1, 12]), [1])
        ref.reduce(op, xr, ri, None, z0, shape_info_np([1, 16]), [0])
        hr["reduce_%d" % op] = {"dim1": hexbits(z1), "dim0": hexbits(z0),
                                "scalar": hexbits(np.array([ref.reduce_scalar(op, xr, ri, None)], np.float16))}
    for op in (0, 1):
        z1, z0 = np.zeros(12, np.float16), np.zeros(16, np.float16)
        ref.indexreduce(op, xr, ri, None, z1, shape_info_np([1, 12]), [1])
        ref.indexreduce(op, xr, ri, None, z0, shape_info_np([1, 16]), [0])
        hr["indexreduce_%d" % op] = {"dim1": hexbits(z1), "dim0": hexbits(z0),
                                     "scalar": hexbits(np.array([ref.indexreduce_scalar(op, xr, ri, None)], np.float16))}
    for op in (0, 1):
        for bias in (0, 1):
            z1, z0 = np.zeros(12, np.float16), np.zeros(16, np.float16)
            ref.summarystats(op, bias, xr, ri, z1, shape_info_np([1, 12]), [1])
            ref.summarystats(op, bias, xr, ri, z0, shape_info_np([1, 16]), [0])
            hr["summarystats_%d_%d" % (op, bias)] = {"dim1": hexbits(z1), "dim0": hexbits(z0),
                                                     "scalar": hexbits(np.array([ref.summarystats_scalar(op, bias, xr, ri)], np.float16))}
    ops["f16_reductions_12x16"] = hr
    # whole-array transforms: Col2Im, Im2col, Histogram, Reverse, Pooling2D
    wa = {}
    for name, op, x, x_info, z_info, extra, z0 in whole_array_cases():
        z = z0.copy()
        ref.transform(op, x, x_info, z, z_info, extra)
        wa[name] = hexbits(z)
    ops["whole_array_f32"] = wa
    out["ops"] = ops

    with open(os.path.join(HERE, "ref_vectors.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote ref_vectors.json", os.path.getsize(os.path.join(HERE, "ref_vectors.json")), "bytes")


if __name__ == "__main__":
    main()
