"""Writes the fixtures in this folder from the reference's own host objects.

Run in the container that holds the reference tree, after `make -C oracle` has built
oracle/_ref/libsapphire_ref.so from the reference's NaiveGemm.cpp, NaiveBasic.cpp, shape.cpp
and Broadcast.hpp.  The fixtures are data only (shapes, seeds, offsets, output bits):

    gemm_plans.json      leaves of Compute::Gemm's broadcast walk for a list of shape triples
    naive_gemm_kat.npz   outputs of Dense::Naive::Gemm / the Compute::Gemm host branch /
                         Naive::ReLU / Naive::Transpose on seeded inputs (the inputs are
                         regenerated from the seeds by sapphire_amd.synth)
    backward_kat.npz     outputs of Naive::Scale / Sub / ReLUBackward and of the Compute::Sub
                         host branch on seeded inputs
    shape_ops.json       Shape::Expand / Shrink / Rows / Cols / Size / GetNumUnits results

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import pyoracle as po  # noqa: E402
from sapphire_amd import synth  # noqa: E402
from tests.golden.cases import (PLAN_CASES, KAT_GEMM_CASES, KAT_OP_CASES, SHAPE_CASES,  # noqa: E402
                                SUB_CASES, SUB_LEAF_CASES)


def main():
    if not po.have_ref():
        raise SystemExit("oracle/_ref/libsapphire_ref.so is not built; run `make -C oracle`")
    import ctypes
    r = po.ref()

    plans = []
    for ys, as_, bs in PLAN_CASES:
        dims, leaves = po.gemm_plan(ys, as_, bs, lib="ref")
        plans.append({"y": ys, "a": as_, "b": bs, "dims": dims,
                      "leaves": [list(map(int, l)) for l in leaves]})
    json.dump(plans, open(os.path.join(HERE, "gemm_plans.json"), "w"), indent=0)

    kat = {}
    for name, ys, as_, bs, seed in KAT_OP_CASES:
        A = synth.uniform(seed + 1, as_)
        B = synth.uniform(seed + 2, bs)
        C = synth.uniform(seed + 3, ys)
        kat["op_" + name] = po.compute_gemm(C.copy(), A, B, lib="ref")
    for name, batch, M, N, K, seed in KAT_GEMM_CASES:
        A = synth.uniform(seed + 1, (batch, M, K))
        B = synth.uniform(seed + 2, (batch, K, N))
        C = synth.uniform(seed + 3, (batch, M, N))
        out = C.copy()
        r.ref_naive_gemm(out.size, po._f(out), po._f(A), po._f(B), M, N, K)
        kat["leaf_" + name] = out
    x = synth.uniform(900, (1000,))
    y = np.empty_like(x)
    r.ref_relu(po._f(y), po._f(x), x.size)
    kat["relu"] = y
    t_in = synth.uniform(901, (3, 5, 7))
    t_out = np.zeros(3 * 5 * 7, np.float32)
    r.ref_transpose(po._f(t_out), po._f(t_in), 5, 7, 3, 0)
    kat["transpose"] = t_out
    np.savez_compressed(os.path.join(HERE, "naive_gemm_kat.npz"), **kat)

    back = {}
    x = synth.normal(950, (1003,))
    y = np.empty_like(x)
    r.ref_scale(po._f(y), po._f(x), 0.37, x.size)
    back["scale"] = y
    dx = synth.uniform(951, (1003,))
    dy = synth.uniform(952, (1003,))
    out = dx.copy()
    r.ref_relu_backward(po._f(out), po._f(dy), po._f(x), x.size)
    back["relu_backward"] = out
    for name, count, stride, bca, bcb, seed in SUB_LEAF_CASES:
        a = synth.uniform(seed + 1, (count,))
        b = synth.uniform(seed + 2, (count,))
        out = np.empty(count, np.float32)
        r.ref_sub(count, po._f(out), po._f(a), po._f(b), stride, int(bca), int(bcb))
        back["subleaf_" + name] = out
    for name, ys, as_, bs, seed in SUB_CASES:
        a = synth.uniform(seed + 1, as_)
        b = synth.uniform(seed + 2, bs)
        back["sub_" + name] = po.compute_sub(ys, a, b, lib="ref")
    np.savez_compressed(os.path.join(HERE, "backward_kat.npz"), **back)

    shapes = []
    for dims in SHAPE_CASES:
        entry = {"dims": dims, "rows": r.ref_shape_query(po._ints(dims), len(dims), 0, 0),
                 "cols": r.ref_shape_query(po._ints(dims), len(dims), 1, 0),
                 "size": r.ref_shape_query(po._ints(dims), len(dims), 2, 0),
                 "units": [r.ref_shape_query(po._ints(dims), len(dims), 3, k) for k in range(5)],
                 "expand": [], "shrink": []}
        for k in range(0, 7):
            out = (ctypes.c_int * 16)()
            n = r.ref_shape_op(po._ints(dims), len(dims), 0, k, out)
            entry["expand"].append([out[i] for i in range(n)])
        for k in range(1, 7):
            out = (ctypes.c_int * 16)()
            n = r.ref_shape_op(po._ints(dims), len(dims), 1, k, out)
            entry["shrink"].append([out[i] for i in range(n)])
        shapes.append(entry)
    json.dump(shapes, open(os.path.join(HERE, "shape_ops.json"), "w"), indent=0)
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
