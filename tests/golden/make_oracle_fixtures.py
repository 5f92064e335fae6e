"""Writes tests/golden/oracle_fixtures.npz: small seeded clouds with everything the CPU oracle computes
for them.  These are ORACLE fixtures (outputs of oracle/f3m_oracle.c in this repository), not outputs of
the reference: the reference holds no golden vectors and cannot run without CUDA.  They freeze the
oracle's behaviour, so that a later change to the oracle or to the engine shows up as a difference
against committed data, and they give the GPU tests inputs with known answers that need no oracle run.

    python tests/golden/make_oracle_fixtures.py

Per case `name`: X, Y (empty if symmetric), b, params (ls, min_points, nr_of_interpolation,
small_field_points, var_compression, eff_var_limit), depth, and per level k: edge, offsets and centres
(uint32 bit patterns) of both trees, the per-point box id, the far / small / keep lists; the node grid;
the product of the oracle's algorithm and the fp64 exact product."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import f3m_oracle as fo  # noqa: E402
from helpers import box_of_point  # noqa: E402

f32 = np.float32
PARAM_KEYS = ("ls", "min_points", "nr_of_interpolation", "small_field_points", "var_compression", "eff_var_limit")


def cases():
    rng = np.random.default_rng(20240607)
    base = dict(ls=0.6, min_points=40, nr_of_interpolation=27, small_field_points=30, var_compression=False,
                eff_var_limit=0.15)
    yield "d1_uniform", rng.random((400, 1), dtype=f32), None, dict(base, nr_of_interpolation=6, ls=0.05)
    yield "d2_normal", rng.standard_normal((500, 2)).astype(f32), None, dict(base, nr_of_interpolation=16)
    yield "d3_uniform", rng.random((512, 3), dtype=f32), None, dict(base)
    yield "d3_two_trees", rng.standard_normal((450, 3)).astype(f32), (rng.random((300, 3)) * 4 - 2).astype(f32), \
        dict(base, nr_of_interpolation=64, min_points=30, small_field_points=10)
    yield "d4_uniform", rng.random((512, 4), dtype=f32), None, dict(base, nr_of_interpolation=16, min_points=30)
    yield "d5_uniform", rng.random((512, 5), dtype=f32), None, dict(base, nr_of_interpolation=32, min_points=20,
                                                                    small_field_points=8)
    g = (np.stack(np.meshgrid(*[np.arange(5)] * 3, indexing="ij"), -1).reshape(-1, 3) / 4.0).astype(f32)
    yield "d3_lattice_duplicates", np.concatenate([g, g[::-1], g[::2]]), None, dict(base, min_points=20,
                                                                                   small_field_points=10)
    yield "d3_var_compression", rng.random((512, 3), dtype=f32), None, dict(base, ls=3.0, var_compression=True,
                                                                            eff_var_limit=0.3, min_points=30,
                                                                            small_field_points=12)
    # Larger clouds whose box pairs hold at least 2 * nr_of_interpolation points, so that pairs two or more
    # boxes apart are FAR (interpolated) instead of falling under the first "small" rule:
    # the default 4 x 4 x 4 grid in 3-D, far pairs at depth 2;
    yield "d3_uniform_64nodes_far", rng.random((8000, 3), dtype=f32), None, dict(base, ls=0.8, nr_of_interpolation=64,
                                                                               min_points=200, small_field_points=80)
    # the 3^5 grid in 5-D: the 32 boxes of depth 1, far across the diagonals of the hypercube;
    yield "d5_uniform_243nodes_far", rng.random((8192, 5), dtype=f32), None, dict(base, ls=1.0, nr_of_interpolation=243,
                                                                                min_points=1000, small_field_points=200)
    # and a thin slab (two long dimensions), 16 boxes at depth 2 with far pairs up to three cells apart.
    yield "d5_slab_243nodes_far", (rng.random((4800, 5)) * np.array([1, 1, .1, .1, .1])).astype(f32), None, \
        dict(base, ls=0.7, nr_of_interpolation=243, min_points=500, small_field_points=200)


def main():
    out = {"names": np.array([c[0] for c in cases()])}
    for name, X, Y, prm in cases():
        M = X.shape[0] if Y is None else Y.shape[0]
        b = np.random.default_rng(len(name)).standard_normal((M, 2)).astype(f32)
        plan = fo.Plan(X, Y, **prm)
        out[name + "/X"] = X
        out[name + "/Y"] = np.zeros((0, X.shape[1]), f32) if Y is None else Y
        out[name + "/b"] = b
        out[name + "/params"] = np.array([float(prm[k]) for k in PARAM_KEYS], np.float64)
        out[name + "/depth"] = np.array(plan.nlevels, np.int64)
        for k in range(plan.nlevels):
            L = plan.level(k)
            pre = "%s/level%d/" % (name, k + 1)
            out[pre + "edge"] = np.array(L["edge"], f32)
            for w in ("x", "y"):
                out[pre + "off" + w] = L["off" + w].astype(np.int32)
                out[pre + "centres_bits_" + w] = L["c" + w].astype(f32).view(np.uint32)
                out[pre + "box_of_point_" + w] = box_of_point(L, w).astype(np.int32)
            for lst in ("far", "small", "keep"):
                out[pre + lst] = L[lst].astype(np.int32).reshape(-1, 2)
        counts = fo.node_counts(X.shape[1], prm["nr_of_interpolation"])
        out[name + "/node_counts"] = np.asarray(counts, np.int32)
        out[name + "/product_oracle"] = plan.apply(b).astype(f32)
        out[name + "/product_exact_f64"] = fo.exact_f64(X, X if Y is None else Y, b, prm["ls"])
    path = os.path.join(HERE, "oracle_fixtures.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, "%.1f KiB" % (os.path.getsize(path) / 1024), "cases:", ", ".join(out["names"].tolist()))


if __name__ == "__main__":
    main()
