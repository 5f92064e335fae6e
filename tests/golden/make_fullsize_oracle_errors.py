"""Writes tests/golden/fullsize_oracle_errors.json: what the CPU oracle (oracle/f3m_oracle.c, the restatement of
the reference algorithm) gives for every benchmark configuration AT FULL SIZE, N = 1e7, on a seeded sample of target
rows: its rel-L2 error against the fp64 exact product (the oracle's own exact_f64) on those rows, the depth of its
tree, and its work counts (point pairs summed exactly, far box pairs, points interpolated).  These are ORACLE outputs
of this repository, not of the reference (which holds no golden vectors and cannot run without CUDA).

    python tests/golden/make_fullsize_oracle_errors.py [name[:nodes] ...]      # ~10 minutes on 8 cores for all

`bench.py` quotes the error as `algorithm_error_at_this_config` (it may not run the oracle itself), and
tests/test_gpu_fullsize.py holds the engine to 1.5x of it on the same rows.  Entries are keyed "name" for the
configurations of f3m_amd.workloads.ALL_CONFIGS and "name:nodes" for the node-count variants of the configurations
that miss 1e-3 at 64 nodes."""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from f3m_amd import workloads  # noqa: E402
from oracle import f3m_oracle as fo  # noqa: E402

OUT = os.path.join(HERE, "fullsize_oracle_errors.json")
N = 10_000_000
ROWS = 256
ROW_SEED = 20


def sample_rows(n=N, rows=ROWS):
    """the seeded target rows of the fixture (the tests and the benchmark draw the same ones)"""
    return np.sort(np.random.default_rng(ROW_SEED).choice(n, rows, replace=False))


def specs():
    for name in workloads.ALL_CONFIGS:
        yield name
    for name in workloads.NODE_VARIANTS_OF:
        for nodes in workloads.NODE_SWEEP[1:]:
            yield "%s:%d" % (name, nodes)


def run(spec):
    name, _, nodes = spec.partition(":")
    X, Y, b, prm = workloads.make(name, N, seed=1, device="cpu", nodes=int(nodes) if nodes else None)
    Xn, Yn, bn = X.numpy(), None if Y is None else Y.numpy(), b.numpy()
    t0 = time.time()
    plan = fo.Plan(Xn, Yn, **prm)
    rows = sample_rows()
    got = plan.apply(bn, rows=rows)[rows]
    exact = fo.exact_f64(Xn[rows], Xn if Yn is None else Yn, bn, prm["ls"])
    rec = {"N": N, "M": int(bn.shape[0]), "params": {k: (float(v) if isinstance(v, float) else v) for k, v in prm.items()},
           "rows": ROWS, "row_seed": ROW_SEED, "oracle_rel_l2_vs_fp64_exact": fo.rel_l2(got, exact),
           "tree_depth": int(plan.nlevels), "near_pairs": float(plan.work_near_pairs),
           "far_box_pairs": float(plan.work_far_pairs), "interp_points": float(plan.work_interp_pts),
           "oracle_seconds": round(time.time() - t0, 1)}
    return rec


def main():
    want = sys.argv[1:] or list(specs())
    try:
        data = json.load(open(OUT))
    except (OSError, ValueError):
        data = {}
    for spec in want:
        data[spec] = run(spec)
        print(spec, data[spec], flush=True)
        with open(OUT, "w") as f:
            json.dump(data, f, indent=1, sort_keys=True)
            f.write("\n")


if __name__ == "__main__":
    main()
