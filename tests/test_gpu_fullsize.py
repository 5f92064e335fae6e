"""Parity at the benchmark size N = 1e7, for every benchmark configuration, against the CPU oracle run on the same
seeded cloud in the same test (the oracle builds the headline's tree and lists in ~6 s and sums selected rows in a
few seconds more):

  * tree and lists BIT FOR BIT: depth, edge, offsets, centres (bit patterns), the box of every point and the far, small
    and keep list of every level (tests/parity_checks.assert_plan_matches_oracle), and the coverage invariant
    (near pairs + pairs covered by far box pairs = N M);
  * the product on the rows of a handful of boxes of the deepest level (the box nearest the middle of the cloud, one
    on a face, two corners, random ones until ~1000 rows) within 1e-5 of the oracle's, and its rel-L2 error against the
    fp64 exact product on those rows within 1.5x the ORACLE's error there (and within the 1e-3 target wherever the
    oracle algorithm reaches it);
  * the same bound on the 256 seeded rows of the committed fixture tests/golden/fullsize_oracle_errors.json (oracle
    errors computed in the build container), whose work counts the engine's plan must reproduce exactly.

The headline configuration is also checked for linearity in b."""
import json
import os

import numpy as np
import pytest

from parity_checks import assert_plan_matches_oracle, rel_l2

pytestmark = pytest.mark.gpu
N = 10_000_000
FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fullsize_oracle_errors.json")


def _names():
    from f3m_amd import workloads
    return list(workloads.CONFIGS) + ["uniform3_125nodes", "uniform3_216nodes", "sweep3_varcomp_125nodes"]


def _fixture_rows():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fullsize_oracle_errors",
                                                  os.path.join(os.path.dirname(FIXTURE), "make_fullsize_oracle_errors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.sample_rows()


def probe_boxes(level, rng, want_rows=1000, max_boxes=24):
    """boxes of the deepest level whose rows are compared: nearest the middle of the cloud, nearest the middle of the
    lowest face of dimension 0, the two extreme corners, then random ones until want_rows rows are covered"""
    ctr = level["cx"].astype(np.float64)
    cnt = np.diff(level["offx"])
    lo, hi = ctr.min(0), ctr.max(0)
    u = (ctr - lo) / np.where(hi > lo, hi - lo, 1.0)
    face = np.full(ctr.shape[1], 0.5)
    face[0] = 0.0
    picks = [int(np.argmin(np.abs(u - 0.5).sum(1))), int(np.argmin(np.abs(u - face).sum(1))),
             int(np.argmin(u.sum(1))), int(np.argmax(u.sum(1)))]
    for bx in rng.permutation(ctr.shape[0]):
        if cnt[picks].sum() >= want_rows or len(picks) >= max_boxes:
            break
        if int(bx) not in picks:
            picks.append(int(bx))
    return sorted(set(picks))


@pytest.mark.parametrize("name", _names())
def test_n1e7_against_the_oracle(name, oracle):
    import torch
    from f3m_amd import engine, workloads
    print("case N=1e7 vs oracle:", name, flush=True)
    X, Y, b, prm = workloads.make(name, N, seed=1, columns=2 if name == "uniform3_ls1" else 1, device="cpu")
    Xn, Yn, bn = X.numpy(), None if Y is None else Y.numpy(), b.numpy()
    M = bn.shape[0]
    ora = oracle.Plan(Xn, Yn, **prm)
    Xd, Yd, bd = X.cuda(), None if Y is None else Y.cuda(), b.cuda()
    plan = engine.Plan(Xd, Yd, **prm)
    assert plan.depth >= 3
    assert_plan_matches_oracle(plan, ora)                                   # tree and lists, bit for bit
    w = plan.work()
    assert w["near_pairs"] + w["far_point_pairs"] == float(N) * M           # every pair exactly once
    assert w["near_pairs"] == ora.work_near_pairs and w["far_pairs"] == ora.work_far_pairs
    fix = json.load(open(FIXTURE))[name]
    assert (fix["tree_depth"], fix["near_pairs"], fix["far_box_pairs"]) == (plan.depth, w["near_pairs"], w["far_pairs"])
    out = plan.apply(bd)
    assert torch.isfinite(out).all()
    if name == "uniform3_ls1":                                              # linearity in b
        comb = plan.apply((bd[:, :1] - 3.0 * bd[:, 1:]).contiguous())
        assert rel_l2(comb.cpu().numpy(), (out[:, :1] - 3.0 * out[:, 1:]).cpu().numpy()) < 1e-5
    plan.close()
    Ys = Xd if Yd is None else Yd

    # rows of selected boxes: engine against the oracle, and both against the fp64 exact product
    deepest = ora.level(ora.nlevels - 1)
    boxes = probe_boxes(deepest, np.random.default_rng(5))
    rows = np.concatenate([deepest["permx"][deepest["offx"][bx]:deepest["offx"][bx + 1]] for bx in boxes]).astype(np.int64)
    want = ora.apply(bn[:, :1], rows=rows)[rows]
    rd = torch.from_numpy(rows).cuda()
    got = out[rd, :1].cpu().numpy()
    exact = engine.exact_f64(Xd[rd].double(), Ys.double(), bd[:, :1].double().contiguous(), prm["ls"]).cpu().numpy()
    e_eng, e_ora, diff = rel_l2(got, exact), rel_l2(want, exact), rel_l2(got, want)
    print("%d rows of %d boxes: engine vs oracle %.2e; vs fp64 exact: engine %.3e, oracle %.3e" % (len(rows), len(boxes), diff,
          e_eng, e_ora), flush=True)
    # 1e-5 against the oracle; where the algorithm's own error is large the two differ by rounding in sums of that size
    assert diff < 1e-5 + 0.02 * e_ora
    assert e_eng <= 1.5 * e_ora + 1e-7
    if e_ora <= 1e-3 / 1.5:
        assert e_eng <= 1e-3

    # the seeded rows of the committed fixture
    frows = torch.from_numpy(_fixture_rows()).cuda()
    exact = engine.exact_f64(Xd[frows].double(), Ys.double(), bd[:, :1].double().contiguous(), prm["ls"])
    e_fix = rel_l2(out[frows, :1].cpu().numpy(), exact.cpu().numpy())
    print("fixture rows: engine %.3e, oracle (committed) %.3e; 1e-3 target %s" % (e_fix, fix["oracle_rel_l2_vs_fp64_exact"],
          "met" if e_fix <= 1e-3 else "NOT met: the algorithm's own error at this node count and lengthscale"), flush=True)
    assert e_fix <= 1.5 * fix["oracle_rel_l2_vs_fp64_exact"] + 1e-7


def test_n1e7_variance_compression():
    """The reference's FALKON experiments run the operator with var_compression=True (experiments/
    experiments_krr_a.py): the extra far-field shortcuts at full size, lengthscales 3 and 1 on the unit cube.  The
    product stays within 1e-4 of the fp64 exact product on seeded rows (measured 1.8e-6 and 3.6e-5)."""
    import torch
    from f3m_amd import engine
    print("case N=1e7 var_compression", flush=True)
    g = torch.Generator(device="cuda").manual_seed(7)
    X = torch.rand(N, 3, generator=g, device="cuda")
    b = torch.randn(N, 1, generator=g, device="cuda")
    rows = torch.randint(0, N, (5000,), generator=torch.Generator().manual_seed(1)).cuda()
    for ls, limit in ((3.0, 0.3), (1.0, 0.15)):
        out = engine.kmvm(X, None, b, ls=ls, var_compression=True, eff_var_limit=limit)
        assert torch.isfinite(out).all()
        exact = engine.exact_f64(X[rows].contiguous(), X, b, ls)
        err = rel_l2(out[rows].cpu().numpy(), exact.cpu().numpy())
        print("ls=%g: rel-L2 on 5000 rows %.3e" % (ls, err), flush=True)
        assert err < 1e-4
