"""Size-independent properties at the benchmark size N = 1e7 for every benchmark configuration: every
point pair is handled exactly once (near pairs + pairs covered by far box pairs = N M), the result is
finite, and its rel-L2 error against the fp64 exact product on a seeded 1e4-row subsample stays within
1.5x the error of the F3M algorithm itself at that configuration (f3m_amd.workloads.ALGORITHM_ERROR_N1E7)
and, where the algorithm reaches it, within the 1e-3 target.  The headline configuration is also checked
for linearity in b."""
import numpy as np
import pytest

from parity_checks import rel_l2

pytestmark = pytest.mark.gpu
N = 10_000_000


def _names():
    from f3m_amd import workloads
    return list(workloads.CONFIGS)


@pytest.mark.parametrize("name", _names())
def test_n1e7_properties(name):
    import torch
    from f3m_amd import engine, workloads
    print("case N=1e7", name, flush=True)
    X, Y, b, prm = workloads.make(name, N, seed=1, columns=2 if name == "uniform3_ls1" else 1)
    M = N if Y is None else Y.shape[0]
    plan = engine.Plan(X, Y, **prm)
    assert plan.depth >= 3
    w = plan.work()
    assert w["near_pairs"] + w["far_point_pairs"] == float(N) * M            # every pair exactly once
    out = plan.apply(b)
    assert torch.isfinite(out).all()
    if name == "uniform3_ls1":                                              # linearity in b
        comb = plan.apply((b[:, :1] - 3.0 * b[:, 1:]).contiguous())
        assert rel_l2(comb.cpu().numpy(), (out[:, :1] - 3.0 * out[:, 1:]).cpu().numpy()) < 1e-5
    plan.close()
    rows = torch.from_numpy(np.random.default_rng(1).choice(N, 10_000, replace=False)).cuda()
    Ys = X if Y is None else Y
    exact = engine.exact_f64(X[rows].double(), Ys.double(), b[:, :1].double().contiguous(), prm["ls"])
    err = rel_l2(out[rows, :1].cpu().numpy(), exact.cpu().numpy())
    bound = 1.5 * workloads.ALGORITHM_ERROR_N1E7[name]
    meets = workloads.ALGORITHM_ERROR_N1E7[name] <= 1e-3 / 1.5
    print("rel-L2 on 1e4 rows: %.3e (bound %.2e; 1e-3 target %s)" % (err, bound, "met" if err <= 1e-3 else "NOT met: the "
          "algorithm's own error at this node count and lengthscale"), flush=True)
    assert err <= bound
    if meets:
        assert err <= 1e-3


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
