"""Size-independent properties at the benchmark size (N = 1e7, d = 3): coverage of every point pair,
linearity, and rel-L2 against the fp64 exact product on a seeded row subsample."""
import numpy as np
import pytest

from parity_checks import rel_l2

pytestmark = pytest.mark.gpu


def test_n1e7_uniform_properties():
    import torch
    from f3m_amd import engine
    print("case N=1e7 uniform d=3", flush=True)
    g = torch.Generator().manual_seed(1)
    N = 10_000_000
    X = torch.rand(N, 3, generator=g).cuda()
    b = torch.randn(N, 2, generator=g).cuda()
    plan = engine.Plan(X, None, ls=1.0)
    w = plan.work()
    assert w["near_pairs"] + w["far_point_pairs"] == float(N) * N
    out = plan.apply(b)
    assert torch.isfinite(out).all()
    # linearity in b
    comb = plan.apply((b[:, :1] - 3.0 * b[:, 1:]).contiguous())
    assert rel_l2(comb.cpu().numpy(), (out[:, :1] - 3.0 * out[:, 1:]).cpu().numpy()) < 1e-5
    # rel-L2 on a seeded 1e4-row subsample against fp64 exact (1e11 pair evaluations)
    rows = torch.from_numpy(np.random.default_rng(1).choice(N, 10_000, replace=False)).cuda()
    exact = engine.exact_f64(X[rows].double(), X.double(), b[:, :1].double().contiguous(), 1.0)
    err = rel_l2(out[rows, :1].cpu().numpy(), exact.cpu().numpy())
    print("rel-L2 on subsample: %.3e" % err, flush=True)
    assert err <= 1e-3
