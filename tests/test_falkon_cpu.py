"""Pins the FALKON preconditioner and conjugate-gradient drivers (no engine involved: the K_nm matrix is
passed densely, the branch the reference takes when K_nm fits in memory,
conjugate_gradient/custom_falkon.py:229-232) against the closed form of the system they solve."""
import pytest

torch = pytest.importorskip("torch")


class DenseGaussian:
    def __init__(self, sigma):
        self.sigma = sigma

    def __call__(self, A, B, opt=None, dtype=torch.float64):
        return torch.exp(-torch.cdist(A.double(), B.double()) ** 2 / (2 * self.sigma ** 2)).to(dtype)


def test_preconditioned_cg_converges_to_closed_form():
    from f3m_amd.conjugate_gradient.custom_conjugate_gradient_falkon import FalkonConjugateGradient_custom
    from f3m_amd.conjugate_gradient.options import FalkonOptions
    from f3m_amd.conjugate_gradient.preconditioner import FalkonPreconditioner
    torch.manual_seed(0)
    n, M, lam, sigma, eps = 3000, 150, 1e-6, 0.5, 1e-5
    X = 2 * torch.rand(n, 3) - 1
    y = (torch.sin(3 * X[:, 0]) * torch.cos(2 * X[:, 1]) + X[:, 2] ** 2 + 0.1 * torch.randn(n))[:, None].double()
    k = DenseGaussian(sigma)
    C = X[torch.randperm(n)[:M]]
    opt = FalkonOptions(cg_tolerance=1e-13, pc_epsilon_32=eps)
    pc = FalkonPreconditioner(lam, k, opt).init(C)
    Knm = k(X, C)
    # triangular factors: T^T T = K_mm + eps M I,  A^T A = T T^T / M + lambda I
    Kmm_j = k(C, C) + eps * M * torch.eye(M, dtype=torch.float64)
    assert torch.allclose(pc.T.T @ pc.T, Kmm_j, atol=1e-10)
    assert torch.allclose(pc.A.T @ pc.A, pc.T @ pc.T.T / M + lam * torch.eye(M, dtype=torch.float64), atol=1e-10)
    v = torch.randn(M, 2, dtype=torch.float64)
    assert torch.allclose(pc.T @ pc.A @ pc.apply(v), v, atol=1e-6) or torch.allclose(pc.A @ (pc.T @ pc.apply(v)), v, atol=1e-6)
    assert torch.allclose(pc.apply_t(v), torch.linalg.solve(pc.A.T, torch.linalg.solve(pc.T.T, v)), atol=1e-8)
    # closed form of the system FALKON solves (the jitter of the preconditioner is part of it)
    H = Knm.T @ Knm + lam * n * Kmm_j
    pred_ref = Knm @ torch.linalg.solve(H, Knm.T @ y)
    errs = []
    for its in (10, 30, 100):
        cg = FalkonConjugateGradient_custom(k, pc, opt)
        beta = cg.solve(Knm, None, y, lam, None, its)
        pred = Knm @ pc.apply(beta)
        errs.append(float((pred - pred_ref).norm() / pred_ref.norm()))
    assert errs[0] > errs[1] > errs[2] and errs[1] < 5e-3 and errs[2] < 1e-7, errs


def test_blocked_preconditioner_matches_the_whole_matrix_form():
    """The tile-by-tile form (fp32 storage, diagonal tiles in fp64; what M = 1e5 centres go through) against the
    whole-matrix fp64 form on the same centres: factor identities, both factors, every solve."""
    from f3m_amd.conjugate_gradient.options import FalkonOptions
    from f3m_amd.conjugate_gradient.preconditioner import BlockedUpperFactor, FalkonPreconditioner
    torch.manual_seed(1)
    M, lam, sigma, eps = 1100, 1e-6, 0.5, 1e-5          # 1100 = 4 tiles of 300 with a ragged last one
    C = 2 * torch.rand(M, 3) - 1
    k = DenseGaussian(sigma)
    k.device = "cpu"
    whole = FalkonPreconditioner(lam, k, FalkonOptions(pc_epsilon_32=eps, pc_blocked=False, pc_explicit_inverse=False)).init(C)
    blocked = FalkonPreconditioner(lam, k, FalkonOptions(pc_epsilon_32=eps, pc_blocked=True, pc_block_size=300)).init(C)
    assert blocked.blocked and isinstance(blocked.T, BlockedUpperFactor) and len(blocked.T.tiles) == 4
    Tb, Ab = blocked.T.dense_upper().double(), blocked.A.dense_upper().double()
    Kj = k(C, C) + eps * M * torch.eye(M, dtype=torch.float64)
    # fp32 storage: identities to fp32 accuracy of entries of size <= M eps + 1
    assert (Tb.T @ Tb - Kj).abs().max() < 2e-5
    assert (Ab.T @ Ab - (Tb @ Tb.T / M + lam * torch.eye(M, dtype=torch.float64))).abs().max() < 2e-6
    assert (Tb - whole.T).abs().max() < 1e-4 * whole.T.abs().max()
    v = torch.randn(M, 2, dtype=torch.float64)
    for name in ("invT", "invTt", "invA", "invAt", "apply", "apply_t"):
        got, want = getattr(blocked, name)(v), getattr(whole, name)(v)
        rel = float((got - want).norm() / want.norm())
        # the solves amplify the fp32 rounding of the factors by their condition (K_MM + eps M I: up to ~1e4 here)
        assert rel < 2e-2, (name, rel)
    # exactness of the solves against the blocked factors themselves (what the CG relies on)
    for fac, dense in ((blocked.T, Tb), (blocked.A, Ab)):
        x = fac.solve(v)
        assert float((dense @ x - v).norm() / v.norm()) < 1e-4
        xt = fac.solve(v[:, 0], transpose=True)
        assert xt.shape == (M,) and float((dense.T @ xt - v[:, 0]).norm() / v[:, 0].norm()) < 1e-4


def test_blocked_preconditioner_in_the_cg_loop():
    """FALKON with the tile-by-tile preconditioner against the closed form of the system.  Its triangular solves run
    in fp32 (as the reference's preconditioner does on fp32 data), and that rounding, amplified by the condition of
    the factors (~1e5 at lambda = 1e-6), is what limits the agreement; the fp64 whole-matrix form reaches 1e-7."""
    from f3m_amd.conjugate_gradient.custom_conjugate_gradient_falkon import FalkonConjugateGradient_custom
    from f3m_amd.conjugate_gradient.options import FalkonOptions
    from f3m_amd.conjugate_gradient.preconditioner import FalkonPreconditioner
    torch.manual_seed(0)
    n, M, lam, sigma, eps = 3000, 150, 1e-6, 0.5, 1e-5
    X = 2 * torch.rand(n, 3) - 1
    y = (torch.sin(3 * X[:, 0]) * torch.cos(2 * X[:, 1]) + X[:, 2] ** 2 + 0.1 * torch.randn(n))[:, None].double()
    k = DenseGaussian(sigma)
    k.device = "cpu"
    C = X[torch.randperm(n)[:M]]
    opt = FalkonOptions(cg_tolerance=1e-13, pc_epsilon_32=eps, pc_blocked=True, pc_block_size=64)
    pc = FalkonPreconditioner(lam, k, opt).init(C)
    Knm = k(X, C)
    H = Knm.T @ Knm + lam * n * (k(C, C) + eps * M * torch.eye(M, dtype=torch.float64))
    pred_ref = Knm @ torch.linalg.solve(H, Knm.T @ y)
    cg = FalkonConjugateGradient_custom(k, pc, opt)
    beta = cg.solve(Knm, None, y, lam, None, 100)
    pred = Knm @ pc.apply(beta)
    assert float((pred - pred_ref).norm() / pred_ref.norm()) < 2e-2
    mse, mse_ref = float(((pred - y) ** 2).mean()), float(((pred_ref - y) ** 2).mean())
    assert mse < 1.02 * mse_ref


def test_options_defaults_are_documented_values():
    from f3m_amd.conjugate_gradient import ConjugateGradientOptions, FalkonOptions
    o = FalkonOptions()
    assert (o.cg_epsilon(torch.float32), o.cg_tolerance, o.cg_full_gradient_every) == (1e-7, 1e-7, 10)
    assert isinstance(o.get_conjgrad_options(), ConjugateGradientOptions)


def test_conjugate_gradient_solves_spd_system():
    from f3m_amd.conjugate_gradient import ConjugateGradient, ConjugateGradientOptions
    g = torch.Generator().manual_seed(0)
    A = torch.randn(60, 60, generator=g, dtype=torch.float64)
    A = A @ A.T + 60 * torch.eye(60, dtype=torch.float64)
    B = torch.randn(60, 3, generator=g, dtype=torch.float64)
    cg = ConjugateGradient(ConjugateGradientOptions(cg_tolerance=1e-9))
    X = cg.solve(None, B, lambda v: A @ v, max_iter=200)
    assert torch.allclose(A @ X, B, atol=1e-7)
    assert cg.iterations_ <= 70             # exact in about dim steps; stops at the tolerance


def test_explicit_inverse_factors_equal_back_substitution():
    """pc_explicit_inverse keeps T^-1 and A^-1 as matrices; every solve must agree with back-substitution."""
    from f3m_amd.conjugate_gradient.options import FalkonOptions
    from f3m_amd.conjugate_gradient.preconditioner import FalkonPreconditioner
    torch.manual_seed(1)
    C = 2 * torch.rand(120, 3) - 1
    k = DenseGaussian(0.5)
    fast = FalkonPreconditioner(1e-6, k, FalkonOptions(pc_explicit_inverse=True)).init(C)
    slow = FalkonPreconditioner(1e-6, k, FalkonOptions(pc_explicit_inverse=False)).init(C)
    assert fast.Tinv is not None and slow.Tinv is None
    v = torch.randn(120, 3, dtype=torch.float64)
    for name in ("invA", "invAt", "invT", "invTt", "apply", "apply_t"):
        a, b = getattr(fast, name)(v), getattr(slow, name)(v)
        assert torch.allclose(a, b, rtol=1e-8, atol=1e-8 * float(b.abs().max())), name
