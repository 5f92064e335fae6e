"""FALKON drivers on the engine (the kernel-ridge-regression benchmark configuration in miniature): the Nystrom coefficients must solve
(K_nm^T K_nm + lambda n (K_mm + eps M I)) alpha = K_nm^T y (eps M I is the preconditioner's jitter, which
the algorithm carries into the system it solves); a dense fp64 solve gives that in closed form."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _problem(n, seed=0):
    import torch
    g = torch.Generator().manual_seed(seed)
    X = 2 * torch.rand(n, 3, generator=g) - 1
    y = torch.sin(3 * X[:, 0]) * torch.cos(2 * X[:, 1]) + X[:, 2] ** 2 + 0.1 * torch.randn(n, generator=g)
    return X.cuda(), y[:, None].cuda()


def test_falkon_matches_closed_form_and_fits():
    import torch
    from f3m_amd.conjugate_gradient import FalkonOptions, custom_Falkon, custom_GaussianKernel
    print("case falkon n=40000 M=400", flush=True)
    n, M, lam, sigma = 40000, 400, 1e-6, 0.5
    X, Y = _problem(n)
    kernel = custom_GaussianKernel(sigma, var_compression=False, interpolation_nr=64)
    model = custom_Falkon(kernel, lam, M, maxiter=30, seed=3, options=FalkonOptions(cg_tolerance=1e-9))
    model.fit(X, Y)
    C = model.ny_points_
    # dense fp64 reference of the same Nystrom system
    Knm = kernel(X, C)
    Kmm = kernel(C, C)
    jitter = model.options.pc_epsilon(torch.float32) * M
    H = Knm.T @ Knm + lam * n * (Kmm + jitter * torch.eye(M, dtype=torch.float64, device="cuda"))
    alpha_ref = torch.linalg.solve(H, Knm.T @ Y.double())
    pred_ref = Knm @ alpha_ref
    pred = model.predict(X).double()
    rel = float((pred - pred_ref).norm() / pred_ref.norm())
    mse, mse_ref = float(((pred - Y.double()) ** 2).mean()), float(((pred_ref - Y.double()) ** 2).mean())
    print("prediction vs closed form rel-L2: %.3e, mse %.5f (closed form %.5f), CG iterations %d, CG time %.3fs"
          % (rel, mse, mse_ref, model.cg_iterations_, model.conjugate_gradient_time), flush=True)
    # the operator of the normal equations, K_nm^T (K_nm v + w), against the dense fp64 one: both engine products
    # (the second is the transposed product on the same plan) with their 1e-3 bound
    g = torch.Generator().manual_seed(5)
    v, w = torch.randn(M, 1, generator=g).cuda(), torch.randn(n, 1, generator=g).cuda()
    dm = kernel.dmmv(X, C, v, w).double()
    dm_ref = Knm.T @ (Knm @ v.double() + w.double())
    rel_dmmv = float((dm - dm_ref).norm() / dm_ref.norm())
    print("dmmv vs dense fp64: %.3e" % rel_dmmv, flush=True)
    assert rel_dmmv < 1e-3
    # With lambda = 1e-6 the Nystrom system is ill conditioned: the ~1e-4 relative error of the engine's
    # products moves the coefficients along weakly determined directions, so the pin of the operator is the
    # dmmv check above and the fit is held tightly below; the predictions themselves agree with the closed form
    # to the level the fp32 solves allow (1e-2 in tests/test_falkon_cpu.py, where the CG + preconditioner
    # arithmetic is pinned against the closed form with a dense kernel).
    assert rel < 1e-2                       # measured 1.1e-3
    assert mse < 1.05 * mse_ref + 1e-4
    ss_tot = float(((Y.double() - Y.double().mean()) ** 2).mean())
    assert 1 - mse / ss_tot > 0.9           # R^2 on the synthetic target (noise sd 0.1, signal var ~0.4)
    # a fresh test set goes through one engine product
    Xt, Yt = _problem(5000, seed=9)
    pt = model.predict(Xt).double()
    assert float(((pt - Yt.double()) ** 2).mean()) < 0.03


def test_blocked_preconditioner_matches_whole_matrix_form_on_the_gpu():
    """M = 12000 centres through the tile-by-tile preconditioner (fp32 storage, tiles of 4096, no library call on
    more than one tile: the form M = 1e5 needs) and through the whole-matrix fp64 form: same solves up to the
    fp32 rounding amplified by the factors' condition, same quality of the fit."""
    import torch
    from f3m_amd.conjugate_gradient import FalkonOptions, custom_Falkon, custom_GaussianKernel
    from f3m_amd.conjugate_gradient.preconditioner import FalkonPreconditioner
    print("case falkon blocked preconditioner n=300000 M=12000", flush=True)
    n, M, lam, sigma = 300000, 12000, 1e-6, 0.5
    X, Y = _problem(n, seed=2)
    fits = {}
    for blocked in (False, True):
        kernel = custom_GaussianKernel(sigma, var_compression=False, interpolation_nr=64)
        opt = FalkonOptions(pc_blocked=blocked, pc_block_size=4096)
        model = custom_Falkon(kernel, lam, M, maxiter=20, seed=3, options=opt)
        model.fit(X, Y)
        pred = model.predict(X).double()
        mse = float(((pred - Y.double()) ** 2).mean())
        fits[blocked] = (mse, pred, model.ny_points_)
        print("blocked=%s: mse %.5f, preconditioner %.2fs, CG %.2fs" % (blocked, mse, model.fit_times_[0], model.conjugate_gradient_time), flush=True)
    assert torch.equal(fits[False][2], fits[True][2])                   # same centres
    assert fits[True][0] < 1.02 * fits[False][0] + 1e-5
    rel = float((fits[True][1] - fits[False][1]).norm() / fits[False][1].norm())
    print("predictions blocked vs whole-matrix: %.3e" % rel, flush=True)
    assert rel < 2e-2
    # the factors themselves, on the same centres
    C = fits[True][2]
    kernel = custom_GaussianKernel(sigma)
    whole = FalkonPreconditioner(lam, kernel, FalkonOptions(pc_blocked=False, pc_explicit_inverse=False)).init(C)
    blk = FalkonPreconditioner(lam, kernel, FalkonOptions(pc_blocked=True, pc_block_size=4096)).init(C)
    assert blk.blocked and len(blk.T.tiles) == 3
    Tb = blk.T.dense_upper().double()
    assert float((Tb - whole.T).abs().max() / whole.T.abs().max()) < 1e-4
    g = torch.Generator().manual_seed(7)
    v = torch.randn(M, 1, generator=g, dtype=torch.float64).cuda()
    for fac, dense in ((blk.T, Tb), (blk.A, blk.A.dense_upper().double())):
        x = fac.solve(v)
        assert float((dense @ x - v).norm() / v.norm()) < 1e-3          # each solve inverts its own factor
        xt = fac.solve(v, transpose=True)
        assert float((dense.T @ xt - v).norm() / v.norm()) < 1e-3


def test_falkon_at_the_benchmark_size():
    """The kernel-ridge-regression configuration at its stated size: N = 1e7 points, M = 1e5 Nystrom centres, 20
    conjugate-gradient iterations (reference protocol: conjugate_gradient/custom_falkon.py:119-244, experiments/
    experiments_krr_a.py:49-97).  The tile-by-tile fp32 preconditioner holds two 40 GB factors: the test skips on a
    device with less than 100 GiB free.  Checks: quality of the fit (R^2 >= 0.96, mse within 5 % of the noise
    variance 0.01), and both engine products of the operator, K_nm v and K_nm^T u on the plan of the fit, against
    the fp64 exact products on 2000 seeded rows each (< 1e-3)."""
    import torch
    from f3m_amd import engine
    from f3m_amd.conjugate_gradient import FalkonOptions, custom_Falkon, custom_GaussianKernel
    print("case falkon n=1e7 M=1e5", flush=True)
    engine.release_cache()
    torch.cuda.empty_cache()
    free = torch.cuda.mem_get_info()[0] / 2 ** 30
    if free < 100:
        pytest.skip("%.0f GiB of device memory free, 100 needed" % free)
    n, M, lam, sigma = 10_000_000, 100_000, 1e-6, 0.5
    X, Y = _problem(n, seed=1)
    opt = FalkonOptions()
    kernel = custom_GaussianKernel(sigma, opt=opt, var_compression=False, interpolation_nr=64)
    model = custom_Falkon(kernel, lam, M, maxiter=20, seed=1, options=opt)
    model.fit(X, Y)
    pred = model.predict(X)
    mse = float(((pred - Y) ** 2).mean())
    r2 = 1 - mse / float(((Y - Y.mean()) ** 2).mean())
    print("fit: preconditioner %.1f s, CG %.2f s (%d iterations), mse %.5f, R^2 %.4f, peak device memory %.1f GiB"
          % (model.fit_times_[0], model.conjugate_gradient_time, model.cg_iterations_, mse, r2,
             torch.cuda.max_memory_allocated() / 2 ** 30), flush=True)
    assert model.cg_iterations_ == 20
    assert r2 >= 0.96
    assert mse <= 1.05 * 0.01
    # the two products of one iteration, on the plan of (X, centres) that the fit used
    C = model.ny_points_
    del model, pred
    torch.cuda.empty_cache()
    g = torch.Generator().manual_seed(11)
    v, u = torch.randn(M, 1, generator=g).cuda(), torch.randn(n, 1, generator=g).cuda()
    rows = torch.randint(0, n, (2000,), generator=g).cuda()
    cols = torch.randint(0, M, (2000,), generator=g).cuda()
    Kv = kernel.mmv(X, C, v)
    Ktu = kernel.dmmv(X, C, None, u)
    Xd, Cd = X.double(), C.double()
    exact_rows = engine.exact_f64(Xd[rows].contiguous(), Cd, v.double(), sigma)
    exact_cols = engine.exact_f64(Cd[cols].contiguous(), Xd, u.double(), sigma)
    e1 = float((Kv[rows].double() - exact_rows).norm() / exact_rows.norm())
    e2 = float((Ktu[cols].double() - exact_cols).norm() / exact_cols.norm())
    print("K_nm v on 2000 rows: %.3e, K_nm^T u on 2000 rows: %.3e (vs fp64 exact)" % (e1, e2), flush=True)
    assert e1 < 1e-3 and e2 < 1e-3
    del kernel, X, Y, Xd, Cd
    engine.release_cache()
    torch.cuda.empty_cache()
