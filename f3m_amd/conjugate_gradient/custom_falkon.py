"""FALKON kernel ridge regression estimator (reference: conjugate_gradient/custom_falkon.py:30-263)."""
import time

import torch

from .custom_conjugate_gradient_falkon import FalkonConjugateGradient_custom
from .options import FalkonOptions
from .preconditioner import FalkonPreconditioner


class custom_Falkon:
    """Nystrom kernel ridge regression solved by preconditioned conjugate gradient.

    Same constructor arguments as the reference (:102-118): ``kernel`` (a custom_GaussianKernel),
    ``penalty`` (lambda), ``M`` (number of uniformly chosen centres), ``maxiter``, ``seed``, ``error_fn`` /
    ``error_every`` (progress callback), ``options``.  ``fit`` (:119-244) picks the centres, builds the
    preconditioner, runs the CG iterations with every K_nm / K_nm^T product through the F3M engine
    and stores ``alpha_`` and ``ny_points_``; ``predict`` (:246-259) is one engine product."""

    def __init__(self, kernel, penalty, M, center_selection="uniform", maxiter=20, seed=None, error_fn=None,
                 error_every=1, weight_fn=None, options=None):
        if center_selection != "uniform":
            raise NotImplementedError("only uniform centre selection is provided")
        if weight_fn is not None:
            raise NotImplementedError("weighted FALKON is not provided")
        self.kernel = kernel
        self.penalty = float(penalty)
        self.M = int(M)
        self.maxiter = int(maxiter)
        self.seed = seed
        self.error_fn = error_fn
        self.error_every = error_every
        self.options = options or FalkonOptions()
        self.alpha_ = None
        self.ny_points_ = None
        self.fit_times_ = []
        self.conjugate_gradient_time = None

    def _select_centers(self, X):
        g = torch.Generator()
        if self.seed is not None:
            g.manual_seed(int(self.seed))
        idx = torch.randperm(X.shape[0], generator=g)[: self.M]
        return X[idx.to(X.device)].contiguous()

    def fit(self, X, Y, Xts=None, Yts=None):
        if X.shape[0] != Y.shape[0]:
            raise ValueError("X and Y must have the same number of rows")
        if Y.dim() == 1:
            Y = Y[:, None]
        if self.M > X.shape[0]:
            raise ValueError("M must not exceed the number of training points")
        self.fit_times_ = []
        t_s = time.time()
        ny_points = self._select_centers(X)
        precond = FalkonPreconditioner(self.penalty, self.kernel, self.options)
        precond.init(ny_points)
        self.fit_times_.append(time.time() - t_s)
        callback = None
        if self.error_fn is not None and self.error_every is not None:
            def callback(it, beta, train_time):
                self.fit_times_.append(self.fit_times_[0] + train_time)
                if it % self.error_every == 0:
                    alpha = precond.apply(beta)
                    Xe, Ye = (Xts, Yts) if (Xts is not None and Yts is not None) else (X, Y)
                    pred = self._predict(Xe, ny_points, alpha)
                    print("Iteration %3d - Elapsed %.2fs - error: %s" % (it, self.fit_times_[-1], self.error_fn(Ye, pred)),
                          flush=True)
        optim = FalkonConjugateGradient_custom(self.kernel, precond, self.options)
        torch.cuda.synchronize()
        start = time.time()
        beta = optim.solve(X, ny_points, Y, self.penalty, initial_solution=None, max_iter=self.maxiter,
                           callback=callback)
        torch.cuda.synchronize()
        self.conjugate_gradient_time = time.time() - start
        self.cg_iterations_ = optim.optimizer.iterations_
        self.mmv_times_ = list(optim.optimizer.mmv_times_)
        self.alpha_ = precond.apply(beta)
        self.ny_points_ = ny_points
        return self

    def _predict(self, X, ny_points, alpha):
        if ny_points is None:
            return X @ alpha
        return self.kernel.mmv(X, ny_points, alpha, opt=self.options)

    def predict(self, X):
        if self.alpha_ is None:
            raise RuntimeError("fit must be called before predict")
        return self._predict(X, self.ny_points_, self.alpha_)

    def to(self, device):
        self.alpha_ = self.alpha_.to(device)
        self.ny_points_ = self.ny_points_.to(device)
        return self
