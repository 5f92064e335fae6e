"""Conjugate-gradient drivers (reference: conjugate_gradient/custom_conjugate_gradient_falkon.py)."""
import functools
import time

import torch

from .options import ConjugateGradientOptions


class Optimizer(object):
    def __init__(self):
        pass


class ConjugateGradient(Optimizer):
    """Plain CG on several right-hand sides at once (reference :40-100): per-column step sizes, the
    epsilon in both denominators, a full residual every ``cg_full_gradient_every`` iterations, stop when
    the largest residual norm falls below ``cg_tolerance``."""

    def __init__(self, opt=None):
        super().__init__()
        self.params = opt or ConjugateGradientOptions()
        self.iterations_ = 0
        self.mmv_times_ = []

    def solve(self, X0, B, mmv, max_iter, callback=None):
        t_start = time.time()
        if X0 is None:
            R = B.clone()
            X = torch.zeros_like(B)
        else:
            R = B - mmv(X0)
            X = X0
        m_eps = self.params.cg_epsilon(X.dtype)
        P = R
        Rsold = torch.sum(R.pow(2), dim=0)
        e_train = time.time() - t_start
        for i in range(max_iter):
            t_start = time.time()
            AP = mmv(P)
            self.mmv_times_.append(time.time() - t_start)
            alpha = Rsold / (torch.sum(P * AP, dim=0) + m_eps)
            X = X + P * alpha
            if (i + 1) % self.params.cg_full_gradient_every == 0:
                R = B - mmv(X)
            else:
                R = R - AP * alpha
            Rsnew = torch.sum(R.pow(2), dim=0)
            self.iterations_ = i + 1
            if Rsnew.abs().max().sqrt() < self.params.cg_tolerance:
                break
            P = R + P * (Rsnew / (Rsold + m_eps))
            Rsold = Rsnew
            e_train += time.time() - t_start
            if callback is not None:
                callback(i + 1, X, e_train)
        return X


class FalkonConjugateGradient_custom(Optimizer):
    r"""Preconditioned CG for FALKON (reference :103-189).  Solves

        B^T H B beta = B^T K_nm^T Y / n,    H = K_nm^T K_nm / n + lambda K_mm,    B = T^-1 A^-1,

    with the preconditioner's triangular factors T and A; alpha = B beta."""

    def __init__(self, kernel, preconditioner, opt, weight_fn=None):
        super().__init__()
        self.kernel = kernel
        self.preconditioner = preconditioner
        self.params = opt
        self.optimizer = ConjugateGradient(opt.get_conjgrad_options())
        self.weight_fn = weight_fn

    def falkon_mmv(self, sol, penalty, X, M, Knm):
        n = Knm.shape[0] if Knm is not None else X.shape[0]
        prec = self.preconditioner
        v = prec.invA(sol)
        v_t = prec.invT(v)
        if Knm is not None:
            cc = Knm.T @ (Knm @ v_t)
        else:
            cc = self.kernel.dmmv(X, M, v_t, None, opt=self.params)
        # A^-T (T^-T (cc / n) + penalty v)
        cc_ = prec.invTt(cc / n) + penalty * v
        return prec.invAt(cc_)

    def solve(self, X, M, Y, _lambda, initial_solution, max_iter, callback=None):
        n = X.size(0)
        Knm = X if M is None else None
        y_over_n = Y / n
        if Knm is not None:
            B = Knm.T @ y_over_n
        else:
            B = self.kernel.dmmv(X, M, None, y_over_n, opt=self.params)
        B = self.preconditioner.apply_t(B)
        mmv = functools.partial(self.falkon_mmv, penalty=_lambda, X=X, M=M, Knm=Knm)
        return self.optimizer.solve(initial_solution, B, mmv, max_iter, callback)

    @property
    def is_weighted(self):
        return self.weight_fn is not None
