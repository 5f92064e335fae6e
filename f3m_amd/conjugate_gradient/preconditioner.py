"""The FALKON preconditioner (Rudi, Carratino, Rosasco 2017, Alg. 1), in PyTorch on the GPU.

The reference calls ``falkon.preconditioner.FalkonPreconditioner`` (conjugate_gradient/custom_falkon.py:
195-199, used through invA/invT/invTt/invAt/apply/apply_t at custom_conjugate_gradient_falkon.py:149-159,
181-182 and custom_falkon.py:241).  With K_MM the kernel matrix of the M Nystrom centres:

    T = chol(K_MM + eps M I)          upper triangular,  T^T T = K_MM + eps M I
    A = chol(T T^T / M + lambda I)    upper triangular

``apply(v) = T^-1 A^-1 v`` maps the preconditioned solution beta to the Nystrom coefficients alpha and
``apply_t(v) = A^-T T^-T v`` is its transpose."""
import torch


class FalkonPreconditioner:
    MAX_MATRIX_BYTES = 8 * 2 ** 30

    def __init__(self, penalty, kernel, opt):
        self.penalty = float(penalty)
        self.kernel = kernel
        self.params = opt
        self.T = None
        self.A = None
        self.Tinv = None
        self.Ainv = None

    def init(self, ny_points, weight_vec=None):
        if weight_vec is not None:
            raise NotImplementedError("weighted FALKON is not provided")
        dt = self.params.pc_dtype
        M = ny_points.shape[0]
        nbytes = M * M * torch.empty((), dtype=dt).element_size()
        if nbytes > self.MAX_MATRIX_BYTES:
            # A run with two 80 GB fp64 factors (M = 1e5) aborted inside the BLAS library on the
            # development machines and could not be diagnosed; sizes beyond what has been validated
            # are refused rather than attempted.
            raise NotImplementedError("preconditioner matrices of %.1f GiB exceed the validated limit of %.0f GiB "
                                      "(M = %d, %s); use fewer centres or pc_dtype=torch.float32"
                                      % (nbytes / 2 ** 30, self.MAX_MATRIX_BYTES / 2 ** 30, M, dt))
        # every factorisation is done in place: at M = 1e5 one fp64 M x M matrix is 80 GB
        K = self.kernel(ny_points, ny_points, dtype=dt)
        eps = self.params.pc_epsilon(ny_points.dtype)
        K.diagonal().add_(eps * M)
        T = torch.linalg.cholesky(K, upper=True, out=K)
        A = torch.empty_like(T)
        torch.mm(T, T.T, out=A)
        A.div_(M)
        A.diagonal().add_(self.penalty)
        self.A = torch.linalg.cholesky(A, upper=True, out=A)
        self.T = T
        self.Tinv = self.Ainv = None
        if getattr(self.params, "pc_explicit_inverse", False) and 4 * nbytes <= self.MAX_MATRIX_BYTES * 2:
            # the loop applies each factor's inverse (or its transpose) once or twice per iteration: as
            # dense upper-triangular matrices these are matrix-vector products at memory speed
            self.Tinv = self._inverse_upper(self.T)
            self.Ainv = self._inverse_upper(self.A)
        return self

    @staticmethod
    def _inverse_upper(U, block=1024):
        """U^-1 by solves against blocks of identity columns (the library's triangular solve needs a
        workspace that grows with the number of right-hand sides)."""
        M = U.shape[0]
        inv = torch.zeros_like(U)
        for j0 in range(0, M, block):
            j1 = min(M, j0 + block)
            rhs = torch.zeros(j1, j1 - j0, dtype=U.dtype, device=U.device)      # rows past j1 of these columns are 0
            rhs[j0:j1] = torch.eye(j1 - j0, dtype=U.dtype, device=U.device)
            inv[:j1, j0:j1] = torch.linalg.solve_triangular(U[:j1, :j1], rhs, upper=True)
        return inv

    def _solve(self, tri, inv, v, transpose):
        w = v.to(tri.dtype)
        if inv is not None:
            out = (inv.T if transpose else inv) @ w
        else:
            out = torch.linalg.solve_triangular(tri.T if transpose else tri, w, upper=not transpose)
        return out.to(v.dtype)

    def invA(self, v):
        return self._solve(self.A, self.Ainv, v, False)

    def invAt(self, v):
        return self._solve(self.A, self.Ainv, v, True)

    def invT(self, v):
        return self._solve(self.T, self.Tinv, v, False)

    def invTt(self, v):
        return self._solve(self.T, self.Tinv, v, True)

    def apply(self, v):
        return self.invT(self.invA(v))

    def apply_t(self, v):
        return self.invAt(self.invTt(v))
