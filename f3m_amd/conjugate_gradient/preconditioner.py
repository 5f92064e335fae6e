"""The FALKON preconditioner (Rudi, Carratino, Rosasco 2017, Alg. 1), in PyTorch on the GPU.

The reference calls ``falkon.preconditioner.FalkonPreconditioner`` (conjugate_gradient/custom_falkon.py:
195-199, used through invA/invT/invTt/invAt/apply/apply_t at custom_conjugate_gradient_falkon.py:149-159,
181-182 and custom_falkon.py:241).  With K_MM the kernel matrix of the M Nystrom centres:

    T = chol(K_MM + eps M I)          upper triangular,  T^T T = K_MM + eps M I
    A = chol(T T^T / M + lambda I)    upper triangular

``apply(v) = T^-1 A^-1 v`` maps the preconditioned solution beta to the Nystrom coefficients alpha and
``apply_t(v) = A^-T T^-T v`` is its transpose.

Two forms.  Small M (both matrices within MAX_MATRIX_BYTES): whole-matrix library calls in
``pc_dtype``.  Large M (the benchmark's M = 1e5: 1e10 entries per matrix): ``BlockedUpperFactor``, fp32
storage, every factorisation, product and solve done tile by tile so that no library call ever sees an
operand larger than one tile (block_size^2 entries); diagonal tiles are factorised and inverted in fp64."""
import torch


def _tiles(M, nb):
    return [(i, min(M, i + nb)) for i in range(0, M, nb)]


class BlockedUpperFactor:
    """Upper-triangular Cholesky factor U (U^T U = S) of a symmetric positive definite fp32 matrix, held in
    the upper triangle of the matrix it was computed from, together with the inverses of its diagonal tiles.

    Right-looking blocked factorisation: for tile row k, (1) the diagonal tile is factorised in fp64 and its
    inverse kept in fp32, (2) the tiles right of it become U_kk^-T S_kj (a product with that inverse), (3) every
    tile (i, j), k < i <= j, loses S_ki^T S_kj.  Triangular solves run tile row by tile row: products of tiles
    with pieces of the vector, and one product with the inverse of the diagonal tile.  HBM: the matrix itself
    (4 M^2 bytes) plus 4 M block_size bytes of diagonal inverses; per solve about 2 M^2 bytes are read."""

    def __init__(self, S, block_size):
        assert S.dim() == 2 and S.shape[0] == S.shape[1] and S.dtype == torch.float32
        self.U = S
        self.M = S.shape[0]
        self.nb = int(block_size)
        self.tiles = _tiles(self.M, self.nb)
        self.dinv = []

    def factorize_(self):
        S, T = self.U, self.tiles
        for k, (k0, k1) in enumerate(T):
            D = S[k0:k1, k0:k1].double()
            D = torch.triu(D) + torch.triu(D, 1).T                     # the lower part of S is never read as data
            U = torch.linalg.cholesky(D, upper=True)
            Ui = FalkonPreconditioner._inverse_upper(U)               # 1024 identity columns per library call
            S[k0:k1, k0:k1] = U.float()
            Ui = Ui.float()
            self.dinv.append(Ui)
            for (j0, j1) in T[k + 1:]:
                S[k0:k1, j0:j1] = Ui.T @ S[k0:k1, j0:j1]
            for a, (i0, i1) in enumerate(T[k + 1:], start=k + 1):
                Ski_t = S[k0:k1, i0:i1].T
                for (j0, j1) in T[a:]:
                    S[i0:i1, j0:j1].addmm_(Ski_t, S[k0:k1, j0:j1], alpha=-1.0)
            del D, U
        return self

    def gram_t(self, out, scale, shift):
        """out (M x M fp32, upper triangle) = scale * U U^T + shift * I, tile by tile."""
        S, T = self.U, self.tiles
        for a, (i0, i1) in enumerate(T):
            for b, (j0, j1) in enumerate(T[a:], start=a):
                acc = torch.zeros(i1 - i0, j1 - j0, dtype=torch.float32, device=S.device)
                for (k0, k1) in T[b:]:                                  # U_ik U_jk^T over the tiles right of both
                    Uik = S[i0:i1, k0:k1]
                    Ujk = S[j0:j1, k0:k1]
                    if k0 == i0:
                        Uik = torch.triu(Uik)                           # below the diagonal of a diagonal tile: not U
                    if k0 == j0:
                        Ujk = torch.triu(Ujk)
                    acc.addmm_(Uik, Ujk.T)
                acc.mul_(scale)
                if a == b:
                    acc.diagonal().add_(shift)
                out[i0:i1, j0:j1] = acc
        return out

    def solve(self, v, transpose=False):
        """U x = v (back substitution) or, transposed, U^T x = v (forward substitution); v is (M,) or (M, c)."""
        S, T = self.U, self.tiles
        x = v.to(torch.float32).clone()
        vec = x.dim() == 1
        if vec:
            x = x[:, None]
        if not transpose:
            for k in range(len(T) - 1, -1, -1):
                k0, k1 = T[k]
                r = x[k0:k1].clone()
                for (j0, j1) in T[k + 1:]:
                    r.addmm_(S[k0:k1, j0:j1], x[j0:j1], alpha=-1.0)
                x[k0:k1] = self.dinv[k] @ r
        else:
            for k, (k0, k1) in enumerate(T):
                r = x[k0:k1].clone()
                for (j0, j1) in T[:k]:
                    r.addmm_(S[j0:j1, k0:k1].T, x[j0:j1], alpha=-1.0)
                x[k0:k1] = self.dinv[k].T @ r
        x = x[:, 0] if vec else x
        return x.to(v.dtype)

    def dense_upper(self):
        """the factor as a dense upper-triangular matrix (tests, small M only)"""
        return torch.triu(self.U)


class FalkonPreconditioner:
    MAX_MATRIX_BYTES = 8 * 2 ** 30          # whole-matrix library calls stay below this
    MAX_BLOCKED_BYTES = 96 * 2 ** 30        # both fp32 matrices of the blocked form together

    def __init__(self, penalty, kernel, opt):
        self.penalty = float(penalty)
        self.kernel = kernel
        self.params = opt
        self.T = None
        self.A = None
        self.Tinv = None
        self.Ainv = None
        self.blocked = False

    def init(self, ny_points, weight_vec=None):
        if weight_vec is not None:
            raise NotImplementedError("weighted FALKON is not provided")
        dt = self.params.pc_dtype
        M = ny_points.shape[0]
        nbytes = M * M * torch.empty((), dtype=dt).element_size()
        want_blocked = getattr(self.params, "pc_blocked", None)
        if want_blocked or (want_blocked is None and nbytes > self.MAX_MATRIX_BYTES):
            return self._init_blocked(ny_points)
        if nbytes > self.MAX_MATRIX_BYTES:
            # Whole-matrix library calls on tens of GB (two 80 GB fp64 factors at M = 1e5) have failed inside
            # the BLAS library on the development machines: such sizes go through the blocked form only.
            raise NotImplementedError("preconditioner matrices of %.1f GiB exceed the limit of %.0f GiB for whole-matrix "
                                      "library calls (M = %d, %s); leave pc_blocked unset or True"
                                      % (nbytes / 2 ** 30, self.MAX_MATRIX_BYTES / 2 ** 30, M, dt))
        # every factorisation is done in place
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
        self.blocked = False
        if getattr(self.params, "pc_explicit_inverse", False) and 4 * nbytes <= self.MAX_MATRIX_BYTES * 2:
            # the loop applies each factor's inverse (or its transpose) once or twice per iteration: as
            # dense upper-triangular matrices these are matrix-vector products at memory speed
            self.Tinv = self._inverse_upper(self.T)
            self.Ainv = self._inverse_upper(self.A)
        return self

    def _init_blocked(self, ny_points):
        M = ny_points.shape[0]
        nb = int(getattr(self.params, "pc_block_size", 8192))
        if 2 * 4 * M * M > self.MAX_BLOCKED_BYTES:
            raise NotImplementedError("two fp32 %d x %d preconditioner matrices (%.0f GiB) exceed the limit of %.0f GiB"
                                      % (M, M, 8 * M * M / 2 ** 30, self.MAX_BLOCKED_BYTES / 2 ** 30))
        dev = self.kernel.device if hasattr(self.kernel, "device") else ny_points.device
        eps = self.params.pc_epsilon(ny_points.dtype)
        # K_MM + eps M I, fp32, upper tiles only (the kernel is evaluated in fp64 tile by tile)
        K = torch.empty(M, M, dtype=torch.float32, device=dev)
        tiles = _tiles(M, nb)
        for a, (i0, i1) in enumerate(tiles):
            for (j0, j1) in tiles[a:]:
                blk = self.kernel(ny_points[i0:i1], ny_points[j0:j1], dtype=torch.float64)
                if i0 == j0:
                    blk.diagonal().add_(eps * M)
                K[i0:i1, j0:j1] = blk
                del blk
        self.T = BlockedUpperFactor(K, nb).factorize_()
        A = torch.empty(M, M, dtype=torch.float32, device=dev)
        self.T.gram_t(A, 1.0 / M, self.penalty)
        self.A = BlockedUpperFactor(A, nb).factorize_()
        self.Tinv = self.Ainv = None
        self.blocked = True
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
        if isinstance(tri, BlockedUpperFactor):
            return tri.solve(v, transpose)
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
