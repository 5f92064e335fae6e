"""Operator classes with the call signatures of the reference's experiments/FFM_classes.py, on top
of f3m_amd.ffm_3d_float.  ``keops_matmul`` (a pykeops baseline) and ``par_FFM_block`` (one process
per GPU) are not provided: this engine targets one GPU and has no pykeops dependency."""
import torch

from . import ffm_3d_float as load_obj


def _check_shapes(X, Y, b):
    try:
        assert Y.shape[1] == X.shape[1]
        assert Y.shape[0] == b.shape[0]
    except AssertionError:
        print('shape mismatch: X and Y need the same number of columns, b one row per row of Y')
        raise AssertionError


class FFM:
    """Fast Gaussian kernel-matrix-vector product (reference: experiments/FFM_classes.py:8-126)."""

    def __init__(self, X, Y=None, ls=1.0, min_points=1000, nr_of_interpolation=64, eff_var_limit=0.15,
                 var_compression=False, small_field_points=1000, device="cuda:0"):
        self.X = X.float().to(device)
        if torch.is_tensor(Y):
            self.Y = Y.float().to(device)
        else:
            self.Y = self.X           # same storage selects the symmetric engine path
        self.d = self.X.shape[1]
        if not 1 <= self.d <= 10:
            raise AssertionError("dimensionality must be between 1 and 10")
        self.ls = float(ls)
        self.min_points = float(min_points)
        self.nr_of_interpolation = int(nr_of_interpolation)
        self.eff_var_limit = float(eff_var_limit)
        self.var_compression = var_compression
        self.device = device
        self.small_field_points = small_field_points

    def update_ls(self, ls):
        if not ls > 0:
            raise AssertionError("ls must be positive")
        self.ls = float(ls)

    def __matmul__(self, b):
        self.b = b.float().to(self.device)
        return self.forward(self.X, self.Y, self.b)

    def grad(self, b):
        self.b = b.float().to(self.device)
        return self.forward_grad(self.X, self.Y, self.b)

    def chunk_forward_transpose(self, b, chunks=10):
        """K(Y, X) b in source chunks (reference :54-61)."""
        self.b = b.float().to(self.device)
        res = 0.0
        for bb, y in zip(torch.chunk(self.b, dim=0, chunks=chunks), torch.chunk(self.X, dim=0, chunks=chunks)):
            res = res + self.forward(self.Y, y, bb)
        return res

    def chunk_forward_example(self, b, chunks=10):
        """K(X, Y) b in source chunks (reference :63-70)."""
        self.b = b.float().to(self.device)
        res = 0.0
        for bb, y in zip(torch.chunk(self.b, dim=0, chunks=chunks), torch.chunk(self.Y, dim=0, chunks=chunks)):
            res = res + self.forward(self.X, y, bb)
        return res

    def forward_grad(self, X, Y, b):
        _check_shapes(X, Y, b)
        return getattr(load_obj, "rbf_float_%d_grad" % self.d)(X, Y, b, self.ls, True)

    def forward(self, X, Y, b):
        assert X.device == Y.device == b.device == torch.device(self.device)
        self.device = str(self.device)
        _check_shapes(X, Y, b)
        return getattr(load_obj, "FFM_XY_FLOAT_%d" % self.d)(
            X, Y, b, self.device, self.ls, self.min_points, self.nr_of_interpolation, self.var_compression,
            self.eff_var_limit, self.small_field_points)


class benchmark_matmul:
    """Exact fp32 product (reference: experiments/FFM_classes.py:264-323)."""
    _dtype = torch.float32
    _prefix = "rbf_float_%d"

    def __init__(self, X, Y=None, ls=1.0, device="cuda:0"):
        self.X = X.to(self._dtype).to(device)
        self.Y = Y.to(self._dtype).to(device) if torch.is_tensor(Y) else self.X
        self.d = self.X.shape[1]
        if not 0 < self.d <= 10:
            raise AssertionError("dimensionality must be between 1 and 10")
        self.ls = float(ls)
        self.device = device

    def update_ls(self, ls):
        if not ls > 0:
            raise AssertionError("ls must be positive")
        self.ls = float(ls)

    def __matmul__(self, b):
        self.b = b.to(self._dtype).to(self.device)
        return self.forward(self.X, self.Y, self.b)

    def forward(self, X, Y, b):
        _check_shapes(X, Y, b)
        return getattr(load_obj, self._prefix % self.d)(X, Y, b, self.ls, True)


class benchmark_matmul_double(benchmark_matmul):
    """Exact fp64 product, the accuracy reference (reference: experiments/FFM_classes.py:325-383)."""
    _dtype = torch.float64
    _prefix = "rbf_double_%d"


class block_FFM_matmul(FFM):
    """Blocked product with host accumulation (reference: experiments/FFM_classes.py:385-435)."""

    def __init__(self, X, Y=None, ls=1.0, min_points=1000, nr_of_interpolation=64, eff_var_limit=0.15,
                 var_compression=False, small_field_points=1000, device="cuda:0", blocks_X=1, blocks_Y=1):
        super().__init__(X=X, Y=Y, ls=ls, min_points=min_points, nr_of_interpolation=nr_of_interpolation,
                         eff_var_limit=eff_var_limit, var_compression=var_compression,
                         small_field_points=small_field_points, device=device)
        self._xy_mode = torch.is_tensor(Y)
        self.blocks_X = blocks_X
        self.blocks_Y = blocks_Y

    def __matmul__(self, b):
        b = b.float().to(self.device)
        outs = []
        x_chunks = torch.chunk(self.X, self.blocks_X, dim=0)
        if self._xy_mode:
            y_chunks = torch.chunk(self.Y, self.blocks_Y, dim=0)
            b_chunks = torch.chunk(b, self.blocks_Y, dim=0)
        else:
            y_chunks = x_chunks
            b_chunks = torch.chunk(b, self.blocks_X, dim=0)
        for i, x in enumerate(x_chunks):
            acc = torch.zeros(x.shape[0], b.shape[1])
            for j, y in enumerate(y_chunks):
                same = (not self._xy_mode) and i == j
                acc += self.forward(x, x if same else y, b_chunks[j]).cpu()
            outs.append(acc)
        return torch.cat(outs, dim=0)
