"""PyTorch-ROCm front end of the C ABI: tensors in, tensors out, raw device pointers in between.
torch is used for device memory and the current stream only."""
import ctypes as C

import numpy as np
import torch

from . import _lib, capi


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("f3m_amd operators need tensors on a HIP device (got %s)" % t.device)


def _prep(t, dtype):
    if t.dtype != dtype or not t.is_contiguous():
        t = t.to(dtype).contiguous()
    return t


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _same_storage(X, Y):
    return Y is None or (Y.data_ptr() == X.data_ptr() and Y.shape == X.shape)


def kmvm(X, Y, b, ls=1.0, min_points=1000, nr_of_interpolation=64, var_compression=False, eff_var_limit=0.15,
         small_field_points=1000):
    """out = K(X,Y) b through the F3M algorithm (reference: FFM_XY, F3M_src/n_tree.cu:1056-1125)."""
    lib = _lib.get()
    _need_cuda(X, b)
    sym = _same_storage(X, Y)
    X = _prep(X, torch.float32)
    Yc = X if sym else _prep(Y, torch.float32)
    b = _prep(b, torch.float32)
    if not sym:
        _need_cuda(Y)
    if X.dim() != 2 or b.dim() != 2 or Yc.shape[1] != X.shape[1] or b.shape[0] != Yc.shape[0]:
        raise AssertionError("shapes of X, Y and b do not match")
    out = torch.empty((X.shape[0], b.shape[1]), dtype=torch.float32, device=X.device)
    prm = capi.make_params(ls, min_points, nr_of_interpolation, var_compression, eff_var_limit, small_field_points)
    with torch.cuda.device(X.device):
        rc = lib.f3m_kmvm_f32(X.shape[1], _ptr(X), X.shape[0], None if sym else _ptr(Yc), Yc.shape[0], _ptr(b),
                              b.shape[1], C.byref(prm), _ptr(out), _stream())
    capi.check(lib, rc)
    return out


def _exact(fn_name, dtype, X, Y, b, ls):
    lib = _lib.get()
    _need_cuda(X, Y, b)
    X, Y, b = _prep(X, dtype), _prep(Y, dtype), _prep(b, dtype)
    if X.dim() != 2 or b.dim() != 2 or Y.shape[1] != X.shape[1] or b.shape[0] != Y.shape[0]:
        raise AssertionError("shapes of X, Y and b do not match")
    out = torch.empty((X.shape[0], b.shape[1]), dtype=dtype, device=X.device)
    with torch.cuda.device(X.device):
        rc = getattr(lib, fn_name)(X.shape[1], _ptr(X), X.shape[0], _ptr(Y), Y.shape[0], _ptr(b), b.shape[1],
                                   float(ls), _ptr(out), _stream())
    capi.check(lib, rc)
    return out


def exact_f32(X, Y, b, ls):
    """Exact dense product (reference: rbf_call<float>, F3M_src/n_tree.cu:185-211)."""
    return _exact("f3m_exact_f32", torch.float32, X, Y, b, ls)


def exact_grad_f32(X, Y, b, ls):
    """sum_j exp(-r^2/(2 ls^2)) r^2 b_j / ls^3 (reference: rbf_call_grad, F3M_src/n_tree.cu:213-241)."""
    return _exact("f3m_exact_grad_f32", torch.float32, X, Y, b, ls)


def exact_f64(X, Y, b, ls):
    """Exact dense product in fp64 (reference: rbf_call<double>)."""
    return _exact("f3m_exact_f64", torch.float64, X, Y, b, ls)


class Plan:
    """Box division and interaction lists of one (X, Y, parameters) problem, reusable for many b.
    Everything FFM_XY (F3M_src/n_tree.cu:1056-1125) computes before it touches b."""

    def __init__(self, X, Y=None, ls=1.0, min_points=1000, nr_of_interpolation=64, var_compression=False,
                 eff_var_limit=0.15, small_field_points=1000):
        self._lib = _lib.get()
        self._h = None
        _need_cuda(X)
        sym = _same_storage(X, Y)
        X = _prep(X, torch.float32)
        Yc = X if sym else _prep(Y, torch.float32)
        if not sym:
            _need_cuda(Y)
        if X.dim() != 2 or Yc.shape[1] != X.shape[1]:
            raise AssertionError("shapes of X and Y do not match")
        self.device = X.device
        self.d, self.N, self.M = X.shape[1], X.shape[0], Yc.shape[0]
        prm = capi.make_params(ls, min_points, nr_of_interpolation, var_compression, eff_var_limit,
                               small_field_points)
        h = C.c_void_p()
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_create(self.d, _ptr(X), self.N, None if sym else _ptr(Yc), self.M, C.byref(prm),
                                           _stream(), C.byref(h))
        capi.check(self._lib, rc)
        self._h = h
        self.depth = self._lib.f3m_plan_depth(h)
        self.symmetric = bool(self._lib.f3m_plan_symmetric(h))

    def close(self):
        if self._h is not None:
            self._lib.f3m_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def apply(self, b):
        _need_cuda(b)
        b = _prep(b, torch.float32)
        if b.dim() != 2 or b.shape[0] != self.M:
            raise AssertionError("b must be (M, c)")
        out = torch.empty((self.N, b.shape[1]), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_apply(self._h, _ptr(b), b.shape[1], _ptr(out), _stream())
        capi.check(self._lib, rc)
        return out

    __matmul__ = apply

    def apply_transpose(self, u):
        """K(X,Y)^T u with this plan's trees and lists (u has N rows, the result M): what a second plan of
        (Y, X) would give (reference: FFM.chunk_forward_transpose, experiments/FFM_classes.py:54-61)."""
        _need_cuda(u)
        u = _prep(u, torch.float32)
        if u.dim() != 2 or u.shape[0] != self.N:
            raise AssertionError("u must be (N, c)")
        out = torch.empty((self.M, u.shape[1]), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_apply_transpose(self._h, _ptr(u), u.shape[1], _ptr(out), _stream())
        capi.check(self._lib, rc)
        return out

    def apply_noalloc(self, b, out):
        """The same product written into `out` (N, c) without any device allocation by the library: its
        temporaries come from static device memory (128 MiB per GPU).  The plan must have been applied once
        with the same number of columns before; b and out must already be contiguous fp32 device tensors."""
        _need_cuda(b, out)
        if b.dtype != torch.float32 or out.dtype != torch.float32 or not b.is_contiguous() or not out.is_contiguous():
            raise AssertionError("b and out must be contiguous fp32 tensors")
        if b.dim() != 2 or b.shape[0] != self.M or out.shape != (self.N, b.shape[1]):
            raise AssertionError("b must be (M, c) and out (N, c)")
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_apply_noalloc(self._h, _ptr(b), b.shape[1], _ptr(out), _stream())
        capi.check(self._lib, rc)
        return out

    def level_sizes(self, level):
        s = (C.c_int64 * 8)()
        e = C.c_float()
        capi.check(self._lib, self._lib.f3m_plan_level_sizes(self._h, level, s, C.byref(e)))
        keys = ("nbx", "nby", "nfar", "nsmall", "nkeep", "num_nodes", "maxcount_x", "maxcount_y")
        out = {k: int(v) for k, v in zip(keys, s)}
        out["edge"] = np.float32(e.value)
        return out

    def list_rows(self, level):
        """[boxes with pairs, their points, their pieces of 128 and of 160 points] of the small list,
        then the same of the keep list: what the near field sizes its launches with."""
        r = (C.c_int64 * 8)()
        capi.check(self._lib, self._lib.f3m_plan_list_rows(self._h, level, r))
        return [int(v) for v in r]

    def level(self, level):
        """Host copies (numpy) of the tree level and its three lists; levels are 1..depth."""
        sz = self.level_sizes(level)
        shapes = {
            "cx": ((sz["nbx"], self.d), np.float32), "cy": ((sz["nby"], self.d), np.float32),
            "offx": ((sz["nbx"] + 1,), np.int32), "offy": ((sz["nby"] + 1,), np.int32),
            "far": ((sz["nfar"], 2), np.int32), "small": ((sz["nsmall"], 2), np.int32),
            "keep": ((sz["nkeep"], 2), np.int32), "permx": ((self.N,), np.int32), "permy": ((self.M,), np.int32),
        }
        out = dict(sz)
        with torch.cuda.device(self.device):
            for name, (shape, dt) in shapes.items():
                a = np.zeros(shape, dt)
                if a.size:
                    capi.check(self._lib, self._lib.f3m_plan_level_copy(self._h, level, capi.LEVEL_ARRAYS[name],
                                                                        a.ctypes.data_as(C.c_void_p), _stream()))
                out[name] = a
        return out

    def far_level(self, level, b, want_expansions=False):
        b = _prep(b, torch.float32)
        sz = self.level_sizes(level)
        out = torch.zeros((self.N, b.shape[1]), dtype=torch.float32, device=self.device)
        mom = loc = None
        if want_expansions:
            per = node_counts(self.d, sz["num_nodes"])
            P = int(np.prod(per))
            mom = torch.zeros((b.shape[1], sz["nby"], P), dtype=torch.float32, device=self.device)
            loc = torch.zeros((b.shape[1], sz["nbx"], P), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_far_level(self._h, level, _ptr(b), b.shape[1], _ptr(out),
                                              None if mom is None else _ptr(mom), None if loc is None else _ptr(loc),
                                              _stream())
        capi.check(self._lib, rc)
        return (out, mom, loc) if want_expansions else out

    def near_level(self, level, which, b):
        b = _prep(b, torch.float32)
        out = torch.zeros((self.N, b.shape[1]), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_near_level(self._h, level, capi.LEVEL_ARRAYS[which], _ptr(b), b.shape[1], _ptr(out),
                                               _stream())
        capi.check(self._lib, rc)
        return out

    def lookup_boxes(self, level, cells, tree="x"):
        """Box id at depth `level` of every integer cell in `cells` (n, d) int32 on the GPU; -1 where the
        cell holds no point (reference: the key -> index hash table, F3M_src/linearprobing.cu:54-87)."""
        assert cells.is_cuda and cells.dtype == torch.int32 and cells.dim() == 2 and cells.shape[1] == self.d
        cells = cells.contiguous()
        ids = torch.empty(cells.shape[0], dtype=torch.int32, device=self.device)
        with torch.cuda.device(self.device):
            rc = self._lib.f3m_plan_lookup_boxes(self._h, level, 0 if tree == "x" else 1, _ptr(cells), cells.shape[0],
                                                 _ptr(ids), _stream())
        capi.check(self._lib, rc)
        return ids

    def work(self):
        """Work model: point pairs summed exactly, far box pairs, interpolated points, far pairs * P^2."""
        w = (C.c_double * 5)()
        with torch.cuda.device(self.device):
            capi.check(self._lib, self._lib.f3m_plan_work(self._h, w))
        return {"near_pairs": w[0], "far_pairs": w[1], "interp_points": w[2], "m2l_evals": w[3],
                "far_point_pairs": w[4]}


def node_counts(d, max_nodes):
    """Nodes per dimension of the tensor grid (reference: get_node_list, F3M_src/n_tree.cu:328-346,
    without its random permutation of the dimensions)."""
    ref = np.float32(float(max_nodes) ** (1.0 / float(np.float32(d))))
    hi, lo, acc = int(np.ceil(ref)), int(np.floor(ref)), 1
    out = []
    for i in range(d):
        fut = int(acc * float(lo) ** (d - (i + 1)) * hi)
        pick = hi if fut <= max_nodes else lo
        pick = max(pick, 1)
        out.append(pick)
        acc *= pick
    return out


def set_timing(enabled):
    _lib.get().f3m_set_timing(int(bool(enabled)))


def get_timing():
    t = (C.c_double * 6)()
    n = (C.c_int * 6)()
    _lib.get().f3m_get_timing(t, n)
    return {k: (t[i], n[i]) for i, k in enumerate(capi.STAGES)}


def release_cache():
    _lib.get().f3m_release_cache()
