"""CPU ORACLE -- TEST INFRASTRUCTURE ONLY.

ctypes front end of ``oracle/f3m_oracle.c`` (the IEEE-fp32 restatement of the F3M algorithm) plus
the exact tiled PyTorch CPU kernel-matrix-vector product that ``bench.py`` times as its
``cpu_baseline``.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product package ``f3m_amd`` never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libf3m_oracle.so")
_lib = None

WHICH = {"cx": 0, "cy": 1, "cntx": 2, "cnty": 3, "offx": 4, "offy": 5, "permx": 6, "permy": 7,
         "far": 8, "small": 9, "keep": 10}


def build(force=False):
    """Compile the C oracle with the Makefile beside it (gcc, no fast-math, no FMA contraction)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "f3m_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        fp, ip, lp, dp = (C.POINTER(C.c_float), C.POINTER(C.c_int), C.POINTER(C.c_long), C.POINTER(C.c_double))
        L.fo_nodes_1d.argtypes = [C.c_int, fp, fp]
        L.fo_node_counts.argtypes = [C.c_int, C.c_int, ip]
        L.fo_node_grid.argtypes = [C.c_int, ip, fp, ip, fp]
        L.fo_node_grid.restype = C.c_int
        L.fo_basis.argtypes = [C.c_int, C.c_int, fp, fp, C.c_float, fp]
        L.fo_root.argtypes = [C.c_int, fp, C.c_long, fp, C.c_long, fp, fp, fp]
        L.fo_plan_create.argtypes = [C.c_int, fp, C.c_long, fp, C.c_long, C.c_float, C.c_float, C.c_int,
                                     C.c_int, C.c_float, C.c_int, C.c_int]
        L.fo_plan_create.restype = C.c_void_p
        L.fo_plan_destroy.argtypes = [C.c_void_p]
        L.fo_plan_status.argtypes = [C.c_void_p]
        L.fo_plan_message.argtypes = [C.c_void_p]
        L.fo_plan_message.restype = C.c_char_p
        L.fo_plan_nlevels.argtypes = [C.c_void_p]
        L.fo_plan_symmetric.argtypes = [C.c_void_p]
        L.fo_plan_lcs.argtypes = [C.c_void_p]
        L.fo_plan_lcs.restype = C.c_float
        L.fo_plan_work.argtypes = [C.c_void_p, dp]
        L.fo_plan_level_sizes.argtypes = [C.c_void_p, C.c_int, lp, fp]
        L.fo_plan_level_ptr.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.fo_plan_level_ptr.restype = C.c_void_p
        L.fo_plan_apply.argtypes = [C.c_void_p, fp, C.c_int, fp]
        L.fo_plan_far_level.argtypes = [C.c_void_p, C.c_int, fp, C.c_int, fp, fp, fp]
        L.fo_plan_near_level.argtypes = [C.c_void_p, C.c_int, C.c_int, fp, C.c_int, fp]
        L.fo_plan_apply_rows.argtypes = [C.c_void_p, fp, C.c_int, fp, C.c_char_p]
        L.fo_plan_far_level_rows.argtypes = [C.c_void_p, C.c_int, fp, C.c_int, fp, fp, fp, C.c_char_p]
        L.fo_plan_near_level_rows.argtypes = [C.c_void_p, C.c_int, C.c_int, fp, C.c_int, fp, C.c_char_p]
        L.fo_exact_f32.argtypes = [C.c_int, fp, C.c_long, fp, C.c_long, fp, C.c_int, C.c_float, fp]
        L.fo_exact_grad_f32.argtypes = [C.c_int, fp, C.c_long, fp, C.c_long, fp, C.c_int, C.c_float, fp]
        L.fo_exact_f64.argtypes = [C.c_int, dp, C.c_long, dp, C.c_long, dp, C.c_int, C.c_double, dp]
        L.fo_m2l_block.argtypes = [C.c_int, C.c_int, fp, fp, C.c_float, C.c_float, fp]
        L.fo_m2l_block.restype = C.c_int
        up = C.POINTER(C.c_uint32)
        L.fo_hash32.argtypes = [C.c_uint32]
        L.fo_hash32.restype = C.c_uint32
        L.fo_hash_slot.argtypes = [C.c_uint32, C.c_uint32]
        L.fo_hash_slot.restype = C.c_uint32
        L.fo_hash_clear.argtypes = [up, C.c_uint32]
        L.fo_hash_insert.argtypes = [up, C.c_uint32, C.c_uint32, C.c_uint32]
        L.fo_hash_lookup.argtypes = [up, C.c_uint32, C.c_uint32]
        L.fo_hash_lookup.restype = C.c_uint32
        L.fo_cell_key.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_int32)]
        L.fo_cell_key.restype = C.c_int32
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int))


def _dp(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


def nodes_1d(n):
    t = np.empty(n, np.float32)
    w = np.empty(n, np.float32)
    lib().fo_nodes_1d(n, _fp(t), _fp(w))
    return t, w


def node_counts(d, max_nodes):
    out = np.empty(d, np.int32)
    lib().fo_node_counts(d, int(max_nodes), _ip(out))
    return out


def node_grid(d, max_nodes):
    """-> per_dim (d,), nodes_cat, w_cat, idx (P,d), coords (P,d)"""
    per = node_counts(d, max_nodes)
    ts, ws = zip(*[nodes_1d(int(n)) for n in per])
    nodes = np.concatenate(ts)
    w = np.concatenate(ws)
    P = int(np.prod(per))
    idx = np.empty((P, d), np.int32)
    coords = np.empty((P, d), np.float32)
    lib().fo_node_grid(d, _ip(per), _fp(nodes), _ip(idx), _fp(coords))
    return per, nodes, w, idx, coords


def basis(d, nr_interp, x, center, edge):
    per = node_counts(d, nr_interp)
    P = int(np.prod(per))
    out = np.empty(P, np.float32)
    x = _f32(x)
    center = _f32(center)
    lib().fo_basis(d, int(nr_interp), _fp(x), _fp(center), np.float32(edge), _fp(out))
    return out


def root(X, Y=None):
    X = _f32(X)
    d = X.shape[1]
    e = C.c_float()
    xmin = np.empty(d, np.float32)
    ymin = np.empty(d, np.float32)
    if Y is None:
        lib().fo_root(d, _fp(X), X.shape[0], None, 0, C.byref(e), _fp(xmin), _fp(ymin))
    else:
        Y = _f32(Y)
        lib().fo_root(d, _fp(X), X.shape[0], _fp(Y), Y.shape[0], C.byref(e), _fp(xmin), _fp(ymin))
    return np.float32(e.value), xmin, ymin


class Plan:
    """All tree levels and interaction lists of one (X, Y, parameters) problem."""

    def __init__(self, X, Y=None, ls=1.0, min_points=1000, nr_of_interpolation=64, var_compression=False,
                 eff_var_limit=0.15, small_field_points=1000, max_levels=0):
        self.X = _f32(X)
        self.Y = None if Y is None else _f32(Y)
        self.d = self.X.shape[1]
        self.N = self.X.shape[0]
        self.M = self.N if self.Y is None else self.Y.shape[0]
        self._h = lib().fo_plan_create(self.d, _fp(self.X), self.N,
                                       None if self.Y is None else _fp(self.Y), self.M,
                                       float(ls), float(min_points), int(nr_of_interpolation),
                                       int(bool(var_compression)), float(eff_var_limit),
                                       int(small_field_points), int(max_levels))
        st = lib().fo_plan_status(self._h)
        if st:
            msg = lib().fo_plan_message(self._h).decode()
            lib().fo_plan_destroy(self._h)
            self._h = None
            raise RuntimeError("oracle plan failed (%d): %s" % (st, msg))
        self.nlevels = lib().fo_plan_nlevels(self._h)
        self.symmetric = bool(lib().fo_plan_symmetric(self._h))
        self.lcs = np.float32(lib().fo_plan_lcs(self._h))
        w = np.zeros(3, np.float64)
        lib().fo_plan_work(self._h, _dp(w))
        self.work_near_pairs, self.work_far_pairs, self.work_interp_pts = w

    def __del__(self):
        if getattr(self, "_h", None) and lib is not None:      # module globals are gone at interpreter exit
            lib().fo_plan_destroy(self._h)
            self._h = None

    def level(self, k):
        """Level k (0-based: k=0 is depth 1) as a dict of numpy arrays."""
        s = (C.c_long * 6)()
        e = C.c_float()
        lib().fo_plan_level_sizes(self._h, k, s, C.byref(e))
        nbx, nby, nfar, nsmall, nkeep, nn = [int(v) for v in s]
        d = self.d

        def grab(which, shape, dt):
            n = int(np.prod(shape))
            if n == 0:
                return np.zeros(shape, dt)
            p = lib().fo_plan_level_ptr(self._h, k, WHICH[which])
            buf = (C.c_char * (n * np.dtype(dt).itemsize)).from_address(p)
            return np.frombuffer(buf, dtype=dt).reshape(shape).copy()

        return {
            "depth": k + 1, "edge": np.float32(e.value), "num_nodes": nn,
            "cx": grab("cx", (nbx, d), np.float32), "cy": grab("cy", (nby, d), np.float32),
            "cntx": grab("cntx", (nbx,), np.int32), "cnty": grab("cnty", (nby,), np.int32),
            "offx": grab("offx", (nbx + 1,), np.int32), "offy": grab("offy", (nby + 1,), np.int32),
            "permx": grab("permx", (self.N,), np.int32), "permy": grab("permy", (self.M,), np.int32),
            "far": grab("far", (nfar, 2), np.int32), "small": grab("small", (nsmall, 2), np.int32),
            "keep": grab("keep", (nkeep, 2), np.int32),
        }

    def _rowsel(self, rows):
        """Flags (bytes, one per row of X) of the target rows in `rows`, or None for every row."""
        if rows is None:
            return None
        sel = np.zeros(self.N, np.uint8)
        sel[np.asarray(rows, np.int64)] = 1
        return sel.tobytes()

    def apply(self, b, rows=None):
        """The product; with `rows` (indices into X) only those rows are computed, the others stay zero
        (the same sums: M2L only for the boxes that hold a requested row)."""
        b = _f32(b)
        if b.ndim == 1:
            b = b[:, None]
        assert b.shape[0] == self.M
        out = np.zeros((self.N, b.shape[1]), np.float32)
        rc = lib().fo_plan_apply_rows(self._h, _fp(b), b.shape[1], _fp(out), self._rowsel(rows))
        if rc:
            raise RuntimeError("oracle apply failed")
        return out

    def far_level(self, k, b, rows=None):
        """-> (out contribution, moments (nby,P,c), locals (nbx,P,c)) of level k's far field; with `rows`
        the local expansions of boxes without a requested row, and the other rows of out, stay zero."""
        b = _f32(b)
        if b.ndim == 1:
            b = b[:, None]
        c = b.shape[1]
        lv = self.level(k)
        P = int(np.prod(node_counts(self.d, lv["num_nodes"])))
        out = np.zeros((self.N, c), np.float32)
        mom = np.zeros((lv["cy"].shape[0], P, c), np.float32)
        loc = np.zeros((lv["cx"].shape[0], P, c), np.float32)
        lib().fo_plan_far_level_rows(self._h, k, _fp(b), c, _fp(out), _fp(mom), _fp(loc), self._rowsel(rows))
        return out, mom, loc

    def near_level(self, k, which, b, rows=None):
        b = _f32(b)
        if b.ndim == 1:
            b = b[:, None]
        out = np.zeros((self.N, b.shape[1]), np.float32)
        lib().fo_plan_near_level_rows(self._h, k, 0 if which == "small" else 1, _fp(b), b.shape[1], _fp(out),
                                      self._rowsel(rows))
        return out


def kmvm(X, Y, b, **kw):
    """One-shot F3M product by the oracle."""
    return Plan(X, Y, **kw).apply(b)


def exact_f32(X, Y, b, ls):
    X, Y, b = _f32(X), _f32(Y), _f32(b)
    if b.ndim == 1:
        b = b[:, None]
    out = np.empty((X.shape[0], b.shape[1]), np.float32)
    lib().fo_exact_f32(X.shape[1], _fp(X), X.shape[0], _fp(Y), Y.shape[0], _fp(b), b.shape[1], float(ls), _fp(out))
    return out


def exact_grad_f32(X, Y, b, ls):
    X, Y, b = _f32(X), _f32(Y), _f32(b)
    if b.ndim == 1:
        b = b[:, None]
    out = np.empty((X.shape[0], b.shape[1]), np.float32)
    lib().fo_exact_grad_f32(X.shape[1], _fp(X), X.shape[0], _fp(Y), Y.shape[0], _fp(b), b.shape[1], float(ls), _fp(out))
    return out


def exact_f64(X, Y, b, ls):
    X = np.ascontiguousarray(X, np.float64)
    Y = np.ascontiguousarray(Y, np.float64)
    b = np.ascontiguousarray(b, np.float64)
    if b.ndim == 1:
        b = b[:, None]
    out = np.empty((X.shape[0], b.shape[1]), np.float64)
    lib().fo_exact_f64(X.shape[1], _dp(X), X.shape[0], _dp(Y), Y.shape[0], _dp(b), b.shape[1], float(ls), _dp(out))
    return out


def m2l_block(d, nr_interp, cx, cy, edge, lcs):
    per = node_counts(d, nr_interp)
    P = int(np.prod(per))
    K = np.empty((P, P), np.float32)
    cx, cy = _f32(cx), _f32(cy)
    lib().fo_m2l_block(d, int(nr_interp), _fp(cx), _fp(cy), np.float32(edge), np.float32(lcs), _fp(K))
    return K


# ---------------------------------------------------------------------------------------------
# Exact tiled PyTorch CPU product: the CPU baseline timed by bench.py.  The reference has no CPU
# path; this follows the tiling idea of its exact CUDA kernel (F3M_src/1_d_conv.cu:171-214, a
# block of target rows against successive source tiles) behind benchmark_matmul
# (experiments/FFM_classes.py:264-323).

def hash32(k):
    """Murmur3 32-bit finaliser (F3M_src/linearprobing.cu:18-26 before the reduction)."""
    return int(lib().fo_hash32(int(k) & 0xffffffff))


def hash_slot(key, capacity):
    return int(lib().fo_hash_slot(int(key) & 0xffffffff, int(capacity)))


def grid_key(d, k, cell):
    c = np.ascontiguousarray(np.asarray(cell, np.int32))
    return int(lib().fo_cell_key(int(d), int(k), c.ctypes.data_as(C.POINTER(C.c_int32))))


class HashTable:
    """Key -> value table of F3M_src/linearprobing.cu:41-87 (capacity pairs of uint32, empty = 0xffffffff)."""

    def __init__(self, capacity):
        self.capacity = int(capacity)
        self.table = np.empty(2 * self.capacity, np.uint32)
        lib().fo_hash_clear(self._p(), self.capacity)

    def _p(self):
        return self.table.ctypes.data_as(C.POINTER(C.c_uint32))

    def insert(self, key, value):
        lib().fo_hash_insert(self._p(), self.capacity, int(key) & 0xffffffff, int(value) & 0xffffffff)

    def lookup(self, key):
        v = int(lib().fo_hash_lookup(self._p(), self.capacity, int(key) & 0xffffffff))
        return -1 if v == 0xffffffff else v


def exact_tiled_torch(X, Y, b, ls, row_tile=2048, col_tile=16384, dtype=None):
    import torch
    X = torch.as_tensor(X)
    Y = torch.as_tensor(Y)
    b = torch.as_tensor(b)
    if dtype is not None:
        X, Y, b = X.to(dtype), Y.to(dtype), b.to(dtype)
    if b.dim() == 1:
        b = b[:, None]
    lcs = 1.0 / (2.0 * float(ls) * float(ls))
    out = torch.zeros(X.shape[0], b.shape[1], dtype=X.dtype)
    y2 = (Y * Y).sum(1)
    for i0 in range(0, X.shape[0], row_tile):
        xi = X[i0:i0 + row_tile]
        x2 = (xi * xi).sum(1, keepdim=True)
        acc = torch.zeros(xi.shape[0], b.shape[1], dtype=X.dtype)
        for j0 in range(0, Y.shape[0], col_tile):
            yj = Y[j0:j0 + col_tile]
            r2 = (x2 + y2[j0:j0 + col_tile][None, :] - 2.0 * (xi @ yj.T)).clamp_min_(0)
            acc += torch.exp_(r2.mul_(-lcs)) @ b[j0:j0 + col_tile]
        out[i0:i0 + row_tile] = acc
    return out


def rel_l2(approx, truth):
    """||t-a||_2 / ||t||_2  (experiments/run_obj.py:100-101)."""
    a = np.asarray(approx, np.float64)
    t = np.asarray(truth, np.float64)
    return float(np.linalg.norm(t - a) / np.linalg.norm(t))
