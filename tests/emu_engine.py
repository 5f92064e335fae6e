"""TEST INFRASTRUCTURE: numpy front end of the CPU-emulated build of the engine's kernel sources
(tests/cpu_emu).  Mirrors f3m_amd.engine.Plan closely enough that the same checks run against the
emulated kernels here and against the gfx950 library on a GPU."""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "cpu_emu"))

from f3m_amd import capi  # noqa: E402  (ctypes declarations only; loads nothing)

_lib = None


def lib():
    global _lib
    if _lib is None:
        import build_emu
        _lib = capi.bind(C.CDLL(build_emu.build()))
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, np.float32))


def exact(fn, X, Y, b, ls, dtype=np.float32):
    X, Y, b = (np.ascontiguousarray(np.asarray(v, dtype)) for v in (X, Y, b))
    out = np.empty((X.shape[0], b.shape[1]), dtype)
    capi.check(lib(), getattr(lib(), fn)(X.shape[1], _p(X), X.shape[0], _p(Y), Y.shape[0], _p(b), b.shape[1],
                                         float(ls), _p(out), None))
    return out


def kmvm(X, Y, b, **kw):
    X, b = _f32(X), _f32(b)
    Yc = None if Y is None else _f32(Y)
    out = np.empty((X.shape[0], b.shape[1]), np.float32)
    prm = capi.make_params(**kw)
    capi.check(lib(), lib().f3m_kmvm_f32(X.shape[1], _p(X), X.shape[0], None if Yc is None else _p(Yc),
                                         0 if Yc is None else Yc.shape[0], _p(b), b.shape[1], C.byref(prm), _p(out), None))
    return out


class Plan:
    def __init__(self, X, Y=None, **kw):
        self.X = _f32(X)
        self.Y = None if Y is None else _f32(Y)
        self.d, self.N = self.X.shape[1], self.X.shape[0]
        self.M = self.N if self.Y is None else self.Y.shape[0]
        prm = capi.make_params(**kw)
        h = C.c_void_p()
        capi.check(lib(), lib().f3m_plan_create(self.d, _p(self.X), self.N, None if self.Y is None else _p(self.Y),
                                                self.M, C.byref(prm), None, C.byref(h)))
        self._h = h
        self.depth = lib().f3m_plan_depth(h)

    def __del__(self):
        if getattr(self, "_h", None) is not None:
            lib().f3m_plan_destroy(self._h)
            self._h = None

    def level_sizes(self, level):
        s = (C.c_int64 * 8)()
        e = C.c_float()
        capi.check(lib(), lib().f3m_plan_level_sizes(self._h, level, s, C.byref(e)))
        keys = ("nbx", "nby", "nfar", "nsmall", "nkeep", "num_nodes", "maxcount_x", "maxcount_y")
        out = {k: int(v) for k, v in zip(keys, s)}
        out["edge"] = np.float32(e.value)
        return out

    def list_rows(self, level):
        r = (C.c_int64 * 8)()
        capi.check(lib(), lib().f3m_plan_list_rows(self._h, level, r))
        return [int(v) for v in r]

    def lookup_boxes(self, level, cells, tree="x"):
        cells = np.ascontiguousarray(np.asarray(cells, np.int32))
        ids = np.empty(cells.shape[0], np.int32)
        capi.check(lib(), lib().f3m_plan_lookup_boxes(self._h, level, 0 if tree == "x" else 1, _p(cells), cells.shape[0],
                                                      _p(ids), None))
        return ids

    def level(self, level):
        sz = self.level_sizes(level)
        shapes = {
            "cx": ((sz["nbx"], self.d), np.float32), "cy": ((sz["nby"], self.d), np.float32),
            "offx": ((sz["nbx"] + 1,), np.int32), "offy": ((sz["nby"] + 1,), np.int32),
            "far": ((sz["nfar"], 2), np.int32), "small": ((sz["nsmall"], 2), np.int32),
            "keep": ((sz["nkeep"], 2), np.int32), "permx": ((self.N,), np.int32), "permy": ((self.M,), np.int32),
        }
        out = dict(sz)
        for name, (shape, dt) in shapes.items():
            a = np.zeros(shape, dt)
            if a.size:
                capi.check(lib(), lib().f3m_plan_level_copy(self._h, level, capi.LEVEL_ARRAYS[name], _p(a), None))
            out[name] = a
        return out

    def apply(self, b):
        b = _f32(b)
        out = np.empty((self.N, b.shape[1]), np.float32)
        capi.check(lib(), lib().f3m_plan_apply(self._h, _p(b), b.shape[1], _p(out), None))
        return out

    def apply_transpose(self, u):
        u = _f32(u)
        out = np.empty((self.M, u.shape[1]), np.float32)
        capi.check(lib(), lib().f3m_plan_apply_transpose(self._h, _p(u), u.shape[1], _p(out), None))
        return out

    def far_level(self, level, b, P):
        b = _f32(b)
        sz = self.level_sizes(level)
        out = np.zeros((self.N, b.shape[1]), np.float32)
        mom = np.zeros((b.shape[1], sz["nby"], P), np.float32)
        loc = np.zeros((b.shape[1], sz["nbx"], P), np.float32)
        capi.check(lib(), lib().f3m_plan_far_level(self._h, level, _p(b), b.shape[1], _p(out), _p(mom), _p(loc), None))
        return out, mom, loc

    def near_level(self, level, which, b):
        b = _f32(b)
        out = np.zeros((self.N, b.shape[1]), np.float32)
        capi.check(lib(), lib().f3m_plan_near_level(self._h, level, capi.LEVEL_ARRAYS[which], _p(b), b.shape[1], _p(out), None))
        return out

    def work(self):
        w = (C.c_double * 5)()
        capi.check(lib(), lib().f3m_plan_work(self._h, w))
        return list(w)
