"""Drop-in for the reference's compiled module ``ffm_3d_float`` (F3M_src/pybinder_setup.cu:7-72,
F3M_src/setup.py:9-12): the same 40 function names with the same positional arguments, backed by
the gfx950 C ABI.

    FFM_XY_FLOAT_{1..10}(X, Y, b, device, ls, min_points, nr_of_interpolation, var_compression,
                         eff_var_limit, small_field_points) -> (N, c) float32
    rbf_float_{1..10}(X, Y, b, ls, shared) / rbf_float_{1..10}_grad(...) -> (N, c) float32
    rbf_double_{1..10}(X, Y, b, ls, shared) -> (N, c) float64

``X.data_ptr() == Y.data_ptr()`` selects the symmetric case, as in F3M_src/n_tree.cu:1072.  The
``device`` string and the ``shared`` flag are accepted for compatibility; tensors decide the device.
"""
from . import engine


def _make_ffm(nd):
    def fn(X, Y, b, device, ls, min_points, nr_of_interpolation, var_compression, eff_var_limit, small_field_points):
        if X.shape[1] != nd:
            raise RuntimeError("FFM_XY_FLOAT_%d called with %d-dimensional data" % (nd, X.shape[1]))
        return engine.kmvm(X, Y, b, ls=ls, min_points=min_points, nr_of_interpolation=nr_of_interpolation,
                           var_compression=var_compression, eff_var_limit=eff_var_limit,
                           small_field_points=small_field_points)
    fn.__name__ = "FFM_XY_FLOAT_%d" % nd
    fn.__doc__ = "xy %d (reference: FFM_XY<float,%d>, F3M_src/n_tree.cu:1056-1125)" % (nd, nd)
    return fn


def _make_rbf(nd, which):
    impl = {"float": engine.exact_f32, "grad": engine.exact_grad_f32, "double": engine.exact_f64}[which]

    def fn(X, Y, b, ls, shared=True):
        if X.shape[1] != nd:
            raise RuntimeError("rbf_%s_%d called with %d-dimensional data" % (which, nd, X.shape[1]))
        return impl(X, Y, b, ls)
    return fn


for _nd in range(1, 11):
    globals()["FFM_XY_FLOAT_%d" % _nd] = _make_ffm(_nd)
    globals()["rbf_float_%d" % _nd] = _make_rbf(_nd, "float")
    globals()["rbf_float_%d_grad" % _nd] = _make_rbf(_nd, "grad")
    globals()["rbf_double_%d" % _nd] = _make_rbf(_nd, "double")
del _nd

__all__ = [n for n in globals() if n.startswith(("FFM_XY_FLOAT_", "rbf_float_", "rbf_double_"))]
