"""ctypes declarations of the C ABI in include/f3m.h."""
import ctypes as C

LEVEL_ARRAYS = {"cx": 0, "cy": 1, "offx": 2, "offy": 3, "far": 4, "small": 5, "keep": 6, "permx": 7, "permy": 8}
STAGES = ("plan", "near", "p2m", "m2l", "l2p", "perm")


class F3MParams(C.Structure):
    _fields_ = [("ls", C.c_float), ("min_points", C.c_float), ("nr_of_interpolation", C.c_int),
                ("var_compression", C.c_int), ("eff_var_limit", C.c_float), ("small_field_points", C.c_int)]


class F3MError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("f3m error %d: %s" % (code, msg))
        self.code = code


SYMBOLS = [
    "f3m_kmvm_f32", "f3m_exact_f32", "f3m_exact_grad_f32", "f3m_exact_f64", "f3m_plan_create", "f3m_plan_apply",
    "f3m_plan_apply_noalloc", "f3m_plan_apply_transpose", "f3m_plan_destroy", "f3m_plan_depth", "f3m_plan_symmetric", "f3m_plan_level_sizes", "f3m_plan_list_rows", "f3m_plan_level_copy",
    "f3m_plan_far_level", "f3m_plan_near_level", "f3m_plan_work", "f3m_plan_lookup_boxes", "f3m_hash_slot",
    "f3m_set_timing", "f3m_get_timing",
    "f3m_last_error", "f3m_release_cache", "f3m_version",
]


def bind(lib):
    """Declare argument and result types on a loaded library; returns it."""
    vp, i64, i, f, dbl = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_double
    pp = C.POINTER(F3MParams)
    lib.f3m_kmvm_f32.argtypes = [i, vp, i64, vp, i64, vp, i, pp, vp, vp]
    lib.f3m_exact_f32.argtypes = [i, vp, i64, vp, i64, vp, i, f, vp, vp]
    lib.f3m_exact_grad_f32.argtypes = [i, vp, i64, vp, i64, vp, i, f, vp, vp]
    lib.f3m_exact_f64.argtypes = [i, vp, i64, vp, i64, vp, i, dbl, vp, vp]
    lib.f3m_plan_create.argtypes = [i, vp, i64, vp, i64, pp, vp, C.POINTER(vp)]
    lib.f3m_plan_apply.argtypes = [vp, vp, i, vp, vp]
    lib.f3m_plan_apply_noalloc.argtypes = [vp, vp, i, vp, vp]
    lib.f3m_plan_apply_transpose.argtypes = [vp, vp, i, vp, vp]
    lib.f3m_plan_destroy.argtypes = [vp]
    lib.f3m_plan_depth.argtypes = [vp]
    lib.f3m_plan_symmetric.argtypes = [vp]
    lib.f3m_plan_level_sizes.argtypes = [vp, i, C.POINTER(i64), C.POINTER(f)]
    lib.f3m_plan_list_rows.argtypes = [vp, i, C.POINTER(i64)]
    lib.f3m_plan_level_copy.argtypes = [vp, i, i, vp, vp]
    lib.f3m_plan_far_level.argtypes = [vp, i, vp, i, vp, vp, vp, vp]
    lib.f3m_plan_near_level.argtypes = [vp, i, i, vp, i, vp, vp]
    lib.f3m_plan_work.argtypes = [vp, C.POINTER(dbl)]
    lib.f3m_set_timing.argtypes = [i]
    lib.f3m_get_timing.argtypes = [C.POINTER(dbl), C.POINTER(i)]
    lib.f3m_last_error.restype = C.c_char_p
    lib.f3m_version.restype = C.c_char_p
    lib.f3m_plan_lookup_boxes.argtypes = [vp, i, i, vp, i64, vp, vp]
    lib.f3m_hash_slot.argtypes = [C.c_uint32, C.c_uint32]
    lib.f3m_hash_slot.restype = C.c_uint32
    for name in SYMBOLS:
        fn = getattr(lib, name)
        if name not in ("f3m_last_error", "f3m_version", "f3m_hash_slot"):
            fn.restype = C.c_int
    return lib


def check(lib, rc):
    if rc != 0:
        raise F3MError(rc, lib.f3m_last_error().decode(errors="replace"))


def make_params(ls=1.0, min_points=1000, nr_of_interpolation=64, var_compression=False, eff_var_limit=0.15,
                small_field_points=1000):
    return F3MParams(float(ls), float(min_points), int(nr_of_interpolation), int(bool(var_compression)),
                     float(eff_var_limit), int(small_field_points))
