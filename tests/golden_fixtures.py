"""Loads tests/golden/oracle_fixtures.npz (written by tests/golden/make_oracle_fixtures.py: outputs of this
repository's CPU oracle on small seeded clouds, not outputs of the reference) and checks a plan against
a case of it."""
import os

import numpy as np

from helpers import box_of_point
from parity_checks import rel_l2

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "oracle_fixtures.npz")
PARAM_KEYS = ("ls", "min_points", "nr_of_interpolation", "small_field_points", "var_compression", "eff_var_limit")


def load():
    return np.load(PATH, allow_pickle=False)


def names():
    return load()["names"].tolist()


def case(fx, name):
    X, Y, b = fx[name + "/X"], fx[name + "/Y"], fx[name + "/b"]
    p = dict(zip(PARAM_KEYS, fx[name + "/params"].tolist()))
    p["nr_of_interpolation"] = int(p["nr_of_interpolation"])
    p["small_field_points"] = int(p["small_field_points"])
    p["var_compression"] = bool(p["var_compression"])
    return X, (None if Y.shape[0] == 0 else Y), b, p


def assert_plan_matches_fixture(plan, depth, fx, name):
    """plan.level(k) (k = 1..depth) must give the fixture's offsets, centres (bit patterns), per-point box
    ids and the three lists, bit for bit."""
    assert depth == int(fx[name + "/depth"]), (name, depth)
    for k in range(1, depth + 1):
        L = plan.level(k)
        pre = "%s/level%d/" % (name, k)
        assert np.float32(L["edge"]) == fx[pre + "edge"], (name, k)
        for w in ("x", "y"):
            assert np.array_equal(L["off" + w], fx[pre + "off" + w]), (name, k, w, "offsets")
            assert np.array_equal(np.asarray(L["c" + w], np.float32).view(np.uint32), fx[pre + "centres_bits_" + w]), (name, k, w)
            assert np.array_equal(box_of_point(L, w), fx[pre + "box_of_point_" + w]), (name, k, w, "box ids")
        for lst in ("far", "small", "keep"):
            assert np.array_equal(np.asarray(L[lst]).reshape(-1, 2), fx[pre + lst]), (name, k, lst)


def assert_product_matches_fixture(got, fx, name, tol=1e-5):
    """the engine's product against the oracle's stored one, and its error against the stored fp64 exact
    product no worse than 1.5x the oracle's (plus 3e-6: the fp32 evaluation floor of exp2 and of a
    different summation order, which matters where the oracle's own error is that small)"""
    want, exact = fx[name + "/product_oracle"], fx[name + "/product_exact_f64"]
    assert rel_l2(got, want) < tol, (name, rel_l2(got, want))
    assert rel_l2(got, exact) <= 1.5 * rel_l2(want, exact) + 3e-6, (name, rel_l2(got, exact), rel_l2(want, exact))
