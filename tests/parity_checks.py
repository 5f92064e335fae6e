"""Checks shared by the CPU-emulation tests and the GPU tests: an engine plan (anything with the
interface of f3m_amd.engine.Plan.level) against the oracle's plan."""
import numpy as np


def canonical_box_of_point(level, which):
    perm, off = level["perm" + which], level["off" + which]
    box = np.empty(perm.shape[0], np.int64)
    box[perm] = np.repeat(np.arange(off.shape[0] - 1), np.diff(off))
    return box


def assert_plan_matches_oracle(eng_plan, ora_plan, depth_attr="depth"):
    """Bit-exact: depth, per-point box ids, counts, centres (as bit patterns) and the three lists."""
    depth = getattr(eng_plan, depth_attr)
    assert depth == ora_plan.nlevels, (depth, ora_plan.nlevels)
    for k in range(1, depth + 1):
        E = eng_plan.level(k)
        O = ora_plan.level(k - 1)
        assert E["edge"] == O["edge"], k
        for w in ("x", "y"):
            assert np.array_equal(E["off" + w], O["off" + w]), (k, w, "offsets")
            assert np.array_equal(E["c" + w].view(np.uint32), O["c" + w].view(np.uint32)), (k, w, "centres")
            assert np.array_equal(canonical_box_of_point(E, w), canonical_box_of_point(O, w)), (k, w, "box ids")
            assert np.array_equal(np.sort(E["perm" + w]), np.arange(E["perm" + w].shape[0]))
        for name in ("far", "small", "keep"):
            assert E[name].shape == O[name].shape, (k, name, E[name].shape, O[name].shape)
            assert np.array_equal(E[name], O[name]), (k, name)


def rel_l2(a, t):
    a = np.asarray(a, np.float64)
    t = np.asarray(t, np.float64)
    return float(np.linalg.norm(a - t) / np.linalg.norm(t))


def expected_list_rows(level):
    """row statistics of the small and keep list of a level (dict of Plan.level): boxes with pairs, their
    points, their pieces of 128 and of 160 points"""
    cnt = np.diff(np.asarray(level["offx"], np.int64))
    out = []
    for which in ("small", "keep"):
        pairs = np.asarray(level[which]).reshape(-1, 2)
        n = cnt[np.unique(pairs[:, 0])] if len(pairs) else np.zeros(0, np.int64)
        out += [len(n), int(n.sum()), int(((n + 127) // 128).sum()), int(((n + 159) // 160).sum())]
    return out
