"""Runs the engine's real kernel sources, compiled for the CPU by tests/cpu_emu, against the oracle
on small inputs: box division and lists bit-exact, every numeric stage within tolerance.  These are
logic tests of the HIP code (indexing, barriers, ballots); numerics on the device are covered by
the -m gpu tests."""
import numpy as np
import pytest

import emu_engine as ee
from helpers import box_of_point, cell_coords
from parity_checks import assert_plan_matches_oracle, rel_l2

f32 = np.float32


def _cloud(name, rng):
    if name == "uniform3":
        return rng.random((3000, 3), dtype=f32), None
    if name == "normal2":
        return rng.standard_normal((2500, 2)).astype(f32), None
    if name == "uniform1":
        return rng.random((1200, 1), dtype=f32), None
    if name == "uniform4":
        return rng.random((3000, 4), dtype=f32), None
    if name == "asym3":
        X = rng.standard_normal((2500, 3)).astype(f32)
        Y = (rng.random((1800, 3)) * 5 - 2.5).astype(f32)
        return X, Y
    if name == "dups_faces":
        g = (np.stack(np.meshgrid(*[np.arange(9)] * 3, indexing="ij"), -1).reshape(-1, 3) / 8.0).astype(f32)
        return np.concatenate([g, g[::-1], g[::3]]), None
    raise KeyError(name)


PRM = dict(ls=0.6, min_points=60, nr_of_interpolation=27, small_field_points=40)


@pytest.fixture(autouse=True)
def _vector_near_kernel(monkeypatch):
    # the emulated matrix instruction costs two fiber barriers per call; the bulk of these tests
    # therefore runs the all-vector near-field kernel and test_mfma_near_field covers the other one
    monkeypatch.setenv("F3M_NEAR", "valu")


@pytest.mark.parametrize("name", ["uniform3", "normal2", "uniform1", "uniform4", "asym3", "dups_faces"])
def test_tree_and_lists_bit_exact(oracle, name):
    X, Y = _cloud(name, np.random.default_rng(21))
    eng = ee.Plan(X, Y, **PRM)
    ora = oracle.Plan(X, Y, **PRM)
    assert_plan_matches_oracle(eng, ora)
    w = eng.work()
    assert w[0] == ora.work_near_pairs and w[1] == ora.work_far_pairs and w[2] == ora.work_interp_pts


def test_level_scans_one_by_one(oracle, monkeypatch):
    """The level loop scans its list counts and its "candidate box is not empty" flags in one set of launches; levels
    with more than 2048 x 2048 boxes take the scans one after the other.  F3M_LEVEL_SCANS=separate forces that path:
    same tree, same lists."""
    monkeypatch.setenv("F3M_LEVEL_SCANS", "separate")
    for name in ("uniform3", "asym3"):
        X, Y = _cloud(name, np.random.default_rng(21))
        assert_plan_matches_oracle(ee.Plan(X, Y, **PRM), oracle.Plan(X, Y, **PRM))


def test_deep_tree_bit_exact(oracle):
    """A tight cluster inside a sparse cloud forces divisions down to the depth cap; the engine sorts
    further key bits only when a division needs them."""
    rng = np.random.default_rng(12)
    X = np.concatenate([rng.normal(0.3, 1e-3, (2000, 3)), rng.random((500, 3))]).astype(f32)
    eng = ee.Plan(X, None, **PRM)
    assert eng.depth >= 9
    assert_plan_matches_oracle(eng, oracle.Plan(X, None, **PRM))
    b = rng.standard_normal((2500, 1)).astype(f32)
    assert rel_l2(eng.apply(b), oracle.Plan(X, None, **PRM).apply(b)) < 1e-5


@pytest.mark.parametrize("name", ["uniform3", "asym3", "normal2"])
def test_box_lookup_by_cell(oracle, name):
    """Grid cell -> box id through the engine's open-addressing table: every point's cell (restated in
    numpy) gives the box that holds the point; cells without points give -1; the slot function is the
    reference's (F3M_src/linearprobing.cu:18-26)."""
    X, Y = _cloud(name, np.random.default_rng(21))
    eng = ee.Plan(X, Y, **PRM)
    edge0, xmin, ymin = oracle.root(X, Y)
    for tree, pts, org in (("x", X, xmin), ("y", X if Y is None else Y, xmin if Y is None else ymin)):
        for k in range(1, eng.depth + 1):
            L = eng.level(k)
            cells = cell_coords(pts, org, edge0, k).astype(np.int32)
            assert np.array_equal(eng.lookup_boxes(k, cells, tree), box_of_point(L, tree))
            side = 1 << k
            grid = np.stack(np.meshgrid(*[np.arange(-1, side + 1)] * X.shape[1], indexing="ij"), -1)
            grid = grid.reshape(-1, X.shape[1])[:: max(1, (side + 2) ** X.shape[1] // 5000)].astype(np.int32)
            occupied = {tuple(c) for c in cells.tolist()}
            got = eng.lookup_boxes(k, grid, tree)
            for c, g in zip(grid.tolist(), got.tolist()):
                assert (g >= 0) == (tuple(c) in occupied)
    for key, cap in ((1, 1 << 20), (0xFFFFFFFF, 1024), (123456789, 4096), (0, 2048)):
        assert ee.lib().f3m_hash_slot(key, cap) == oracle.hash_slot(key, cap)


def test_var_compression_lists_bit_exact(oracle):
    X, _ = _cloud("uniform3", np.random.default_rng(3))
    prm = dict(PRM, var_compression=True, eff_var_limit=0.3, ls=2.0)
    assert_plan_matches_oracle(ee.Plan(X, None, **prm), oracle.Plan(X, None, **prm))


def test_exact_kernels(oracle):
    rng = np.random.default_rng(0)
    for d in (1, 3, 5):
        X = rng.standard_normal((300, d)).astype(f32)
        Y = rng.standard_normal((700, d)).astype(f32)
        b = rng.standard_normal((700, 2)).astype(f32)
        ref = oracle.exact_f64(X, Y, b, 0.8)
        assert rel_l2(ee.exact("f3m_exact_f32", X, Y, b, 0.8), ref) < 1e-5
        assert rel_l2(ee.exact("f3m_exact_f64", X, Y, b, 0.8, np.float64), ref) < 1e-12
        assert rel_l2(ee.exact("f3m_exact_grad_f32", X, Y, b, 0.8), oracle.exact_grad_f32(X, Y, b, 0.8)) < 1e-5


@pytest.mark.parametrize("name,P", [("uniform3", 27), ("normal2", 16), ("asym3", 64), ("uniform4", 16)])
def test_stages_and_product(oracle, name, P):
    rng = np.random.default_rng(8)
    X, Y = _cloud(name, rng)
    M = X.shape[0] if Y is None else Y.shape[0]
    b = rng.standard_normal((M, 2)).astype(f32)
    prm = dict(PRM, nr_of_interpolation=P)
    eng = ee.Plan(X, Y, **prm)
    ora = oracle.Plan(X, Y, **prm)
    nodes = int(np.prod(oracle.node_counts(X.shape[1], P)))
    did_far = False
    for k in range(1, eng.depth + 1):
        sz = eng.level_sizes(k)
        if sz["nsmall"]:
            assert rel_l2(eng.near_level(k, "small", b), ora.near_level(k - 1, "small", b)) < 1e-5
        if sz["nfar"]:
            did_far = True
            out, mom, loc = eng.far_level(k, b, nodes)
            o_out, o_mom, o_loc = ora.far_level(k - 1, b)
            assert rel_l2(mom, np.moveaxis(o_mom, 2, 0)) < 1e-4
            assert rel_l2(loc, np.moveaxis(o_loc, 2, 0)) < 1e-4
            assert rel_l2(out, o_out) < 1e-4
    assert did_far
    if eng.level_sizes(eng.depth)["nkeep"]:
        assert rel_l2(eng.near_level(eng.depth, "keep", b), ora.near_level(eng.depth - 1, "keep", b)) < 1e-5
    got = eng.apply(b)
    assert rel_l2(got, ora.apply(b)) < 1e-5
    exact = oracle.exact_f64(X, X if Y is None else Y, b, prm["ls"])
    assert rel_l2(got, exact) <= 1.5 * rel_l2(ora.apply(b), exact) + 1e-6
    assert rel_l2(ee.kmvm(X, Y, b, **prm), got) == 0.0


@pytest.mark.parametrize("name,P", [("asym3", 64), ("asym3", 27)])
def test_transposed_product_on_the_same_plan(oracle, name, P):
    """K(X,Y)^T u from the plan of (X, Y) -- trees swapped, lists read from their Y boxes -- is what the plan
    of (Y, X) gives, bit for bit (same lists, same kernels, same order), and the oracle's product of (Y, X)."""
    rng = np.random.default_rng(23)
    X, Y = _cloud(name, rng)
    u = rng.standard_normal((X.shape[0], 2)).astype(f32)
    prm = dict(PRM, nr_of_interpolation=P)
    fwd, bwd = ee.Plan(X, Y, **prm), ee.Plan(Y, X, **prm)
    assert fwd.depth == bwd.depth and sum(fwd.level_sizes(k)["nfar"] for k in range(1, fwd.depth + 1)) > 0
    for k in range(1, fwd.depth + 1):                       # the lists of (Y, X) are the transposed lists of (X, Y)
        A, B = fwd.level(k), bwd.level(k)
        for lst in ("far", "small", "keep"):
            t = A[lst][:, ::-1]
            assert np.array_equal(t[np.lexsort((t[:, 1], t[:, 0]))], B[lst]), (k, lst)
    got = fwd.apply_transpose(u)
    assert np.array_equal(got, bwd.apply(u))
    assert rel_l2(got, oracle.kmvm(Y, X, u, **prm)) < 1e-5
    assert np.array_equal(fwd.apply_transpose(u[:, :1]), got[:, :1])       # the kept transposed lists, one column
    # one tree: K(X,X) is symmetric, the transposed product is the product
    sym = ee.Plan(X, None, **prm)
    assert np.array_equal(sym.apply_transpose(u), sym.apply(u))


def test_far_sweeps_match_per_level_interpolation(oracle, monkeypatch):
    """The engine interpolates the points once and moves moments / local expansions between levels;
    F3M_FAR=levels interpolates every level from the points as the reference does
    (F3M_src/n_tree.cu:489-593).  Both are the same sums up to rounding."""
    rng = np.random.default_rng(21)
    X = rng.random((8000, 2), dtype=f32)
    b = rng.standard_normal((8000, 2)).astype(f32)
    prm = dict(ls=0.7, min_points=60, nr_of_interpolation=9, small_field_points=4)
    eng = ee.Plan(X, None, **prm)
    far_levels = [k for k in range(1, eng.depth + 1) if eng.level_sizes(k)["nfar"]]
    assert len(far_levels) >= 3                      # moments travel through at least two levels
    sweeps = eng.apply(b)
    monkeypatch.setenv("F3M_FAR", "levels")
    per_level = eng.apply(b)
    assert 0 < rel_l2(sweeps, per_level) < 2e-6       # two code paths, same sums up to rounding
    assert rel_l2(sweeps, oracle.Plan(X, None, **prm).apply(b)) < 1e-5


def test_far_sweeps_with_level_dependent_node_counts(oracle, monkeypatch):
    """var_compression lowers the node count of deep levels (F3M_src/n_tree.cu:971-978): expansions
    cannot be handed from a 4x4 grid to a 3x3 grid exactly, so those levels are interpolated directly."""
    rng = np.random.default_rng(22)
    X = rng.random((4000, 2), dtype=f32)
    b = rng.standard_normal((4000, 1)).astype(f32)
    prm = dict(ls=1.0, min_points=100, nr_of_interpolation=16, small_field_points=10, var_compression=True,
               eff_var_limit=0.1)
    eng = ee.Plan(X, None, **prm)
    used = {eng.level_sizes(k)["num_nodes"] for k in range(1, eng.depth + 1) if eng.level_sizes(k)["nfar"]}
    assert used == {16, 9}
    sweeps = eng.apply(b)
    assert rel_l2(sweeps, oracle.Plan(X, None, **prm).apply(b)) < 1e-5
    monkeypatch.setenv("F3M_FAR", "levels")
    assert rel_l2(sweeps, eng.apply(b)) < 2e-6


@pytest.mark.parametrize("d,n,P,mp", [(3, 3000, 27, 60), (4, 3000, 16, 60), (3, 3000, 8, 30)])
def test_m2l_forms_agree(monkeypatch, d, n, P, mp):
    """Three forms of M2L: sibling-group separable (default here), per-box separable, direct
    (the reference's, F3M_src/1_d_conv.cu:741-817).  Same sums up to rounding."""
    rng = np.random.default_rng(3)
    X = rng.random((n, d), dtype=f32)
    b = rng.standard_normal((n, 1)).astype(f32)
    eng = ee.Plan(X, None, ls=0.6, min_points=mp, nr_of_interpolation=P, small_field_points=P + 10)
    assert any(eng.level_sizes(k)["nfar"] for k in range(1, eng.depth + 1))
    grouped = eng.apply(b)
    monkeypatch.setenv("F3M_M2L", "separable")
    per_box = eng.apply(b)
    monkeypatch.setenv("F3M_M2L", "direct")
    direct = eng.apply(b)
    assert 0 < rel_l2(grouped, per_box) < 2e-6
    assert rel_l2(grouped, direct) < 3e-6


@pytest.mark.parametrize("d,n", [(4, 2000), (5, 5000)])
def test_m2l_cells_listed_by_every_sibling_summed_once(oracle, monkeypatch, d, n):
    """3^4 and 3^5 grids: the far cells that every child of a parent lists are summed once per combination of sibling
    bits (m2l_shared_kernel), the sibling-group kernel adds the rest.  A thin slab (two long dimensions) reaches the
    third level, where such cells exist, with a few thousand points.  Same sums as the sibling-group kernel alone up
    to rounding, and as the oracle's."""
    rng = np.random.default_rng(9)
    X = rng.random((n, d), dtype=f32)
    X[:, 2:] *= 0.12
    b = rng.standard_normal((n, 1)).astype(f32)
    prm = dict(ls=0.3, min_points=50, nr_of_interpolation=3 ** d, small_field_points=2)
    eng = ee.Plan(X, None, **prm)
    assert eng.depth == 3 and eng.level_sizes(2)["nfar"] > 100
    monkeypatch.setenv("F3M_M2L_SHARED", "1")
    shared = eng.apply(b)
    monkeypatch.setenv("F3M_M2L_SHARED", "0")
    plain = eng.apply(b)
    assert 0 < rel_l2(shared, plain) < 1e-6            # not the same bits: some cells did go the other way
    assert rel_l2(shared, oracle.Plan(X, None, **prm).apply(b)) < 3e-6


@pytest.mark.parametrize("P", [125, 216])
def test_grids_of_five_and_six_nodes_per_dimension(oracle, monkeypatch, P):
    """5 x 5 x 5 and 6 x 6 x 6 nodes (the grids of the reference's own sweep, experiments/experiments.py:47-49) on
    their one-wavefront kernels: interpolation, sibling-group M2L, transfers between two levels, evaluation.  A thin
    slab keeps the near field small for the emulation: 8 x 8 x 1 boxes of ~230 points at depth 3, far pairs at depths
    2 and 3, half of every family of siblings missing."""
    rng = np.random.default_rng(9)
    X = (rng.random((15000, 3)) * np.array([1.0, 1.0, 1e-3])).astype(f32)
    b = rng.standard_normal((15000, 1)).astype(f32)
    prm = dict(ls=0.6, min_points=300, nr_of_interpolation=P, small_field_points=300)
    eng = ee.Plan(X, None, **prm)
    ora = oracle.Plan(X, None, **prm)
    assert_plan_matches_oracle(eng, ora)
    far_levels = [k for k in range(1, eng.depth + 1) if eng.level_sizes(k)["nfar"]]
    assert len(far_levels) >= 2
    for k in far_levels:                                  # P2M and M2L of every level against the oracle
        out, mom, loc = eng.far_level(k, b, P)
        o_out, o_mom, o_loc = ora.far_level(k - 1, b)
        assert rel_l2(mom, np.moveaxis(o_mom, 2, 0)) < 1e-4
        assert rel_l2(loc, np.moveaxis(o_loc, 2, 0)) < 1e-4
        assert rel_l2(out, o_out) < 1e-4
    sweeps = eng.apply(b)                                 # one interpolation, transfers between the levels, one evaluation
    assert rel_l2(sweeps, ora.apply(b)) < 1e-5
    monkeypatch.setenv("F3M_FAR", "levels")
    assert 0 < rel_l2(sweeps, eng.apply(b)) < 3e-6
    monkeypatch.delenv("F3M_FAR")
    monkeypatch.setenv("F3M_M2L", "direct")
    assert 0 < rel_l2(sweeps, eng.apply(b)) < 3e-6


@pytest.mark.parametrize("parts", [2, 6])
def test_m2l_sibling_table_in_parts(monkeypatch, parts):
    """the sibling-group M2L can fill and walk its table of far cells in several parts (for tables that do not fit LDS whole):
    same sums as in one part, bit for bit, because the walking order does not change"""
    rng = np.random.default_rng(4)
    X = rng.random((3000, 3), dtype=f32)
    b = rng.standard_normal((3000, 1)).astype(f32)
    eng = ee.Plan(X, None, ls=0.6, min_points=60, nr_of_interpolation=27, small_field_points=37)
    monkeypatch.setenv("F3M_SIB_PASSES", "1")
    whole = eng.apply(b)
    monkeypatch.setenv("F3M_SIB_PASSES", str(parts))
    assert np.array_equal(whole, eng.apply(b))


def test_m2l_sibling_parents_longest_first(monkeypatch):
    """the sibling-group M2L may start the parents with the longest far rows first: the same sums, bit for bit"""
    rng = np.random.default_rng(8)
    X = rng.random((3000, 3), dtype=f32)
    b = rng.standard_normal((3000, 1)).astype(f32)
    eng = ee.Plan(X, None, ls=0.6, min_points=60, nr_of_interpolation=27, small_field_points=37)
    monkeypatch.setenv("F3M_SIB_ORDER", "0")
    plain = eng.apply(b)
    monkeypatch.setenv("F3M_SIB_ORDER", "1")
    assert np.array_equal(plain, eng.apply(b))


@pytest.mark.parametrize("P", [8, 64])
def test_m2l_sibling_nodes_shared_by_two_lanes(monkeypatch, P):
    """3-D sibling-group M2L: two lanes share the n0 x n1 nodes of a lane (full wavefronts); same sums as the
    one-lane form up to the order of two additions"""
    rng = np.random.default_rng(6)
    n, mp = (2500, 60) if P == 8 else (6000, 150)
    X = rng.random((n, 3), dtype=f32)
    b = rng.standard_normal((n, 1)).astype(f32)
    eng = ee.Plan(X, None, ls=0.6, min_points=mp, nr_of_interpolation=P, small_field_points=P + 10)
    assert any(eng.level_sizes(k)["nfar"] for k in range(1, eng.depth + 1))
    monkeypatch.setenv("F3M_M2L", "sibling")               # also at levels with few parents
    shared = eng.apply(b)
    monkeypatch.setenv("F3M_SIB_SPLIT", "0")
    single = eng.apply(b)
    assert 0 < rel_l2(shared, single) < 1e-6
    monkeypatch.setenv("F3M_M2L", "direct")
    assert rel_l2(shared, eng.apply(b)) < 3e-6


def test_mfma_near_field(oracle, monkeypatch):
    monkeypatch.setenv("F3M_NEAR", "mfma")
    rng = np.random.default_rng(5)
    for d, n in ((3, 520), (2, 400), (4, 450)):
        X = rng.random((n, d), dtype=f32)
        Y = (rng.random((n - 123, d)) * 1.1).astype(f32)
        b = rng.standard_normal((n - 123, 3 if d == 2 else 1)).astype(f32)   # 3 columns: the four-column kernel
        prm = dict(ls=0.4, min_points=50, nr_of_interpolation=8, small_field_points=30)
        eng = ee.Plan(X, Y, **prm)
        ora = oracle.Plan(X, Y, **prm)
        checked = 0
        for k in range(1, eng.depth + 1):
            sz = eng.level_sizes(k)
            for which in ("small", "keep"):
                if sz["n" + which] and (which == "small" or k == eng.depth):
                    assert rel_l2(eng.near_level(k, which, b), ora.near_level(k - 1, which, b)) < 1e-5
                    checked += 1
        assert checked > 0
        if d == 3:              # 3000 box pairs take the emulation half a minute per pass: the level check above is the pass
            continue
        got = eng.apply(b)
        assert rel_l2(got, ora.apply(b)) < 1e-5
        if b.shape[1] > 1:      # columns taken four at a time give the same bits as one at a time
            for col in range(b.shape[1]):
                assert np.array_equal(eng.apply(b[:, col:col + 1]), got[:, col:col + 1])


@pytest.mark.parametrize("name", ["uniform3", "normal2", "uniform1", "uniform4", "dups_faces"])
def test_symmetric_near_field(oracle, monkeypatch, name):
    """One tree, one column: the tiles of a pair of boxes are evaluated once and added in both directions, the second
    one through the wavefront's LDS block and as fixed-point sums.  (F3M_SPLIT_TARGET=1: one wavefront per work item on
    these tiny clouds, which the symmetric form needs.)  Against the oracle, against the plain form (close, and not the
    same bits: the symmetric kernel did run), and with a weight that is not finite (the kernel then adds floats)."""
    monkeypatch.setenv("F3M_NEAR", "mfma")
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    rng = np.random.default_rng(9)
    X, _ = _cloud(name, rng)
    X = X[:1500]
    b = rng.standard_normal((X.shape[0], 1)).astype(f32)
    prm = dict(ls=0.4, min_points=50, nr_of_interpolation=8, small_field_points=30)
    sym = ee.kmvm(X, None, b, **prm)
    assert rel_l2(sym, oracle.kmvm(X, None, b, **prm)) < 1e-5
    assert np.array_equal(ee.kmvm(X, None, b, **prm), sym)
    monkeypatch.setenv("F3M_NEAR_SYM", "0")
    plain = ee.kmvm(X, None, b, **prm)
    assert 0 < rel_l2(sym, plain) < 1e-6
    if name == "uniform3":
        b[7] = np.inf
        plain = ee.kmvm(X, None, b, **prm)
        monkeypatch.setenv("F3M_NEAR_SYM", "1")
        sym = ee.kmvm(X, None, b, **prm)
        assert not np.isfinite(sym[7]).any() and not np.isfinite(plain[7]).any()
        both = np.isfinite(sym[:, 0]) & np.isfinite(plain[:, 0])        # (the far field carries the weight to most targets)
        assert np.array_equal(np.isfinite(sym), np.isfinite(plain))
        assert not both.any() or rel_l2(sym[both], plain[both]) < 1e-5


def test_symmetric_near_field_five_dimensions(oracle, monkeypatch):
    """d = 5: the symmetric form goes with the factored exponent (the second direction carries the targets' factor into
    the sums and gets the sources' factor after the column sums)."""
    monkeypatch.setenv("F3M_NEAR", "mfma")
    monkeypatch.setenv("F3M_NEAR_FACT", "1")
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    rng = np.random.default_rng(13)
    X = rng.random((2200, 5), dtype=f32)
    b = rng.standard_normal((2200, 1)).astype(f32)
    prm = dict(ls=1.0, min_points=80, nr_of_interpolation=32, small_field_points=40)
    sym = ee.kmvm(X, None, b, **prm)
    assert rel_l2(sym, oracle.kmvm(X, None, b, **prm)) < 1e-5
    monkeypatch.setenv("F3M_NEAR_SYM", "0")
    assert 0 < rel_l2(sym, ee.kmvm(X, None, b, **prm)) < 1e-6


@pytest.mark.parametrize("form", ["0", "1"])
def test_mfma_near_field_five_dimensions(oracle, monkeypatch, form):
    """d = 5: two matrix instructions per tile in the plain form, one in the factored form (the weights carry
    exp2(-|y'|^2), the sum of a run of sources is multiplied by exp2(-|x''|^2)); one and three columns."""
    monkeypatch.setenv("F3M_NEAR", "mfma")
    monkeypatch.setenv("F3M_NEAR_FACT", form)
    rng = np.random.default_rng(5)
    n = 420
    X = rng.random((n, 5), dtype=f32)
    Y = (rng.random((n - 100, 5)) * 1.1).astype(f32)
    prm = dict(ls=0.7, min_points=40, nr_of_interpolation=32, small_field_points=30)
    ora = oracle.Plan(X, Y, **prm)
    for nc in (1, 3) if form == "1" else (1,):
        b = rng.standard_normal((n - 100, nc)).astype(f32)
        eng = ee.Plan(X, Y, **prm)
        assert eng.depth == 1 and eng.level_sizes(1)["nsmall"] == 1024
        if nc == 1:
            want = ora.near_level(0, "small", b)
            assert rel_l2(eng.near_level(1, "small", b), want) < 1e-5       # lists cut into slices (few work items)
            monkeypatch.setenv("F3M_SPLIT_TARGET", "1")                     # whole lists: runs of boxes, shared anchors
            eng2 = ee.Plan(X, Y, **prm)
            assert rel_l2(eng2.near_level(1, "small", b), want) < 1e-5
            monkeypatch.delenv("F3M_SPLIT_TARGET")
        else:           # the product goes through the four-column kernel
            assert rel_l2(eng.apply(b), ora.apply(b)) < 1e-5


def test_no_division_returns_exact_product(oracle):
    rng = np.random.default_rng(2)
    X = rng.random((200, 3), dtype=f32)
    b = rng.standard_normal((200, 1)).astype(f32)
    out = ee.kmvm(X, None, b, ls=0.5, min_points=1000)
    assert rel_l2(out, oracle.exact_f64(X, X, b, 0.5)) < 1e-5


def test_error_paths():
    rng = np.random.default_rng(2)
    X = rng.random((50, 3), dtype=f32)
    b = rng.standard_normal((50, 1)).astype(f32)
    from f3m_amd.capi import F3MError
    with pytest.raises(F3MError):
        ee.kmvm(X, None, b, ls=-1.0)
    with pytest.raises(F3MError):
        ee.kmvm(np.zeros((50, 11), f32), None, b)
    # all points identical: cannot be divided, exact product
    assert np.allclose(ee.kmvm(np.ones((50, 3), f32), None, b, min_points=10), b.sum(0), rtol=1e-5)


def test_emulation_refuses_exchange_in_divergent_branch(tmp_path):
    """A lane exchange that only some lanes of a wavefront reach (here: on the right of `&&`) reads switched-off lanes
    on the GPU.  The emulation tags every wave-wide operation with its source line and stops when the lanes of a
    wavefront meet at different ones; the same kernel with the exchange made by every lane runs through."""
    import os
    import subprocess
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpu_emu")
    exe = str(tmp_path / "divergent_exchange")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-DF3M_CPU_EMU", "-I", here, "-I",
                           os.path.join(here, "..", "..", "f3m_amd", "csrc"), "-w",
                           os.path.join(here, "divergent_exchange.cpp"), "-o", exe, "-lpthread"])
    good = subprocess.run([exe, "good"], capture_output=True, text=True)
    assert good.returncode == 0 and good.stdout.strip() == "32"
    bad = subprocess.run([exe, "bad"], capture_output=True, text=True)
    assert bad.returncode != 0 and "different wave-wide operations" in bad.stderr
