"""GPU parity tests: the gfx950 library, called through its C ABI, against the CPU oracle on the
same seeded inputs.  Box division and interaction lists are compared bit for bit; floating-point
stages with the tolerance written at each assert (north star: rel-L2 <= 1e-3 against an fp64 exact
product and no worse than 1.5x the oracle algorithm's own error)."""
import numpy as np
import pytest

from parity_checks import assert_plan_matches_oracle, canonical_box_of_point, expected_list_rows, rel_l2

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def eng():
    import torch
    assert torch.cuda.is_available(), "these tests need a GPU"
    from f3m_amd import engine
    engine._lib.get()          # fails loudly if the gfx950 library is not built
    return engine


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def clouds(name, rng):
    if name == "C1_uniform3":        # config 1: N=1e5 uniform, ls=1, 64 nodes, cutoff 1000
        return rng.random((100000, 3), dtype=f32), None, dict(ls=1.0)
    if name == "normal3":
        return rng.standard_normal((60000, 3)).astype(f32), None, dict(ls=1.0)
    if name == "clustered_xy":       # config 3 in miniature
        mu, sd = rng.random((50, 3)) * 10, 0.05 + 0.45 * rng.random((50, 3))
        X = np.concatenate([rng.normal(m, s, (1500, 3)) for m, s in zip(mu, sd)]).astype(f32)
        Y = (X.min(0) + (X.max(0) - X.min(0)) * rng.random((30000, 3))).astype(f32)
        return X, Y, dict(ls=0.5)
    if name == "uniform4":
        return rng.random((60000, 4), dtype=f32), None, dict(ls=1.0, nr_of_interpolation=81)
    if name == "uniform5":
        return rng.random((60000, 5), dtype=f32), None, dict(ls=1.0, nr_of_interpolation=32, min_points=100,
                                                              small_field_points=40)
    if name == "normal5":            # near lists on several levels in 5-D (the factored near-field form, operand
        # tables of listed boxes only, two columns at a time)
        return rng.standard_normal((60000, 5)).astype(f32), None, dict(ls=2.0, nr_of_interpolation=32, min_points=300,
                                                                        small_field_points=100)
    if name == "uniform5_243":       # config 4: 3^5 nodes per box; 390 points per box at depth 2, so pairs of boxes
        # there hold more than 2 * 243 points and are far wherever they are two or more boxes apart
        return rng.random((400000, 5), dtype=f32), None, dict(ls=1.0, nr_of_interpolation=243, min_points=1000,
                                                               small_field_points=300)
    if name in ("uniform3_ls0.1", "uniform3_ls10"):      # config 2 in miniature: lengthscales 0.1 and 10
        return rng.random((100000, 3), dtype=f32), None, dict(ls=float(name.split("ls")[1]))
    if name in ("normal3_ls0.1", "normal3_ls10"):
        return rng.standard_normal((60000, 3)).astype(f32), None, dict(ls=float(name.split("ls")[1]))
    if name == "uniform5_1024":      # 4^5 nodes: the siblings of a box do not fit one workgroup and are split in two
        return rng.random((1500000, 5), dtype=f32), None, dict(ls=1.5, nr_of_interpolation=1024, min_points=1000,
                                                                small_field_points=300)
    if name in ("uniform3_125", "uniform3_216"):     # the larger grids of the reference's own sweep (experiments/
        # experiments.py:47-49): 390 points per box at depth 3, far pairs at depths 2 and 3
        return rng.random((200000, 3), dtype=f32), None, dict(ls=1.0, nr_of_interpolation=int(name.split("_")[1]))
    if name == "uniform2":
        return rng.random((80000, 2), dtype=f32), None, dict(ls=0.2)
    if name == "uniform1":
        return rng.random((50000, 1), dtype=f32), None, dict(ls=0.05, nr_of_interpolation=8)
    if name == "lattice_faces_dups":
        g = (np.stack(np.meshgrid(*[np.arange(33)] * 3, indexing="ij"), -1).reshape(-1, 3) / 32.0).astype(f32)
        return np.concatenate([g, g[::-1], g[::2]]), None, dict(ls=0.3, min_points=200, small_field_points=100)
    if name == "uniform3_varcomp":   # the reference's FALKON experiments run with var_compression=True
        return rng.random((80000, 3), dtype=f32), None, dict(ls=3.0, var_compression=True, eff_var_limit=0.3,
                                                              min_points=500, small_field_points=300)
    raise KeyError(name)


NAMES = ["C1_uniform3", "normal3", "clustered_xy", "uniform4", "uniform5", "uniform5_243", "uniform2", "uniform1",
         "lattice_faces_dups", "uniform3_varcomp"]
# Clouds whose complete far field would keep the CPU oracle busy for minutes (far pairs x 243^2 kernel
# evaluations): the oracle computes the target rows of a few boxes only (same sums, restricted to those rows)
# and the GPU results are compared on them.
ROW_BOXES = {"uniform5_243": [0, 17, 333, 512, 800, 1023], "uniform3_125": [0, 7, 100, 255, 256, 300, 480, 511],
             "uniform3_216": [0, 7, 100, 255, 256, 300, 480, 511]}


def selected_rows(name, level):
    """rows of X that lie in the boxes ROW_BOXES[name] of the deepest level, or None for every row"""
    if name not in ROW_BOXES:
        return None
    return np.concatenate([level["permx"][level["offx"][bx]:level["offx"][bx + 1]] for bx in ROW_BOXES[name]])


@pytest.mark.parametrize("fixture_name", __import__("golden_fixtures").names())
def test_committed_oracle_fixtures(eng, fixture_name):
    """tests/golden/oracle_fixtures.npz: box division and lists bit for bit, product within tolerance,
    without running the oracle."""
    import golden_fixtures as gf
    print("case fixture", fixture_name, flush=True)
    fx = gf.load()
    X, Y, b, prm = gf.case(fx, fixture_name)
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    gf.assert_plan_matches_fixture(plan, plan.depth, fx, fixture_name)
    for k in range(1, plan.depth + 1):
        assert plan.list_rows(k) == expected_list_rows(plan.level(k)), (fixture_name, k)
    gf.assert_product_matches_fixture(plan.apply(dev(b)).cpu().numpy(), fx, fixture_name)
    gf.assert_product_matches_fixture(eng.kmvm(dev(X), None if Y is None else dev(Y), dev(b), **prm).cpu().numpy(), fx,
                                      fixture_name)


@pytest.mark.parametrize("fixture_name", __import__("golden_fixtures").names())
def test_near_field_source_runs_on_matrix_pipe(eng, monkeypatch, fixture_name):
    """The matrix-pipe near field with whole lists per wavefront (no slicing), where source boxes that
    follow each other under one parent cell are taken as one run.  The lattice fixture has targets whose
    -|x''|^2 is an exact tie between two f16 values: hi and lo of the split must come from one rounding."""
    import golden_fixtures as gf
    print("case fixture (matrix pipe, unsliced)", fixture_name, flush=True)
    monkeypatch.setenv("F3M_NEAR", "mfma")
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    fx = gf.load()
    X, Y, b, prm = gf.case(fx, fixture_name)
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    gf.assert_product_matches_fixture(plan.apply(dev(b)).cpu().numpy(), fx, fixture_name)


@pytest.mark.parametrize("fixture_name", __import__("golden_fixtures").names())
def test_near_field_all_vector_kernel_on_fixtures(eng, monkeypatch, fixture_name):
    """The all-vector near-field kernel (LDS-staged sources, fp32 throughout), which the library takes by
    itself only where boxes are large against the lengthscale, forced on every fixture."""
    import golden_fixtures as gf
    print("case fixture (all-vector near field)", fixture_name, flush=True)
    monkeypatch.setenv("F3M_NEAR", "valu")
    fx = gf.load()
    X, Y, b, prm = gf.case(fx, fixture_name)
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    gf.assert_product_matches_fixture(plan.apply(dev(b)).cpu().numpy(), fx, fixture_name)


@pytest.mark.parametrize("d,n,boxes", [(3, 40000, None), (5, 200000, [0, 100, 341, 682, 900, 1023])])
@pytest.mark.parametrize("side", ["below", "above"])
def test_near_field_kernel_switch_at_its_threshold(eng, oracle, monkeypatch, d, n, boxes, side):
    """The library sums near pairs on the matrix pipe (split-f16 operands) while 30 d (sc edge)^2 <= 1200,
    sc = sqrt(log2(e) / (2 ls^2)), and with the all-vector kernel beyond.  Lengthscales that put the boxes of
    the deepest level 1 % below and 1 % above that switch: the matrix-pipe kernel must stay within 3e-5 of
    the oracle's sums (the bound the switch is derived from) below it, the all-vector kernel within 1e-5 on
    both sides, and the library's own choice must be the matrix pipe below and the all-vector kernel above."""
    print("case near switch d=%d %s" % (d, side), flush=True)
    rng = np.random.default_rng(21)
    X = rng.random((n, d), dtype=f32)
    b = rng.standard_normal((n, 2)).astype(f32)
    prm = dict(min_points=1000, nr_of_interpolation=64 if d == 3 else 32)
    probe = eng.Plan(dev(X), None, ls=1.0, **prm)                       # the box edge does not depend on ls
    depth = probe.depth
    edge = float(probe.level_sizes(depth)["edge"])
    probe.close()
    s_edge = np.sqrt(1200.0 / (30.0 * d)) * (0.99 if side == "below" else 1.01)      # sc * edge aimed at
    ls = float(np.sqrt(np.log2(np.e) / 2.0) * edge / s_edge)
    plan = eng.Plan(dev(X), None, ls=ls, **prm)
    ora = oracle.Plan(X, None, ls=ls, **prm)
    assert plan.depth == depth and ora.nlevels == depth
    sc_edge = np.sqrt(float(ora.lcs) * np.log2(np.e)) * edge
    assert (30 * d * sc_edge ** 2 <= 1200) == (side == "below")
    L = ora.level(depth - 1)
    which = "small" if len(L["small"]) else "keep"
    rows = None if boxes is None else np.concatenate([L["permx"][L["offx"][bx]:L["offx"][bx + 1]] for bx in boxes])
    sel = slice(None) if rows is None else rows
    want = ora.near_level(depth - 1, which, b, rows=rows)[sel]
    assert np.abs(want).max() > 0
    auto = plan.near_level(depth, which, dev(b)).cpu().numpy()[sel]
    monkeypatch.setenv("F3M_NEAR", "mfma")
    mfma = plan.near_level(depth, which, dev(b)).cpu().numpy()[sel]
    monkeypatch.setenv("F3M_NEAR", "valu")
    valu = plan.near_level(depth, which, dev(b)).cpu().numpy()[sel]
    e_mfma, e_valu = rel_l2(mfma, want), rel_l2(valu, want)
    print("sc*edge %.4f  rel-L2 vs oracle: matrix pipe %.3e, all-vector %.3e" % (sc_edge, e_mfma, e_valu), flush=True)
    assert e_valu < 1e-5
    if side == "below":
        assert e_mfma < 3e-5
        assert np.array_equal(auto, mfma)
    else:
        assert np.array_equal(auto, valu)


@pytest.mark.parametrize("d,n,boxes", [(5, 200000, [0, 100, 341, 682, 900, 1023]), (10, 120000, [0, 341, 1023])])
@pytest.mark.parametrize("side", ["below", "above"])
def test_near_field_factored_form_at_its_threshold(eng, oracle, monkeypatch, d, n, boxes, side):
    """In 5 and 10 dimensions the matrix-pipe near field takes its factored form (exp2(-|x''|^2) exp2(2x''.y')
    exp2(-|y'|^2) b, one matrix instruction fewer per tile) while 10 d (sc edge)^2 <= 30, the plain form beyond.
    Lengthscales 1 % below and above that switch: both forms within 1e-5 of the oracle's sums on both sides, and the
    library's own choice (fixed when a level's operand table is built, hence one plan per setting) has the bits of the
    factored form below and of the plain form above."""
    print("case near factored d=%d %s" % (d, side), flush=True)
    rng = np.random.default_rng(22)
    X = rng.random((n, d), dtype=f32)
    b = rng.standard_normal((n, 2)).astype(f32)
    prm = dict(min_points=1000, nr_of_interpolation=32 if d == 5 else 64)
    probe = eng.Plan(dev(X), None, ls=1.0, **prm)
    depth = probe.depth
    edge = float(probe.level_sizes(depth)["edge"])
    probe.close()
    s_edge = np.sqrt(30.0 / (10.0 * d)) * (0.99 if side == "below" else 1.01)
    ls = float(np.sqrt(np.log2(np.e) / 2.0) * edge / s_edge)
    ora = oracle.Plan(X, None, ls=ls, **prm)
    assert ora.nlevels == depth
    sc_edge = np.sqrt(float(ora.lcs) * np.log2(np.e)) * edge
    assert (10 * d * sc_edge ** 2 <= 30) == (side == "below")
    L = ora.level(depth - 1)
    which = "small" if len(L["small"]) else "keep"
    rows = np.concatenate([L["permx"][L["offx"][bx]:L["offx"][bx + 1]] for bx in boxes])
    want = ora.near_level(depth - 1, which, b, rows=rows)[rows]
    assert np.abs(want).max() > 0
    got = {}
    for form in (None, "0", "1"):
        if form is None:
            monkeypatch.delenv("F3M_NEAR_FACT", raising=False)
        else:
            monkeypatch.setenv("F3M_NEAR_FACT", form)
        plan = eng.Plan(dev(X), None, ls=ls, **prm)
        got[form] = plan.near_level(depth, which, dev(b)).cpu().numpy()[rows]
        if form is None:
            # huge weights: the factored form sums exp2(2x''.y') b before the target's factor comes in; inside its
            # range that stays finite where every term of the plain form is
            scale = f32(2.0 ** 83)              # ~1e25, and a power of two: every sum scales without rounding
            big = plan.near_level(depth, which, dev(b * scale)).cpu().numpy()[rows]
            assert np.isfinite(big).all() and np.array_equal(big / scale, got[None])
        plan.close()
    e_plain, e_fact = rel_l2(got["0"], want), rel_l2(got["1"], want)
    print("sc*edge %.4f  rel-L2 vs oracle: plain %.3e, factored %.3e" % (sc_edge, e_plain, e_fact), flush=True)
    assert e_plain < 1e-5 and e_fact < 1e-5
    assert not np.array_equal(got["0"], got["1"])
    assert np.array_equal(got[None], got["1" if side == "below" else "0"])


@pytest.mark.parametrize("name", NAMES)
def test_box_division_and_lists_bit_exact(eng, oracle, name):
    print("case", name, flush=True)
    X, Y, prm = clouds(name, np.random.default_rng(100))
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    ora = oracle.Plan(X, Y, **prm)
    assert ora.nlevels >= 1
    assert_plan_matches_oracle(plan, ora)
    w = plan.work()
    assert w["near_pairs"] == ora.work_near_pairs and w["far_pairs"] == ora.work_far_pairs
    assert w["interp_points"] == ora.work_interp_pts
    M = X.shape[0] if Y is None else Y.shape[0]
    assert w["near_pairs"] + w["far_point_pairs"] == float(X.shape[0]) * M      # every pair exactly once


@pytest.mark.parametrize("name", ["normal3", "clustered_xy", "uniform4"])
def test_level_scans_one_by_one(eng, oracle, monkeypatch, name):
    """F3M_LEVEL_SCANS=separate: the scans of a level one after the other (the path of levels with more than
    2048 x 2048 boxes) instead of in one set of launches: same tree and lists, and the same row statistics."""
    print("case separate level scans", name, flush=True)
    monkeypatch.setenv("F3M_LEVEL_SCANS", "separate")
    X, Y, prm = clouds(name, np.random.default_rng(11))
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    ora = oracle.Plan(X, Y, **prm)
    assert_plan_matches_oracle(plan, ora)
    for k in range(1, plan.depth + 1):
        assert plan.list_rows(k) == expected_list_rows(ora.level(k - 1)), k


@pytest.mark.parametrize("name", ["normal3", "clustered_xy", "uniform5"])
def test_box_lookup_by_cell(eng, oracle, name):
    """The HBM key -> index table (reference: F3M_src/linearprobing.cu:18-87): the cell of every point,
    restated in numpy, must map to the box that holds the point; absent cells map to -1."""
    import torch
    from helpers import box_of_point, cell_coords
    print("case box lookup", name, flush=True)
    X, Y, prm = clouds(name, np.random.default_rng(7))
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    edge0, xmin, ymin = oracle.root(X, Y)
    for tree, pts, org in (("x", X, xmin), ("y", X if Y is None else Y, xmin if Y is None else ymin)):
        for k in range(1, plan.depth + 1):
            L = plan.level(k)
            cells = cell_coords(pts, org, edge0, k).astype(np.int32)
            got = plan.lookup_boxes(k, dev(cells), tree).cpu().numpy()
            assert np.array_equal(got, box_of_point(L, tree)), (tree, k)
            shifted = cells + (1 << k)                 # outside the grid: never a box
            assert (plan.lookup_boxes(k, dev(shifted), tree).cpu().numpy() == -1).all()
    nb = plan.level_sizes(plan.depth)["nbx"]
    side = 1 << plan.depth
    rnd = np.random.default_rng(8).integers(0, side, (20000, X.shape[1])).astype(np.int32)
    got = plan.lookup_boxes(plan.depth, dev(rnd), "x").cpu().numpy()
    occupied = {tuple(c) for c in cell_coords(X, xmin, edge0, plan.depth).tolist()}
    assert all((g >= 0) == (tuple(c) in occupied) for c, g in zip(rnd.tolist(), got.tolist()))
    assert got.max() < nb
    lib = eng._lib.get()
    for key, cap in ((1, 1 << 20), (0xFFFFFFFF, 1024), (123456789, 4096)):
        assert lib.f3m_hash_slot(key, cap) == oracle.hash_slot(key, cap)


@pytest.mark.parametrize("d", [1, 2, 3, 5, 10])
def test_exact_kernels(eng, oracle, d):
    print("case exact d=%d" % d, flush=True)
    rng = np.random.default_rng(d)
    X = rng.standard_normal((1500, d)).astype(f32)
    Y = rng.standard_normal((2300, d)).astype(f32)
    b = rng.standard_normal((2300, 3)).astype(f32)
    ls = 0.9 * np.sqrt(d)
    ref = oracle.exact_f64(X, Y, b, ls)
    assert rel_l2(eng.exact_f32(dev(X), dev(Y), dev(b), ls).cpu().numpy(), ref) < 1e-5
    assert rel_l2(eng.exact_f64(dev(X.astype(np.float64)), dev(Y.astype(np.float64)), dev(b.astype(np.float64)), ls).cpu().numpy(), ref) < 1e-12
    assert rel_l2(eng.exact_grad_f32(dev(X), dev(Y), dev(b), ls).cpu().numpy(), oracle.exact_grad_f32(X, Y, b, ls)) < 1e-5


@pytest.mark.parametrize("name", ["normal3", "clustered_xy", "uniform4", "uniform2", "uniform5", "uniform5_243", "normal5",
                                  "uniform3_varcomp", "uniform3_125", "uniform3_216"])
def test_stages_against_oracle(eng, oracle, name):
    print("case stages", name, flush=True)
    rng = np.random.default_rng(7)
    X, Y, prm = clouds(name, rng)
    if name not in ("uniform5", "uniform5_243", "uniform3_125", "uniform3_216"):   # these need their points to have far pairs
        X = X[:30000]
        Y = None if Y is None else Y[:12000]
    M = X.shape[0] if Y is None else Y.shape[0]
    b = rng.standard_normal((M, 2)).astype(f32)
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    ora = oracle.Plan(X, Y, **prm)
    assert_plan_matches_oracle(plan, ora)
    rows = selected_rows(name, ora.level(ora.nlevels - 1))
    sel = slice(None) if rows is None else rows
    far_levels = 0
    for k in range(1, plan.depth + 1):
        sz = plan.level_sizes(k)
        if sz["nsmall"]:
            got = plan.near_level(k, "small", dev(b)).cpu().numpy()
            assert rel_l2(got[sel], ora.near_level(k - 1, "small", b, rows=rows)[sel]) < 1e-5   # fp32 summation order only
        if sz["nfar"]:
            far_levels += 1
            out, mom, loc = plan.far_level(k, dev(b), want_expansions=True)
            o_out, o_mom, o_loc = ora.far_level(k - 1, b, rows=rows)
            loc = loc.cpu().numpy()
            o_loc = np.moveaxis(o_loc, 2, 0)
            if rows is not None:                         # local expansions of the boxes that hold a selected row
                L = ora.level(k - 1)
                boxes = np.unique(canonical_box_of_point(L, "x")[rows])
                assert np.abs(o_loc[:, boxes]).max() > 0
                loc, o_loc = loc[:, boxes], o_loc[:, boxes]
            assert rel_l2(mom.cpu().numpy(), np.moveaxis(o_mom, 2, 0)) < 1e-4     # P2M
            assert rel_l2(loc, o_loc) < 1e-4                                      # M2L
            assert rel_l2(out.cpu().numpy()[sel], o_out[sel]) < 1e-4              # L2P
    assert far_levels >= (2 if name in ("uniform5_243", "uniform3_125", "uniform3_216") else 1)
    if plan.level_sizes(plan.depth)["nkeep"]:
        got = plan.near_level(plan.depth, "keep", dev(b)).cpu().numpy()
        assert rel_l2(got[sel], ora.near_level(plan.depth - 1, "keep", b, rows=rows)[sel]) < 1e-5
    got = plan.apply(dev(b)).cpu().numpy()
    assert rel_l2(got[sel], ora.apply(b, rows=rows)[sel]) < 1e-5


@pytest.mark.parametrize("d,n,prm", [
    (6, 60000, dict(ls=1.0, nr_of_interpolation=64, min_points=1000, small_field_points=200)),
    (8, 100000, dict(ls=1.5, nr_of_interpolation=256, min_points=1000, small_field_points=300)),
    (10, 120000, dict(ls=2.0, nr_of_interpolation=64, min_points=1000, small_field_points=100)),
])
def test_six_to_ten_dimensions_against_oracle(eng, oracle, d, n, prm):
    """The reference exports its operator for 1 to 10 dimensions (F3M_src/pybinder_setup.cu:17-36).  Beyond five
    the engine runs its general kernels (any tensor grid: 2^6, 2^8 and 2^6 x 1^4 nodes here; two matrix instructions
    per near-field tile): box division and lists bit for bit, every stage and the product against the oracle on the
    rows of eight boxes (the oracle's complete M2L would take minutes: up to 868 352 far pairs of 64^2 to 256^2 terms)."""
    print("case d=%d" % d, flush=True)
    rng = np.random.default_rng(d)
    X = rng.random((n, d), dtype=f32)
    b = rng.standard_normal((n, 1)).astype(f32)
    plan = eng.Plan(dev(X), None, **prm)
    ora = oracle.Plan(X, None, **prm)
    assert_plan_matches_oracle(plan, ora)
    L = ora.level(ora.nlevels - 1)
    nb = len(L["offx"]) - 1
    boxes = np.unique(np.linspace(0, nb - 1, 8).astype(int))
    rows = np.concatenate([L["permx"][L["offx"][bx]:L["offx"][bx + 1]] for bx in boxes])
    far_levels = 0
    for k in range(1, plan.depth + 1):
        sz = plan.level_sizes(k)
        if sz["nsmall"]:
            got = plan.near_level(k, "small", dev(b)).cpu().numpy()
            assert rel_l2(got[rows], ora.near_level(k - 1, "small", b, rows=rows)[rows]) < 1e-5
        if sz["nfar"]:
            far_levels += 1
            out, mom, loc = plan.far_level(k, dev(b), want_expansions=True)
            o_out, o_mom, o_loc = ora.far_level(k - 1, b, rows=rows)
            lvl = ora.level(k - 1)
            mine = np.unique(canonical_box_of_point(lvl, "x")[rows])
            assert rel_l2(mom.cpu().numpy(), np.moveaxis(o_mom, 2, 0)) < 1e-4
            assert rel_l2(loc.cpu().numpy()[:, mine], np.moveaxis(o_loc, 2, 0)[:, mine]) < 1e-4
            assert rel_l2(out.cpu().numpy()[rows], o_out[rows]) < 1e-4
    assert far_levels >= 1
    if plan.level_sizes(plan.depth)["nkeep"]:
        got = plan.near_level(plan.depth, "keep", dev(b)).cpu().numpy()
        assert rel_l2(got[rows], ora.near_level(plan.depth - 1, "keep", b, rows=rows)[rows]) < 1e-5
    got = plan.apply(dev(b)).cpu().numpy()
    want = ora.apply(b, rows=rows)
    assert rel_l2(got[rows], want[rows]) < 1e-5
    exact = oracle.exact_f64(X[rows], X, b, prm["ls"])
    assert rel_l2(got[rows], exact) <= 1.5 * rel_l2(want[rows], exact) + 1e-7


def random_cloud(rng, kind, n, d):
    if kind == "uniform":
        return rng.random((n, d), dtype=f32)
    if kind == "normal":
        return rng.standard_normal((n, d)).astype(f32)
    if kind == "clustered":
        mu, sd = rng.random((8, d)) * 4, 0.02 + 0.3 * rng.random((8, d))
        return np.concatenate([rng.normal(m, s, (n // 8 + 1, d)) for m, s in zip(mu, sd)])[:n].astype(f32)
    if kind == "lattice":            # points on box faces at every level, and duplicates
        m = max(2, int(round(n ** (1.0 / d))))
        g = (np.stack(np.meshgrid(*[np.arange(m)] * d, indexing="ij"), -1).reshape(-1, d) / f32(m - 1)).astype(f32)
        return np.concatenate([g, g[::3]])[:max(n, 10)]
    if kind == "line":               # a noisy segment: deep, thin trees
        return (rng.random((n, 1)) * rng.standard_normal((1, d)) + 1e-3 * rng.standard_normal((n, d))).astype(f32)
    raise KeyError(kind)


def random_configuration(case):
    """One draw of (X, Y, b, parameters): dimension 1-6, five kinds of cloud, one tree or two, lengthscale 0.05-20,
    node counts that are and are not full tensor grids, both cutoffs, variance compression, 1-5 columns."""
    rng = np.random.default_rng(1000 + case)
    d = int(rng.choice([1, 2, 3, 3, 3, 4, 5, 6]))
    kind = str(rng.choice(["uniform", "normal", "clustered", "lattice", "line"]))
    n = int(rng.integers(500, 40000 if d <= 3 else 25000))
    two = bool(rng.random() < 0.35)
    m = int(rng.integers(300, 30000)) if two else n
    ls = float(np.exp(rng.uniform(np.log(0.05), np.log(20))))
    nodes = int(rng.choice({1: [4, 8, 16], 2: [16, 36, 64, 100], 3: [8, 27, 64, 64, 125], 4: [16, 81, 256], 5: [32, 243],
                            6: [64, 729]}[d]))
    prm = dict(ls=ls, nr_of_interpolation=nodes, min_points=int(rng.choice([50, 200, 500, 1000, 2500])),
               small_field_points=int(rng.choice([20, 100, 300, 1000])))
    varc = bool(rng.random() < 0.25)
    c = int(rng.choice([1, 1, 2, 3, 5]))
    if varc:
        prm.update(var_compression=True, eff_var_limit=float(rng.choice([0.1, 0.3, 1.0])))
    X = random_cloud(rng, kind, n, d)
    Y = random_cloud(rng, str(rng.choice(["uniform", "normal", "clustered"])), m, d) if two else None
    if Y is not None and rng.random() < 0.5:      # sources spread over the targets' region
        Y = (X.min(0) + (X.max(0) - X.min(0)) * rng.random((m, d))).astype(f32)
    b = rng.standard_normal((X.shape[0] if Y is None else Y.shape[0], c)).astype(f32)
    return X, Y, b, prm, kind


# 32 of 540 draws that were run once in the same way (all of them agreed); the seeds are kept so that a failure names
# its case.
@pytest.mark.parametrize("case", [0, 3, 7, 11, 18, 20, 25, 28, 31, 34, 37, 52, 68, 77, 91, 104, 120, 133, 149, 162, 176, 188,
                                  203, 240, 271, 305, 333, 364, 402, 447, 489, 530])
def test_random_configurations_against_oracle(eng, oracle, case):
    """Box division and lists bit for bit, the product no worse than 1.5x the oracle's error against the fp64 exact
    product, the one-shot call with the bits of plan + apply, and for two trees the transposed product against the
    oracle's product of the swapped clouds."""
    X, Y, b, prm, kind = random_configuration(case)
    print("case random %d: d=%d %s n=%d m=%s c=%d %s" % (case, X.shape[1], kind, X.shape[0],
                                                         None if Y is None else Y.shape[0], b.shape[1], prm), flush=True)
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    ora = oracle.Plan(X, Y, **prm)
    assert_plan_matches_oracle(plan, ora)
    got = plan.apply(dev(b)).cpu().numpy()
    want = ora.apply(b)
    exact = oracle.exact_f64(X, X if Y is None else Y, b, prm["ls"])
    assert np.isfinite(got).all()
    if np.linalg.norm(exact) > 0:
        assert rel_l2(got, exact) <= 1.5 * rel_l2(want, exact) + 3e-6, (rel_l2(got, exact), rel_l2(want, exact))
    else:                                          # clouds many lengthscales apart: every term underflows
        assert not got.any() and not want.any()
    one = eng.kmvm(dev(X), None if Y is None else dev(Y), dev(b), **prm).cpu().numpy()
    assert np.array_equal(one, got)
    if Y is not None:
        u = np.random.default_rng(case).standard_normal((X.shape[0], 1)).astype(f32)
        got_t = plan.apply_transpose(dev(u)).cpu().numpy()
        exact_t = oracle.exact_f64(Y, X, u, prm["ls"])
        want_t = oracle.Plan(Y, X, **prm).apply(u)
        if np.linalg.norm(exact_t) > 0:
            assert rel_l2(got_t, exact_t) <= 1.5 * rel_l2(want_t, exact_t) + 3e-6
        else:
            assert not got_t.any()
    plan.close()


# draws of the same generator with one tree (every dimension up to five, every kind of cloud, variance compression)
@pytest.mark.parametrize("case", [0, 2, 3, 7, 10, 13, 16, 19, 22, 28, 33, 42, 48, 50, 55, 62, 72])
def test_random_configurations_symmetric_near_field(eng, oracle, monkeypatch, case):
    """The symmetric near field (one column; F3M_SPLIT_TARGET=1 keeps one wavefront per work item on these small clouds)
    on random one-tree configurations: no worse than 1.5x the oracle's error against the fp64 exact product, within
    1e-5 of the one-directional form, the same bits from the one-shot call and from a plan applied twice."""
    X, Y, b, prm, kind = random_configuration(case)
    assert Y is None
    b = np.ascontiguousarray(b[:, :1])
    print("case random symmetric %d: d=%d %s n=%d %s" % (case, X.shape[1], kind, X.shape[0], prm), flush=True)
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    Xd, bd = dev(X), dev(b)
    plan = eng.Plan(Xd, None, **prm)
    got = plan.apply(bd).cpu().numpy()
    assert np.array_equal(plan.apply(bd).cpu().numpy(), got)
    plan.close()
    assert np.array_equal(eng.kmvm(Xd, None, bd, **prm).cpu().numpy(), got)
    want = oracle.kmvm(X, None, b, **prm)
    exact = oracle.exact_f64(X, X, b, prm["ls"])
    assert np.isfinite(got).all()
    assert rel_l2(got, exact) <= 1.5 * rel_l2(want, exact) + 3e-6, (rel_l2(got, exact), rel_l2(want, exact))
    monkeypatch.setenv("F3M_NEAR_SYM", "0")
    # (another order of the same fp32 sums: up to 3e-6 where the lengthscale spans the cloud and the sums cancel)
    assert rel_l2(got, eng.kmvm(Xd, None, bd, **prm).cpu().numpy()) < 1e-5


PRODUCT_NAMES = ["C1_uniform3", "normal3", "clustered_xy", "uniform4", "uniform5_243", "uniform3_ls0.1", "uniform3_ls10",
                 "normal3_ls0.1", "normal3_ls10"]
# Where the reference algorithm itself (the oracle, same nodes and lengthscale) misses the 1e-3 of the
# north star, the engine cannot meet it either; these are the clouds where that is expected, with the
# oracle's error as measured (the engine must still stay within 1.5x of it).
ORACLE_ABOVE_1E3 = {"uniform3_ls0.1"}


@pytest.mark.parametrize("name", PRODUCT_NAMES)
def test_product_error_vs_fp64_exact(eng, oracle, name):
    print("case product", name, flush=True)
    rng = np.random.default_rng(9)
    X, Y, prm = clouds(name, rng)
    M = X.shape[0] if Y is None else Y.shape[0]
    b = rng.standard_normal((M, 1)).astype(f32)
    Xd, Yd, bd = dev(X), (None if Y is None else dev(Y)), dev(b)
    got = eng.kmvm(Xd, Yd, bd, **prm).cpu().numpy()
    Ys = X if Y is None else Y
    exact = eng.exact_f64(dev(X.astype(np.float64)), dev(Ys.astype(np.float64)), dev(b.astype(np.float64)), prm["ls"]).cpu().numpy()
    ora = oracle.Plan(X, Y, **prm)
    rows = selected_rows(name, ora.level(ora.nlevels - 1))
    sel = slice(None) if rows is None else rows
    err = rel_l2(got, exact)
    err_sel = rel_l2(got[sel], exact[sel])
    err_oracle = rel_l2(ora.apply(b, rows=rows)[sel], exact[sel])
    print("rel-L2 engine %.3e (compared rows %.3e) oracle %.3e" % (err, err_sel, err_oracle), flush=True)
    assert err_sel <= 1.5 * err_oracle + 1e-7            # no worse than 1.5x the reference algorithm
    # north-star tolerance 1e-3 against the fp64 product, on every row
    if name in ORACLE_ABOVE_1E3:
        assert err_oracle > 1e-3 / 1.5 and err <= 1.5 * err_oracle, (err, err_oracle)
    else:
        assert err <= 1e-3, (err, err_oracle)


@pytest.mark.parametrize("name", ["uniform4", "uniform5", "uniform5_243", "uniform5_1024", "uniform3_varcomp", "uniform3_125",
                                  "uniform3_216"])
def test_m2l_forms_agree(eng, monkeypatch, name):
    """Sibling-group separable M2L (default for one tree, d >= 3) against the per-box separable form
    and the direct form of the reference (F3M_src/1_d_conv.cu:741-817): same sums up to rounding."""
    print("case m2l forms", name, flush=True)
    rng = np.random.default_rng(14)
    X, Y, prm = clouds(name, rng)
    b = rng.standard_normal((X.shape[0], 1)).astype(f32)
    plan = eng.Plan(dev(X), None, **prm)
    assert sum(plan.level_sizes(k)["nfar"] for k in range(1, plan.depth + 1)) > 0
    grouped = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_M2L", "separable")
    per_box = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_M2L", "direct")
    direct = plan.apply(dev(b)).cpu().numpy()
    assert rel_l2(grouped, per_box) < 2e-6
    # the direct form evaluates exp per node pair in fp32 (243 x 243 terms per far pair at 3^5 nodes, 1024 x 1024 at 4^5,
    # over the ~900 far boxes of a box in five dimensions), the separable tables are rounded once from fp64
    assert rel_l2(grouped, direct) < (2e-5 if name in ("uniform5_243", "uniform5_1024") else 5e-6)
    if name in ("uniform4", "uniform5_243"):
        # 3^4 and 3^5 grids: the cells that every child of a parent lists summed once per combination of sibling bits
        # (m2l_shared_kernel, which the library takes by itself in 4-D beside the near field), the rest by the
        # sibling-group kernel; against the sibling-group kernel alone
        monkeypatch.delenv("F3M_M2L")
        monkeypatch.setenv("F3M_M2L_SHARED", "1")
        shared = plan.apply(dev(b)).cpu().numpy()
        monkeypatch.setenv("F3M_M2L_SHARED", "0")
        alone = plan.apply(dev(b)).cpu().numpy()
        assert 0 < rel_l2(shared, alone) < 2e-6
        assert rel_l2(shared, direct) < (2e-5 if name == "uniform5_243" else 5e-6)


@pytest.mark.parametrize("name,parts", [("C1_uniform3", 2), ("C1_uniform3", 3), ("uniform4", 6), ("uniform5_243", 2)])
def test_m2l_sibling_table_in_parts(eng, monkeypatch, name, parts):
    """The sibling-group M2L can fill and walk its table of far cells in parts (for tables that do not fit
    LDS whole).  The walking order is the same, so the sums are the same bit for bit."""
    print("case m2l table parts", name, parts, flush=True)
    rng = np.random.default_rng(15)
    X, Y, prm = clouds(name, rng)
    b = rng.standard_normal((X.shape[0], 1)).astype(f32)
    plan = eng.Plan(dev(X), None, **prm)
    default = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_SIB_PASSES", str(parts))
    assert np.array_equal(default, plan.apply(dev(b)).cpu().numpy())


@pytest.mark.parametrize("name", ["C1_uniform3", "uniform4", "uniform5_243"])
def test_m2l_sibling_parents_longest_first(eng, monkeypatch, name):
    """The sibling-group M2L may start the parents with the longest far rows first (default in d >= 4 when
    there are few parents): the same sums, bit for bit."""
    print("case m2l parent order", name, flush=True)
    rng = np.random.default_rng(17)
    X, Y, prm = clouds(name, rng)
    b = rng.standard_normal((X.shape[0], 1)).astype(f32)
    plan = eng.Plan(dev(X), None, **prm)
    monkeypatch.setenv("F3M_SIB_ORDER", "0")
    plain = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_SIB_ORDER", "1")
    assert np.array_equal(plain, plan.apply(dev(b)).cpu().numpy())


def test_plan_with_stream_wait_instead_of_watching_pinned_memory(eng, oracle, monkeypatch):
    """The host normally watches a sequence number in pinned memory for the per-level results; with the
    spin limit at zero it takes the fallback, a stream wait.  Same plan either way."""
    print("case spin limit 0", flush=True)
    rng = np.random.default_rng(19)
    X, Y, prm = clouds("clustered_xy", rng)
    monkeypatch.setenv("F3M_SPIN_LIMIT_MS", "0")
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    assert_plan_matches_oracle(plan, oracle.Plan(X, Y, **prm))


def test_near_field_longest_lists_first(eng, monkeypatch):
    """The matrix-pipe near field may take the boxes with the longest lists first (default from five
    dimensions on): the same sums for every target, bit for bit."""
    print("case near order", flush=True)
    rng = np.random.default_rng(18)
    X = rng.random((3_000_000, 3), dtype=f32)
    b = rng.standard_normal((3_000_000, 1)).astype(f32)
    plan = eng.Plan(dev(X), None, ls=1.0, min_points=200)              # depth 5, ~92 points per box: 32768 work items
    monkeypatch.setenv("F3M_NEAR", "mfma")
    monkeypatch.setenv("F3M_NEAR_ORDER", "0")
    plain = plan.near_level(plan.depth, "small", dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_NEAR_ORDER", "1")
    assert plan.list_rows(plan.depth)[2] >= 16384                      # not sliced: the order applies
    assert np.array_equal(plain, plan.near_level(plan.depth, "small", dev(b)).cpu().numpy())


@pytest.mark.parametrize("nodes", [8, 64])
def test_m2l_sibling_nodes_shared_by_two_lanes(eng, monkeypatch, nodes):
    """3-D sibling-group M2L with two lanes per n0 x n1 node set (default) against one lane per set and
    against the direct form of the reference (F3M_src/1_d_conv.cu:741-817)."""
    print("case m2l shared nodes", nodes, flush=True)
    rng = np.random.default_rng(16)
    X = rng.random((400000, 3), dtype=f32)
    b = rng.standard_normal((400000, 1)).astype(f32)
    plan = eng.Plan(dev(X), None, ls=1.0, nr_of_interpolation=nodes, min_points=150, small_field_points=100)
    assert plan.depth == 4 and plan.level_sizes(4)["nfar"] > 0     # 512 parents at the deepest level
    shared = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_SIB_SPLIT", "0")
    single = plan.apply(dev(b)).cpu().numpy()
    assert 0 < rel_l2(shared, single) < 1e-6
    monkeypatch.setenv("F3M_M2L", "direct")
    assert rel_l2(shared, plan.apply(dev(b)).cpu().numpy()) < 5e-6


def test_m2l_children_of_parent_pairs_kept_on_the_far_threshold(eng, monkeypatch):
    """A parent pair two cells apart along one axis is exactly 2 edges away; fp32 rounding of the centres
    decides whether the reference's predicate (F3M_src/1_d_conv.cu:936-941) calls it far.  Where it is
    kept, its children are far pairs with cell offsets beyond the usual 6^d block; the sibling-group M2L
    handles them through a table of their own."""
    rng = np.random.default_rng(0)
    sc, sh = rng.random() * 5 + 0.1, rng.standard_normal() * 3
    X = (rng.random((45000, 3)) * sc + sh).astype(f32)
    b = rng.standard_normal((45000, 1)).astype(f32)
    plan = eng.Plan(dev(X), None, ls=0.6 * sc, min_points=12, nr_of_interpolation=8, small_field_points=4)
    beyond = 0
    for k in range(3, plan.depth + 1):
        L = plan.level(k)
        cells = np.rint((L["cx"] - X.min(0)) / float(L["edge"]) - 0.5).astype(int)
        if len(L["far"]):
            u = cells[L["far"][:, 1]] - 2 * (cells[L["far"][:, 0]] >> 1)
            beyond += int(((u < -2) | (u > 3)).any(1).sum())
    assert beyond > 0                                  # the case is present in this cloud
    grouped = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_M2L", "separable")
    per_box = plan.apply(dev(b)).cpu().numpy()
    assert 0 < rel_l2(grouped, per_box) < 2e-6


@pytest.mark.parametrize("name", ["C1_uniform3", "normal3", "clustered_xy", "uniform5", "uniform3_varcomp", "uniform3_125",
                                  "uniform3_216", "uniform4", "uniform5_243"])
def test_far_sweeps_match_per_level_interpolation(eng, monkeypatch, name):
    """Default: points interpolated once, moments and local expansions moved between levels.
    F3M_FAR=levels: every level interpolated from the points like the reference
    (F3M_src/n_tree.cu:489-593).  The same sums up to fp32 rounding."""
    print("case far sweeps", name, flush=True)
    rng = np.random.default_rng(13)
    X, Y, prm = clouds(name, rng)
    M = X.shape[0] if Y is None else Y.shape[0]
    b = rng.standard_normal((M, 1)).astype(f32)
    plan = eng.Plan(dev(X), None if Y is None else dev(Y), **prm)
    sweeps = plan.apply(dev(b)).cpu().numpy()
    monkeypatch.setenv("F3M_FAR", "levels")
    per_level = plan.apply(dev(b)).cpu().numpy()
    assert rel_l2(sweeps, per_level) < 5e-6


@pytest.mark.parametrize("name", ["clustered_xy", "falkon_shape"])
def test_transposed_product_on_the_same_plan(eng, oracle, name):
    """K(X,Y)^T u from the plan of (X, Y) -- trees swapped, every list read from its Y boxes -- against a second
    plan of (Y, X) (the same lists, kernels and order: the same bits) and against the oracle's product of
    (Y, X).  Reference: FFM.chunk_forward_transpose, experiments/FFM_classes.py:54-61."""
    print("case transposed", name, flush=True)
    rng = np.random.default_rng(24)
    if name == "falkon_shape":           # many targets against few centres, the kernel wrapper's tree parameters
        X = (rng.random((30000, 3)) * 2 - 1).astype(f32)
        Y = X[rng.choice(30000, 400, replace=False)].copy()
        prm = dict(ls=0.5, min_points=64, nr_of_interpolation=64, small_field_points=64, var_compression=True,
                   eff_var_limit=0.3)
    else:
        X, Y, prm = clouds(name, rng)
    u = rng.standard_normal((X.shape[0], 3)).astype(f32)
    fwd, bwd = eng.Plan(dev(X), dev(Y), **prm), eng.Plan(dev(Y), dev(X), **prm)
    assert fwd.depth == bwd.depth >= 1
    got = fwd.apply_transpose(dev(u)).cpu().numpy()
    assert got.shape == (Y.shape[0], 3)
    assert np.array_equal(got, bwd.apply(dev(u)).cpu().numpy())
    assert rel_l2(got, oracle.kmvm(Y, X, u, **prm)) < 1e-5
    exact = oracle.exact_f64(Y, X, u, prm["ls"])
    assert rel_l2(got, exact) <= 1.5 * rel_l2(oracle.kmvm(Y, X, u, **prm), exact) + 1e-6
    # the forward product of the same plan is untouched by the transposed lists
    b = rng.standard_normal((Y.shape[0], 1)).astype(f32)
    assert np.array_equal(fwd.apply(dev(b)).cpu().numpy(), eng.kmvm(dev(X), dev(Y), dev(b), **prm).cpu().numpy())
    # no division at all: the exact product, transposed
    small = eng.Plan(dev(X[:500]), dev(Y[:300]), ls=0.5)
    assert small.depth == 0
    assert rel_l2(small.apply_transpose(dev(u[:500])).cpu().numpy(), oracle.exact_f64(Y[:300], X[:500], u[:500], 0.5)) < 1e-5


def test_repeated_products_have_the_same_bits(eng):
    """One-shot products and plan products of clouds of very different sizes, interleaved and repeated: every
    repetition must give the bits of the first.  The library queues work on two streams and recycles its device
    buffers between them; a buffer handed out while a kernel of the other stream still uses it would show up here
    (on small clouds every cached buffer fits every request)."""
    import golden_fixtures as gf
    print("case repeated products", flush=True)
    fx = gf.load()
    rng = np.random.default_rng(41)
    cases = []
    for name in ("d2_normal", "d3_two_trees", "d5_slab_243nodes_far"):
        X, Y, b, prm = gf.case(fx, name)
        cases.append((dev(X), None if Y is None else dev(Y), dev(b), prm))
    Xm = rng.random((200000, 3), dtype=f32)
    cases.append((dev(Xm), None, dev(rng.standard_normal((200000, 3)).astype(f32)), dict(ls=0.3)))
    Xa, Ya = rng.standard_normal((50000, 3)).astype(f32), rng.random((3000, 3), dtype=f32)
    cases.append((dev(Xa), dev(Ya), dev(rng.standard_normal((3000, 1)).astype(f32)), dict(ls=0.5, min_points=200)))
    first = [eng.kmvm(X, Y, b, **prm).cpu().numpy() for X, Y, b, prm in cases]
    plans = [eng.Plan(X, Y, **prm) for X, Y, b, prm in cases]
    for rep in range(6):
        for i, (X, Y, b, prm) in enumerate(cases):
            assert np.array_equal(eng.kmvm(X, Y, b, **prm).cpu().numpy(), first[i]), (rep, i, "one-shot")
            assert np.array_equal(plans[i].apply(b).cpu().numpy(), first[i]), (rep, i, "plan")


@pytest.mark.parametrize("name", ["C1_uniform3", "normal3", "clustered_xy", "uniform5_243"])
def test_one_stream_and_two_streams_give_the_same_bits(eng, monkeypatch, name):
    """The far field runs on a second stream beside the near field, and on clouds with near lists on several levels
    the tables of the shallower levels' lists are built there while the deepest level's lists are summed.  With
    F3M_OVERLAP=0 everything is queued on the caller's stream.  The launches that add to a target come in the same
    order either way (deepest level first), and near and far sums meet in one addition: the bits must not depend on the
    mode, for a one-shot product and for a kept plan, with one and three columns."""
    print("case one stream / two streams", name, flush=True)
    rng = np.random.default_rng(31)
    X, Y, prm = clouds(name, rng)
    M = X.shape[0] if Y is None else Y.shape[0]
    Xd, Yd = dev(X), None if Y is None else dev(Y)
    for c in (1, 3):
        b = dev(rng.standard_normal((M, c)).astype(f32))
        two = eng.kmvm(Xd, Yd, b, **prm).cpu().numpy()
        plan = eng.Plan(Xd, Yd, **prm)
        lists = sum(1 for k in range(1, plan.depth + 1) for w in ("nsmall", "nkeep")
                    if plan.level_sizes(k)[w] and (w == "nsmall" or k == plan.depth))
        if name == "normal3":
            assert lists >= 2                      # the case the order of launches matters for
        assert np.array_equal(plan.apply(b).cpu().numpy(), two)
        plan.close()
        monkeypatch.setenv("F3M_OVERLAP", "0")
        one = eng.kmvm(Xd, Yd, b, **prm).cpu().numpy()
        plan = eng.Plan(Xd, Yd, **prm)
        one_plan = plan.apply(b).cpu().numpy()
        plan.close()
        monkeypatch.delenv("F3M_OVERLAP")
        assert np.array_equal(one, two) and np.array_equal(one_plan, two)


@pytest.mark.parametrize("name", ["C1_uniform3", "normal3", "uniform2", "uniform1", "uniform4", "uniform5", "normal5",
                                  "lattice_faces_dups", "uniform3_varcomp"])
def test_symmetric_near_field_against_oracle(eng, oracle, monkeypatch, name):
    """One tree and one column: the near field evaluates the tiles of a pair of boxes once and adds them in both
    directions (half the exponentials), the second direction as fixed-point sums.  On these small clouds the lists
    would be cut into slices, which take the plain form; F3M_SPLIT_TARGET=1 keeps one wavefront per work item, so the
    symmetric kernel runs.  Against the oracle to 1e-5 level by level and for the product; against the plain form to
    1e-6 (and not the same bits: the symmetric kernel did run); the same bits when repeated."""
    print("case symmetric near field", name, flush=True)
    rng = np.random.default_rng(77)
    X, Y, prm = clouds(name, rng)
    assert Y is None
    b = rng.standard_normal((X.shape[0], 1)).astype(f32)
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    Xd, bd = dev(X), dev(b)
    sym = eng.kmvm(Xd, None, bd, **prm).cpu().numpy()
    ora = oracle.Plan(X, None, **prm)
    assert rel_l2(sym, ora.apply(b)) < 1e-5
    plan = eng.Plan(Xd, None, **prm)
    for rep in range(3):
        assert np.array_equal(plan.apply(bd).cpu().numpy(), sym), rep
        assert np.array_equal(eng.kmvm(Xd, None, bd, **prm).cpu().numpy(), sym), rep
    plan.close()
    if name != "uniform4":      # (5-D takes the factored exponent; on the 3^4 grid the far field shares M2L sums between siblings only beside a near field:
        # other rounding of the far field in one-stream mode, whatever the near field's form)
        monkeypatch.setenv("F3M_OVERLAP", "0")
        assert np.array_equal(eng.kmvm(Xd, None, bd, **prm).cpu().numpy(), sym)
        monkeypatch.delenv("F3M_OVERLAP")
    monkeypatch.setenv("F3M_NEAR_SYM", "0")
    plain = eng.kmvm(Xd, None, bd, **prm).cpu().numpy()
    assert rel_l2(sym, plain) < 1e-6
    # (with var_compression at this lengthscale no pair of boxes is left to the near field: nothing to differ in)
    assert name == "uniform3_varcomp" or not np.array_equal(sym, plain)


def test_symmetric_near_field_at_a_size_that_takes_it_by_itself(eng, monkeypatch):
    """2.6e6 uniform points: 20480 work items, the symmetric form is the default.  Same bits from the one-shot call, a
    kept plan and repetitions of both (integer additions commute); within 1e-6 of the plain form and within 1e-5 of
    the fp32 exact sums on the rows of a few boxes."""
    print("case symmetric near field, default path", flush=True)
    import torch
    rng = np.random.default_rng(43)
    n = 2_600_000
    X = dev(rng.random((n, 3), dtype=f32))
    b = dev(rng.standard_normal((n, 1)).astype(f32))
    first = eng.kmvm(X, None, b, ls=1.0)
    plan = eng.Plan(X, None, ls=1.0)
    for rep in range(3):
        assert torch.equal(plan.apply(b), first), rep
        assert torch.equal(eng.kmvm(X, None, b, ls=1.0), first), rep
    plan.close()
    monkeypatch.setenv("F3M_NEAR_SYM", "0")
    plain = eng.kmvm(X, None, b, ls=1.0)
    rel = float((first - plain).norm() / plain.norm())
    assert 0 < rel < 1e-6
    rows = torch.from_numpy(rng.choice(n, 2000, replace=False)).cuda()
    exact = eng.exact_f64(X[rows].double(), X.double(), b.double(), 1.0)
    err = lambda o: float((o[rows].double() - exact).norm() / exact.norm())
    assert err(first) < 1e-4 and err(first) < 1.05 * err(plain) + 1e-7


def test_symmetric_near_field_weights_of_any_size(eng, monkeypatch):
    """The fixed-point sums are scaled by the largest |weight| of the product.  Weights of 2^83 beside weights of
    order one, tiny weights (2^-100), and weights that are all zero: within 1e-5 of the plain form relative to the
    largest result.  A weight that is not finite: the kernel adds floats instead, and the targets near that source are
    not finite in either form."""
    print("case symmetric near field, weights", flush=True)
    rng = np.random.default_rng(45)
    n = 60000
    X = rng.random((n, 3), dtype=f32)
    Xd = dev(X)
    prm = dict(ls=0.5)
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    cases = {"mixed": rng.standard_normal((n, 1)).astype(f32), "tiny": (rng.standard_normal((n, 1)) * 2.0 ** -100).astype(f32),
             "zero": np.zeros((n, 1), f32)}
    cases["mixed"][::1000] *= f32(2.0 ** 83)
    for what, b in cases.items():
        monkeypatch.setenv("F3M_NEAR_SYM", "1")
        sym = eng.kmvm(Xd, None, dev(b), **prm).cpu().numpy()
        monkeypatch.setenv("F3M_NEAR_SYM", "0")
        plain = eng.kmvm(Xd, None, dev(b), **prm).cpu().numpy()
        assert np.isfinite(sym).all(), what
        # (sums in another order: a few 1e-6 of the largest result; the partial products of the tiny weights reach
        # the subnormal range, where both forms lose bits)
        scale = np.abs(plain).max()
        assert np.abs(sym.astype(np.float64) - plain).max() <= (1e-4 if what == "tiny" else 1e-5) * scale, what
    b = rng.standard_normal((n, 1)).astype(f32)
    b[12345] = np.inf
    monkeypatch.setenv("F3M_NEAR_SYM", "1")
    sym = eng.kmvm(Xd, None, dev(b), **prm).cpu().numpy()
    monkeypatch.setenv("F3M_NEAR_SYM", "0")
    plain = eng.kmvm(Xd, None, dev(b), **prm).cpu().numpy()
    close = np.linalg.norm(X - X[12345], axis=1) < 0.05
    assert close.sum() > 1 and not np.isfinite(sym[close]).any() and not np.isfinite(plain[close]).any()
    both = np.isfinite(sym[:, 0]) & np.isfinite(plain[:, 0])            # (the far field carries the weight to most targets)
    assert np.array_equal(np.isfinite(sym), np.isfinite(plain))
    assert not both.any() or rel_l2(sym[both], plain[both]) < 1e-5


@pytest.mark.parametrize("c", [1, 3, 6])
def test_results_added_straight_into_the_output_array(eng, monkeypatch, c):
    """Where the near field is one launch with one wavefront per work item and the far field is evaluated once, both
    add their sums straight into the caller's array (atomic additions into a cleared array, two per element) instead
    of going through sorted arrays and a scatter pass.  Same bits as the scatter form (a + b either way), for the
    one-shot call and for a kept plan, with one, three (padded to four) and six (four + two) columns; and the same
    bits again when repeated."""
    import torch
    from f3m_amd.capi import F3MError
    print("case direct output, %d columns" % c, flush=True)
    rng = np.random.default_rng(41)
    n = 2_600_000                                   # 4096 boxes of ~635 points: 20480 work items of 128 targets
    X = dev(rng.random((n, 3), dtype=f32))
    b = dev(rng.standard_normal((n, c)).astype(f32))
    if c == 1:
        # a single column on one tree would take the symmetric near field, whose sums go through the scatter pass
        monkeypatch.setenv("F3M_NEAR_SYM", "0")
    monkeypatch.setenv("F3M_DIRECT", "0")
    want = eng.kmvm(X, None, b, ls=1.0)
    monkeypatch.setenv("F3M_DIRECT", "2")           # fails if the product does not take the direct path
    got = eng.kmvm(X, None, b, ls=1.0)
    assert torch.equal(got, want)
    plan = eng.Plan(X, None, ls=1.0)
    assert torch.equal(plan.apply(b), want)
    assert torch.equal(plan.apply(b), want)
    plan.close()
    # a cloud whose near field is cut into slices does not qualify
    small = dev(rng.random((100000, 3), dtype=f32))
    with pytest.raises(F3MError) as e:
        eng.kmvm(small, None, dev(rng.standard_normal((100000, 1)).astype(f32)), ls=1.0)
    assert e.value.code == 37


def test_inputs_at_any_four_byte_alignment(eng):
    """Views that start in the middle of an allocation (12-byte rows) are not 16-byte aligned."""
    rng = np.random.default_rng(17)
    big = dev(rng.random((30001, 3), dtype=f32))
    b = dev(rng.standard_normal((30000, 1)).astype(f32))
    for start in (1, 0):
        view = big[start:start + 30000]
        assert view.is_contiguous()
        got = eng.kmvm(view, None, b, ls=0.5)
        ref = eng.kmvm(view.clone(), None, b, ls=0.5)
        assert np.array_equal(got.cpu().numpy(), ref.cpu().numpy())


def test_columns_linearity_and_plan_reuse(eng, oracle):
    rng = np.random.default_rng(11)
    X = rng.random((40000, 3), dtype=f32)
    b = rng.standard_normal((40000, 3)).astype(f32)
    plan = eng.Plan(dev(X), None, ls=0.4)
    o = plan.apply(dev(b)).cpu().numpy()
    for col in range(3):
        assert np.array_equal(plan.apply(dev(b[:, col:col + 1])).cpu().numpy(), o[:, col:col + 1])
    comb = plan.apply(dev((2 * b[:, :1] - b[:, 1:2]).astype(f32))).cpu().numpy()
    assert rel_l2(comb, 2.0 * o[:, :1] - o[:, 1:2]) < 1e-5
    one_shot = eng.kmvm(dev(X), None, dev(b), ls=0.4).cpu().numpy()
    assert np.array_equal(one_shot, o)                   # deterministic: no float atomics anywhere


@pytest.mark.parametrize("c", [2, 5, 6, 9])
def test_column_groups(eng, c):
    """Columns are multiplied four at a time, a last single column on its own; every column must equal
    the product of that column alone, bit for bit, for two trees as well."""
    rng = np.random.default_rng(c)
    X = rng.random((30000, 3), dtype=f32)
    Y = rng.random((20000, 3), dtype=f32)
    b = rng.standard_normal((20000, c)).astype(f32)
    plan = eng.Plan(dev(X), dev(Y), ls=0.4)
    all_cols = plan.apply(dev(b)).cpu().numpy()
    for col in range(c):
        one = plan.apply(dev(b[:, col:col + 1])).cpu().numpy()
        assert np.array_equal(one[:, 0], all_cols[:, col]), col


def test_edge_cases(eng, oracle):
    import torch
    from f3m_amd.capi import F3MError
    rng = np.random.default_rng(12)
    X = rng.random((600, 3), dtype=f32)
    b = rng.standard_normal((600, 2)).astype(f32)
    # N <= min_points: no division, exact product
    out = eng.kmvm(dev(X), None, dev(b), ls=0.5).cpu().numpy()
    assert rel_l2(out, oracle.exact_f64(X, X, b, 0.5)) < 1e-5
    # nothing far: reduces to the dense product
    X2 = rng.random((3000, 3), dtype=f32)
    b2 = rng.standard_normal((3000, 1)).astype(f32)
    out = eng.kmvm(dev(X2), None, dev(b2), ls=0.5, small_field_points=10000).cpu().numpy()
    assert rel_l2(out, oracle.exact_f64(X2, X2, b2, 0.5)) < 1e-5
    # tiny and ragged
    Xt = rng.random((1, 3), dtype=f32)
    assert np.allclose(eng.kmvm(dev(Xt), None, dev(np.ones((1, 1), f32)), ls=1.0).cpu().numpy(), 1.0)
    Y3 = rng.random((2001, 3), dtype=f32)
    out = eng.kmvm(dev(X2[:1777]), dev(Y3), dev(rng.standard_normal((2001, 1)).astype(f32)), ls=0.3, min_points=100,
                   small_field_points=50, nr_of_interpolation=27)
    assert out.shape == (1777, 1) and torch.isfinite(out).all()
    with pytest.raises(F3MError):
        eng.kmvm(dev(X), None, dev(b), ls=0.0)
    # all points identical: cannot be divided, exact product
    assert np.allclose(eng.kmvm(dev(np.ones((2000, 3), f32)), None, dev(np.ones((2000, 1), f32))).cpu().numpy(), 2000.0)
    with pytest.raises(RuntimeError):
        eng.kmvm(torch.from_numpy(X), None, torch.from_numpy(b))                      # host tensors
    with pytest.raises(AssertionError):
        eng.kmvm(dev(X), None, dev(b[:100]))


def test_c_program_on_the_abi(eng):
    """tests/abi_c/abi_smoke.c: a plain C program (HIP runtime for device memory, no Python in the process) calls
    f3m_kmvm_f32, a plan forward and transposed, and the exact product through include/f3m.h."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi_c", "_build", "abi_smoke")
    assert os.path.exists(exe), "tests/abi_c/build_smoke.py has not been run"
    print("case C program", flush=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0 and res.stdout.strip().endswith("OK"), res.stdout + res.stderr


def test_reference_operator_classes(eng, oracle):
    import torch
    from f3m_amd import ffm_3d_float
    from f3m_amd.FFM_classes import FFM, benchmark_matmul, benchmark_matmul_double, block_FFM_matmul
    assert len(ffm_3d_float.__all__) == 40
    rng = np.random.default_rng(13)
    X = rng.random((30000, 3), dtype=f32)
    Y = rng.random((9000, 3), dtype=f32)
    b = rng.standard_normal((30000, 1)).astype(f32)
    by = rng.standard_normal((9000, 1)).astype(f32)
    Xt, Yt, bt, byt = (torch.from_numpy(v) for v in (X, Y, b, by))
    ref = (benchmark_matmul_double(Xt, ls=0.5) @ bt).cpu().numpy()
    assert rel_l2(ref[:500], oracle.exact_f64(X[:500], X, b, 0.5)) < 1e-12
    assert rel_l2((FFM(Xt, ls=0.5) @ bt).cpu().numpy(), ref) < 1e-3
    assert rel_l2((benchmark_matmul(Xt, ls=0.5) @ bt).cpu().numpy(), ref) < 1e-5
    ffm = FFM(Xt, Yt, ls=0.5)
    refxy = (benchmark_matmul_double(Xt, Yt, ls=0.5) @ byt).cpu().numpy()
    assert rel_l2((ffm @ byt).cpu().numpy(), refxy) < 1e-3
    assert rel_l2(ffm.chunk_forward_example(byt, chunks=3).cpu().numpy(), refxy) < 1e-3
    refT = (benchmark_matmul_double(Yt, Xt, ls=0.5) @ bt).cpu().numpy()
    assert rel_l2(ffm.chunk_forward_transpose(bt, chunks=3).cpu().numpy(), refT) < 1e-3
    blk = block_FFM_matmul(Xt, ls=0.5, blocks_X=2) @ bt
    assert rel_l2(blk.numpy(), ref) < 1e-3
    g = ffm.grad(byt).cpu().numpy()
    assert rel_l2(g, oracle.exact_grad_f32(X, Y, by, 0.5)) < 1e-5
