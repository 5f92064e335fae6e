"""Pins the oracle's numerics against dense fp64 products and library routines
(reference: F3M_src/1_d_conv.cu:60-73,171-214,255-335,451-817; F3M_src/n_tree.cu:489-593,1056-1125)."""
import numpy as np
import pytest
from scipy.spatial.distance import cdist

f32 = np.float32


def dense64(X, Y, b, ls):
    K = np.exp(-cdist(X.astype(np.float64), Y.astype(np.float64), "sqeuclidean") / (2 * ls * ls))
    return K @ b.astype(np.float64)


def test_exact_kernels_vs_dense(oracle):
    rng = np.random.default_rng(0)
    X = rng.standard_normal((300, 4)).astype(f32)
    Y = rng.standard_normal((450, 4)).astype(f32)
    b = rng.standard_normal((450, 3)).astype(f32)
    ref = dense64(X, Y, b, 0.7)
    assert oracle.rel_l2(oracle.exact_f32(X, Y, b, 0.7), ref) < 2e-6
    assert oracle.rel_l2(oracle.exact_f64(X, Y, b, 0.7), ref) < 1e-13
    assert oracle.rel_l2(oracle.exact_tiled_torch(X, Y, b, 0.7, row_tile=64, col_tile=100).numpy(), ref) < 5e-6
    # d/d ls of the product: finite difference of the dense fp64 product
    h = 1e-5
    fd = (dense64(X, Y, b, 0.7 + h) - dense64(X, Y, b, 0.7 - h)) / (2 * h)
    assert oracle.rel_l2(oracle.exact_grad_f32(X, Y, b, 0.7), fd) < 1e-5


@pytest.mark.parametrize("d,P", [(1, 6), (2, 16), (3, 64), (4, 81), (5, 243)])
def test_m2l_block_is_dense_gaussian_of_shifted_nodes(oracle, d, P):
    rng = np.random.default_rng(d)
    per, nodes, w, idx, coords = oracle.node_grid(d, P)
    edge = f32(0.25)
    cx = rng.random(d).astype(f32)
    cy = (cx + edge * rng.integers(-3, 4, d)).astype(f32)
    lcs = f32(1 / (2 * 0.3 ** 2))
    K = oracle.m2l_block(d, P, cx, cy, edge, lcs)
    nx = cx.astype(np.float64) + coords.astype(np.float64) * edge / 2 + edge / 2
    ny = cy.astype(np.float64) + coords.astype(np.float64) * edge / 2 + edge / 2
    ref = np.exp(-np.float64(lcs) * cdist(nx, ny, "sqeuclidean"))
    assert np.abs(K - ref).max() < 2e-5
    assert K.shape == (len(coords), len(coords))


def test_reduces_to_dense_product_when_nothing_is_far(oracle):
    # small_field_points > N and d <= 3: at depth 1 every child pair is adjacent and "small"
    rng = np.random.default_rng(1)
    for d in (1, 2, 3):
        X = rng.random((1500, d)).astype(f32)
        b = rng.standard_normal((1500, 2)).astype(f32)
        P = oracle.Plan(X, None, ls=0.4, min_points=1000, small_field_points=5000)
        assert P.nlevels == 1
        L = P.level(0)
        assert len(L["far"]) == 0 and len(L["keep"]) == 0
        assert oracle.rel_l2(P.apply(b), dense64(X, X, b, 0.4)) < 3e-6


CASES = [
    ("sym3", 3, 6000, None, 0.5, 64),
    ("sym2", 2, 5000, None, 0.3, 64),
    ("asym3", 3, 5000, 3000, 0.7, 64),
    ("sym4", 4, 6000, None, 1.0, 81),
]


@pytest.mark.parametrize("name,d,N,M,ls,P", CASES, ids=[c[0] for c in CASES])
def test_end_to_end_rel_l2(oracle, name, d, N, M, ls, P):
    rng = np.random.default_rng(2)
    X = rng.random((N, d)).astype(f32)
    Y = None if M is None else (rng.random((M, d)) * 1.2 - 0.1).astype(f32)
    b = rng.standard_normal((N if M is None else M, 1)).astype(f32)
    plan = oracle.Plan(X, Y, ls=ls, min_points=200, nr_of_interpolation=P, small_field_points=200)
    assert sum(len(plan.level(k)["far"]) for k in range(plan.nlevels)) > 0
    out = plan.apply(b)
    ref = dense64(X, X if Y is None else Y, b, ls)
    assert oracle.rel_l2(out, ref) < 1e-3


def test_stage_outputs_sum_to_the_product(oracle):
    rng = np.random.default_rng(3)
    X = rng.random((5000, 3)).astype(f32)
    b = rng.standard_normal((5000, 2)).astype(f32)
    plan = oracle.Plan(X, None, ls=0.5, min_points=200, small_field_points=200)
    total = np.zeros((5000, 2), np.float64)
    for k in range(plan.nlevels):
        total += plan.near_level(k, "small", b)
        L = plan.level(k)
        if len(L["far"]):
            o, mom, loc = plan.far_level(k, b)
            total += o
            # moments of a box interpolate its weights: sum of moments == sum of b over the box
            by = np.unique(L["far"][:, 1])
            for bb in by[:5]:
                pts = L["permy"][L["offy"][bb]:L["offy"][bb + 1]]
                assert np.allclose(mom[bb].sum(0), b[pts].sum(0), atol=1e-3)
    total += plan.near_level(plan.nlevels - 1, "keep", b)
    assert oracle.rel_l2(total, plan.apply(b)) < 1e-6


def test_error_decreases_with_node_count_and_linearity(oracle):
    rng = np.random.default_rng(4)
    X = rng.random((6000, 3)).astype(f32)
    b = rng.standard_normal((6000, 2)).astype(f32)
    ref = dense64(X, X, b, 0.4)
    errs = []
    for P in (8, 27, 64, 125):
        errs.append(oracle.rel_l2(oracle.kmvm(X, None, b, ls=0.4, min_points=200, nr_of_interpolation=P,
                                              small_field_points=200), ref))
    assert errs[0] > errs[1] > errs[2] > errs[3], errs
    plan = oracle.Plan(X, None, ls=0.4, min_points=200, small_field_points=200)
    o = plan.apply(b)
    o0 = plan.apply(b[:, :1])
    assert np.allclose(o[:, :1], o0, rtol=0, atol=0)     # columns are independent
    o2 = plan.apply(2.0 * b[:, :1] + b[:, 1:])
    assert oracle.rel_l2(o2, 2.0 * o[:, :1].astype(np.float64) + o[:, 1:]) < 1e-5


def test_sums_restricted_to_selected_rows_are_the_unrestricted_sums(oracle):
    """`rows=`: the same sums for some target rows only (M2L only for the boxes that hold one of them).  Used by
    the GPU tests on clouds whose complete M2L would keep a CPU busy for minutes; on a cloud small enough for both,
    the restricted results must have the bits of the unrestricted ones on those rows and be zero elsewhere."""
    rng = np.random.default_rng(6)
    X = rng.random((5000, 3)).astype(f32)
    Y = rng.random((3000, 3)).astype(f32)
    b = rng.standard_normal((3000, 2)).astype(f32)
    plan = oracle.Plan(X, Y, ls=0.5, min_points=100, nr_of_interpolation=27, small_field_points=60)
    assert plan.nlevels >= 2
    rows = np.unique(rng.integers(0, 5000, 300))
    others = np.setdiff1d(np.arange(5000), rows)
    full, part = plan.apply(b), plan.apply(b, rows=rows)
    assert np.array_equal(part[rows], full[rows]) and not part[others].any()
    did_far = False
    for k in range(plan.nlevels):
        L = plan.level(k)
        for which in ("small", "keep"):
            f, p = plan.near_level(k, which, b), plan.near_level(k, which, b, rows=rows)
            assert np.array_equal(p[rows], f[rows]) and not p[others].any()
        if len(L["far"]):
            did_far = True
            (fo, fm, fl), (po, pm, pl) = plan.far_level(k, b), plan.far_level(k, b, rows=rows)
            assert np.array_equal(pm, fm)                                  # moments of every Y box either way
            assert np.array_equal(po[rows], fo[rows]) and not po[others].any()
            box = np.empty(5000, np.int64)
            box[L["permx"]] = np.repeat(np.arange(len(L["offx"]) - 1), np.diff(L["offx"]))
            mine = np.unique(box[rows])
            assert np.array_equal(pl[mine], fl[mine])                      # local expansions of the boxes that hold a row
            rest = np.setdiff1d(np.arange(len(L["offx"]) - 1), mine)
            assert not pl[rest].any()
    assert did_far
