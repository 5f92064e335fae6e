"""Pins the oracle's interpolation nodes, weights and Lagrange basis against numpy / scipy and
the closed forms (reference: F3M_src/n_tree.cu:265-349, F3M_src/1_d_conv.cu:217-238,418-448,850-884)."""
import numpy as np
import pytest
from numpy.polynomial import chebyshev as npcheb
from scipy.interpolate import BarycentricInterpolator, barycentric_interpolate


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 6, 9])
def test_nodes_are_first_kind_chebyshev_points(oracle, n):
    t, w = oracle.nodes_1d(n)
    ref = npcheb.chebpts1(n)[::-1]                      # descending, like cos((2i+1)pi/(2n))
    assert np.allclose(t, ref, atol=2e-7)
    closed = np.cos((2 * np.arange(n) + 1) * np.pi / (2 * n))
    assert np.allclose(t, closed, atol=2e-7)


@pytest.mark.parametrize("n", [2, 3, 4, 5, 8])
def test_weights_match_scipy_up_to_scale(oracle, n):
    t, w = oracle.nodes_1d(n)
    wi = BarycentricInterpolator(t.astype(np.float64)).wi
    ratio = w.astype(np.float64) / wi
    assert np.allclose(ratio, ratio[0], rtol=1e-5)
    assert np.allclose(w, [(-1) ** i * np.sin((2 * i + 1) * np.pi / (2 * n)) for i in range(n)], atol=2e-7)


def test_node_counts_rule(oracle):
    assert oracle.node_counts(3, 64).tolist() == [4, 4, 4]
    assert oracle.node_counts(4, 81).tolist() == [3, 3, 3, 3]
    assert oracle.node_counts(5, 243).tolist() == [3] * 5
    assert oracle.node_counts(3, 27).tolist() == [3, 3, 3]
    assert oracle.node_counts(3, 100).tolist() == [5, 5, 4]      # non-cube: ceil while product fits
    assert oracle.node_counts(2, 64).tolist() == [8, 8]
    assert oracle.node_counts(1, 7).tolist() == [7]
    for d, P in [(3, 64), (3, 100), (2, 30), (4, 100), (5, 300)]:
        assert int(np.prod(oracle.node_counts(d, P))) <= P


def test_node_grid_dim0_fastest(oracle):
    per, nodes, w, idx, coords = oracle.node_grid(3, 100)
    assert per.tolist() == [5, 5, 4]
    P = 100
    m = np.arange(P)
    assert (idx[:, 0] == m % 5).all()
    assert (idx[:, 1] == 5 + (m // 5) % 5).all()
    assert (idx[:, 2] == 10 + (m // 25)).all()
    assert (coords == nodes[idx]).all()


@pytest.mark.parametrize("d,P", [(1, 5), (2, 16), (3, 64), (3, 27), (4, 81), (5, 243), (3, 100)])
def test_basis_partition_of_unity_and_delta(oracle, d, P):
    rng = np.random.default_rng(d * 100 + P)
    centre = rng.standard_normal(d).astype(np.float32)
    edge = np.float32(0.37)
    for _ in range(20):
        x = (centre + (rng.random(d) - 0.5) * edge).astype(np.float32)
        L = oracle.basis(d, P, x, centre, edge)
        assert abs(L.astype(np.float64).sum() - 1.0) < 5e-5
    # delta property at the nodes themselves (exact-hit branch): local coordinate == node
    per, nodes, w, idx, coords = oracle.node_grid(d, P)
    centre0 = np.zeros(d, np.float32)
    for m in [0, len(coords) // 2, len(coords) - 1]:
        x = coords[m].copy()                            # edge = 2 -> local coordinate is x itself
        L = oracle.basis(d, P, x, centre0, np.float32(2.0))
        e = np.zeros(len(coords), np.float32)
        e[m] = 1
        assert np.array_equal(L, e)


@pytest.mark.parametrize("d,P", [(1, 4), (2, 16), (3, 64), (4, 81)])
def test_basis_reproduces_polynomials(oracle, d, P):
    rng = np.random.default_rng(7)
    per, nodes, w, idx, coords = oracle.node_grid(d, P)
    centre = rng.standard_normal(d).astype(np.float32)
    edge = np.float32(1.5)
    nodepos = centre + coords.astype(np.float64) * edge / 2
    deg = [int(n) - 1 for n in per]

    def poly(z):
        return np.prod([z[..., j] ** deg[j] + 0.5 * z[..., j] + 1 for j in range(d)], axis=0)

    for _ in range(10):
        x = (centre + (rng.random(d) - 0.5) * edge * 0.98).astype(np.float32)
        L = oracle.basis(d, P, x, centre, edge).astype(np.float64)
        assert abs(L @ poly(nodepos) - poly(x.astype(np.float64))) < 2e-4 * max(1.0, abs(poly(x.astype(np.float64))))


def test_basis_matches_scipy_barycentric_1d(oracle):
    rng = np.random.default_rng(3)
    n = 6
    t, w = oracle.nodes_1d(n)
    f = rng.standard_normal(n)
    for _ in range(20):
        x = np.float32(rng.uniform(-1, 1))
        L = oracle.basis(1, n, np.array([x]), np.zeros(1, np.float32), np.float32(2.0)).astype(np.float64)
        ref = barycentric_interpolate(t.astype(np.float64), f, np.float64(x))
        assert abs(L @ f - ref) < 1e-4
