"""The committed oracle fixtures (tests/golden/oracle_fixtures.npz) against (a) the oracle as it is now,
(b) the engine's kernel sources in the CPU emulation.  The GPU library is checked against the same
fixtures in test_gpu_parity.py."""
import numpy as np
import pytest

import golden_fixtures as gf
from parity_checks import rel_l2, expected_list_rows

NAMES = gf.names()


@pytest.mark.parametrize("name", NAMES)
def test_oracle_reproduces_its_fixtures(oracle, name):
    fx = gf.load()
    X, Y, b, prm = gf.case(fx, name)
    plan = oracle.Plan(X, Y, **prm)

    class View:                     # oracle levels are numbered from 0
        @staticmethod
        def level(k):
            return plan.level(k - 1)
    gf.assert_plan_matches_fixture(View, plan.nlevels, fx, name)
    assert np.array_equal(np.asarray(oracle.node_counts(X.shape[1], prm["nr_of_interpolation"]), np.int32),
                          fx[name + "/node_counts"])
    assert rel_l2(plan.apply(b), fx[name + "/product_oracle"]) < 1e-7
    assert rel_l2(oracle.exact_f64(X, X if Y is None else Y, b, prm["ls"]), fx[name + "/product_exact_f64"]) < 1e-14


@pytest.mark.parametrize("name", NAMES)
def test_emulated_engine_matches_fixtures(monkeypatch, name):
    import emu_engine as ee
    monkeypatch.setenv("F3M_NEAR", "valu")
    fx = gf.load()
    X, Y, b, prm = gf.case(fx, name)
    eng = ee.Plan(X, Y, **prm)
    gf.assert_plan_matches_fixture(eng, eng.depth, fx, name)
    for k in range(1, eng.depth + 1):
        assert eng.list_rows(k) == expected_list_rows(eng.level(k)), (name, k)
    gf.assert_product_matches_fixture(eng.apply(b), fx, name)


@pytest.mark.parametrize("name", ["d3_uniform", "d3_two_trees", "d3_lattice_duplicates", "d4_uniform"])
def test_emulated_matrix_pipe_near_field_with_source_runs(monkeypatch, name):
    """the matrix-pipe near field, whole lists per wavefront: source boxes under one parent cell form one run"""
    import emu_engine as ee
    monkeypatch.setenv("F3M_NEAR", "mfma")
    monkeypatch.setenv("F3M_SPLIT_TARGET", "1")
    fx = gf.load()
    X, Y, b, prm = gf.case(fx, name)
    eng = ee.Plan(X, Y, **prm)
    gf.assert_product_matches_fixture(eng.apply(b), fx, name)
