"""CPU checks of the drop-in boundary: the gfx950 library loads and exports every symbol that
include/f3m.h declares, the Python shim exposes the reference's 40 names, and the product refuses
to run without a GPU instead of falling back."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from f3m_amd import _lib, capi
    header = open(os.path.join(ROOT, "include", "f3m.h")).read()
    declared = set(re.findall(r"\b(f3m_[a-z0-9_]+)\s*\(", header))
    assert declared == set(capi.SYMBOLS), declared ^ set(capi.SYMBOLS)
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built yet (python -m f3m_amd.build)")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert capi.bind(lib).f3m_version().startswith(b"f3m-gfx950")


def test_python_shim_has_the_reference_names():
    torch = pytest.importorskip("torch")
    from f3m_amd import ffm_3d_float as m
    names = ["FFM_XY_FLOAT_%d" % k for k in range(1, 11)] + ["rbf_float_%d" % k for k in range(1, 11)] + \
            ["rbf_float_%d_grad" % k for k in range(1, 11)] + ["rbf_double_%d" % k for k in range(1, 11)]
    for n in names:
        assert callable(getattr(m, n)), n
    assert sorted(m.__all__) == sorted(names)
    # no CPU fallback: host tensors are refused
    X = torch.rand(100, 3)
    b = torch.rand(100, 1)
    from f3m_amd import _lib
    if os.path.exists(_lib.LIB_PATH):
        with pytest.raises(RuntimeError):
            m.FFM_XY_FLOAT_3(X, X, b, "cpu", 1.0, 1000.0, 64, False, 0.15, 1000)
        with pytest.raises(RuntimeError):
            m.rbf_float_3(X, X, b, 1.0, True)


def test_product_never_imports_the_oracle():
    import subprocess
    import sys
    code = "import sys; sys.path.insert(0, %r); import f3m_amd.engine, f3m_amd.FFM_classes, f3m_amd.ffm_3d_float; " \
           "bad = [m for m in sys.modules if m.startswith('oracle') or 'emu' in m]; assert not bad, bad" % ROOT
    subprocess.check_call([sys.executable, "-c", code])


def test_node_count_rule_matches_oracle(oracle):
    from f3m_amd import engine
    for d, P in [(3, 64), (4, 81), (5, 243), (3, 100), (2, 30), (1, 9), (5, 32)]:
        assert engine.node_counts(d, P) == oracle.node_counts(d, P).tolist()
