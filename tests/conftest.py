import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import vmo
    return vmo.load("oracle")


@pytest.fixture(scope="session")
def reference():
    """The reference's own headers compiled behind the oracle interface; absent where the reference tree
    was not mounted at build time."""
    from oracle import vmo
    ref = vmo.load("reference")
    if ref is None:
        pytest.skip("oracle/_ref/libvm_ref.so is not built (needs the reference tree)")
    return ref


@pytest.fixture(scope="session")
def oracle64():
    """the restatement compiled for Scalar = double"""
    from oracle import vmo
    return vmo.load("oracle", real="f64")


@pytest.fixture(scope="session")
def reference64():
    """the reference's headers instantiated with Scalar = double"""
    from oracle import vmo
    ref = vmo.load("reference", real="f64")
    if ref is None:
        pytest.skip("oracle/_ref/libvm_ref_f64.so is not built (needs the reference tree)")
    return ref
