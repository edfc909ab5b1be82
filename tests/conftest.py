import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from support import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def ref():
    from support import Reference, ref_available
    if not ref_available():
        pytest.skip("oracle/_ref/libctorch_ref.so not built (reference sources not mounted)")
    return Reference()


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    from support import GOLDEN_DIR

    def load(name):
        return np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
    return load


@pytest.fixture
def exact_math():
    """The library's exact mode (glibc's floats bit for bit, exactly rounded quotients) for one test;
    the default single-precision mode is restored afterwards.  (Through ctypes alone: a test of the
    C++ front-end must not start torch's own HIP runtime after the library's.)"""
    from ctorch_amd import capi
    lib = capi.load()
    prev = lib.ctamd_math_mode()
    assert lib.ctamd_set_math_mode(1) == 0
    yield
    assert lib.ctamd_set_math_mode(prev) == 0
