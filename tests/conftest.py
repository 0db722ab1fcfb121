import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    return entry.load_package()


@pytest.fixture(scope="session")
def synth(pkg):
    import mynah_tts_amd.synth as s
    return s


@pytest.fixture(scope="session")
def orc():
    return entry.load_oracle()


@pytest.fixture(scope="session")
def ref(orc):
    """The compiled reference (stock flags).  Present wherever oracle/_ref was built."""
    if not orc.ref_available():
        pytest.skip("oracle/_ref is not built (needs the reference tree)")
    return orc.load_ref(strict=False)


@pytest.fixture(scope="session")
def ref_strict(orc):
    if not orc.ref_available(strict=True):
        pytest.skip("oracle/_ref is not built (needs the reference tree)")
    return orc.load_ref(strict=True)


@pytest.fixture(scope="session")
def backend(pkg):
    """One backend for the whole GPU session (one process, one stream)."""
    b = pkg.Backend()
    yield b
    b.close()


def norm_err(got, want):
    """max|got - want| / max|want|: the normalised error every f32 tolerance in these tests refers to.
    (Elementwise relative error explodes on near-zero outputs; the reference's own tests floor the
    denominator at 1e-3, src/qmat.c:951.)"""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    denom = float(np.max(np.abs(want)))
    return float(np.max(np.abs(got - want))) / (denom if denom > 0 else 1.0)


@pytest.fixture(scope="session")
def nerr():
    return norm_err
