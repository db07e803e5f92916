import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
TEST_PROGRAMS = ROOT / "tests" / "programs" / "libtftestprograms.so"
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_sessionstart(session):
    """The tests load the libraries that are built in-tree; only when none is there yet (a fresh checkout) are they
    built first. There is no fallback of any kind: without hipcc this fails."""
    lib = ROOT / "tensorfrost_amd" / "lib"
    test_programs = TEST_PROGRAMS
    if not (lib / "libtfhip.so").exists() or not (lib / "libtfhost.so").exists() or not test_programs.exists():
        from tensorfrost_amd import build as tf_build

        tf_build.build_all()
    # The op-by-op programs of this suite live in a library of their own, outside the product library.
    from tensorfrost_amd import host

    host.load_programs(test_programs)
    from oracle import oracle

    if not (ROOT / "oracle" / "liboracle.so").exists():
        oracle.build()


@pytest.fixture(scope="session")
def rt():
    """The device runtime, initialised once per session. Fails (never skips) if the HIP library is absent."""
    from tensorfrost_amd import runtime

    runtime.initialize(0)
    yield runtime
    runtime.synchronize()


def rel_err(got, ref):
    """Max relative error with an absolute floor of 1e-6 * max|ref| for near-zero elements."""
    import numpy as np

    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    floor = 1e-6 * max(float(np.max(np.abs(ref))), 1e-30)
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))


def sum_err(got, ref, abs_sum):
    """Error of a sum relative to the sum of magnitudes of its terms (the conditioning-free measure:
    a sum of n fp32 terms in any order is within n*eps*abs_sum of the exact one)."""
    import numpy as np

    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(got - ref) / np.maximum(np.asarray(abs_sum, dtype=np.float64), 1e-30)))
