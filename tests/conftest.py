import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_runtest_logstart(nodeid, location):
    """Name every GPU test on stderr before it runs: a kernel fault can end the machine with
    the run, and then the end of stderr is all that comes back."""
    if "test_gpu_" in nodeid or "test_zz_" in nodeid or "on_gpu" in nodeid:
        print("\n[gpu test] %s" % nodeid, file=sys.stderr, flush=True)


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def hip():
    """One libfinchhip context on cuda:0.  Fails (does not skip) when the library or the
    GPU is missing: GPU tests must never pass on a fallback."""
    from finchmoe_amd import FinchHip
    ctx = FinchHip(0)
    yield ctx
    ctx.close()


def rel_err(a, b):
    """max |a-b| / max |b| — the 'max relative error' of the parity bar, normalised by
    the largest reference magnitude so that near-zero outputs do not dominate."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30))


def cosine(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(a @ b / max(np.linalg.norm(a) * np.linalg.norm(b), 1e-300))


# parity bar for GEMV/GEMM outputs (fp32 accumulate): max relative error <= 1e-3 and
# cosine >= 0.99999
REL_TOL = 1e-3
COS_TOL = 0.99999


def assert_parity(got, ref, what=""):
    r, c = rel_err(got, ref), cosine(got, ref)
    assert r <= REL_TOL and c >= COS_TOL, "%s: rel_err %.3e cosine %.8f" % (what, r, c)
    return r, c
