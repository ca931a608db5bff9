import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "fastgl-ae_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def small_graph(oracle):
    """R-MAT graph of the CPU-runnable configuration: 100K nodes, ~2.5M directed edges."""
    indptr, indices = oracle.rmat_csr(100_000, 1_500_000, seed=0)
    return indptr, indices


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a GPU")
    import fastgl
    fastgl.lib()  # raises if the HIP library is not built: there is no fallback
    return torch.device("cuda:0")
