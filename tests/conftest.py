import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


ENGINES = {"auto": 0, "lds_table": 1, "direct": 2}


@pytest.fixture(params=list(ENGINES))
def amsim_engine(request):
    """Runs a GPU parity test once per GEMM engine setting (amsim_set_engine): picked per problem,
    LDS-table engine only, direct engine wherever it can index the problem.  Modules opt in with
    ``pytest.mark.usefixtures("amsim_engine")``."""
    import approxtrain_amd
    lib = approxtrain_amd.load_library()
    assert lib.amsim_set_engine(ENGINES[request.param]) == 0
    yield request.param
    lib.amsim_set_engine(0)
