import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__

    return __graft_entry__.import_package()


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def force_grouped_shape(pkg):
    """Forces the kernel family of the grouped Q4_K launches for one test ("" / None = the library's own choice)."""
    lib = pkg._lib.load()

    def force(shape):
        pkg._lib.check(lib.ggq_debug_force_grouped_shape(-1 if shape in ("", None) else int(shape)))

    yield force
    lib.ggq_debug_force_grouped_shape(-1)
