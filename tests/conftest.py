import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import kquant_oracle
    kquant_oracle.lib()
    return kquant_oracle


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a GPU test was selected but no GPU is visible")
    from neuralfn_amd import tile_ops
    tile_ops.load()  # raises if the HIP library is not built: there is no fallback
    return torch.device("cuda:0")
