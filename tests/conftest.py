import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "gpu_perf: timing gates on a real MI355X (run with -m gpu_perf); kept apart from the "
                                       "parity suite so that a clock or occupancy wobble on a shared box cannot turn "
                                       "correctness red")


@pytest.fixture(scope="session")
def hip_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def golden_vectors():
    """The reference's literal test vectors and published known answers (tests/golden/reference_vectors.json)."""
    import json
    from pathlib import Path

    return json.loads((Path(__file__).resolve().parent / "golden" / "reference_vectors.json").read_text())
