import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


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
