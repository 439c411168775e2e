import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    """The committed golden vectors (tests/golden/*.npz), loaded without pickle."""
    import numpy as np

    gdir = os.path.join(ROOT, "tests", "golden")
    out = {}
    for name in sorted(os.listdir(gdir)):
        if name.endswith(".npz"):
            with np.load(os.path.join(gdir, name), allow_pickle=False) as z:
                out[name[:-4]] = {k: z[k] for k in z.files}
    return out


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible (tests marked gpu need an MI355X)")
    return torch.device("cuda:0")
