import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session into a
    temporary folder (never into the repository)."""
    from configs import TINY
    from xinfer_amd.weights import write_random_model
    root = tmp_path_factory.mktemp("models")
    out = {}
    for name, t in TINY.items():
        d = str(root / name)
        write_random_model(d, t["config"], t["seed"], t["linear_std"], t["norm_std"])
        out[name] = d
    return out


@pytest.fixture(scope="session")
def real_model_dirs(tmp_path_factory):
    """Model folders with real layer sizes and few layers (see configs.REAL), written on demand."""
    from configs import REAL
    from xinfer_amd.weights import write_random_model
    root = tmp_path_factory.mktemp("real_models")
    made = {}

    def get(name):
        if name not in made:
            t = REAL[name]
            made[name] = write_random_model(str(root / name), t["config"], t["seed"], t["linear_std"],
                                            t["norm_std"])
        return made[name]
    return get
