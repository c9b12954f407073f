import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Random-weight model folders of the tiny configurations, made once per
    session in a temporary folder."""
    import nnis_amd
    from configs import TINY_CONFIGS

    out = {}
    for name, (config, seed) in TINY_CONFIGS.items():
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        nnis_amd.write_random_model(str(folder), config, seed)
        out[name] = str(folder)
    return out
