import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders (config.json + model.safetensors) of the tiny
    configurations, made once per session in a temporary folder."""
    import tiny
    made = {}

    def get(name, seed=3, store="float32"):
        key = (name, seed, store)
        if key not in made:
            d = tmp_path_factory.mktemp(f"model_{name}_{seed}_{store}")
            tiny.write_model(str(d), tiny.CONFIGS[name], seed, store)
            made[key] = str(d)
        return made[key]
    return get
