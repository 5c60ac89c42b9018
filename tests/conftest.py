import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU and the compiled kernels")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the tiny configurations with random weights, written once per test session:
    ``model_dirs(name, dtype)`` -> folder."""
    from tiny_configs import TINY
    from turboquant_cpp_amd.engine.model import write_random_model_dir
    made = {}

    def get(name: str, dtype: str = "float32") -> str:
        key = (name, dtype)
        if key not in made:
            cfg, init = TINY[name]
            d = str(tmp_path_factory.mktemp(f"tiny_{name}_{dtype}"))
            write_random_model_dir(d, cfg, init["seed"], init["std"], init["norm_std"], dtype)
            made[key] = d
        return made[key]
    return get
