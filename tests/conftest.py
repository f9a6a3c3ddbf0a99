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
def model_folders(tmp_path_factory):
    """One model folder (config.json, model.safetensors) per tiny configuration
    and storage dtype, written once per session into a temporary folder."""
    from helpers import CONFIGS
    from tinyinfer_amd.weights import write_model_folder
    made = {}

    def get(name: str, dtype: str = "bfloat16", sharp: bool = False):
        key = (name, dtype, sharp)
        if key not in made:
            d = tmp_path_factory.mktemp(f"model_{name}_{dtype}_{int(sharp)}")
            write_model_folder(str(d), CONFIGS[name], seed=1234 + len(name), dtype=dtype)
            if sharp:
                from helpers import sharpen_folder
                sharpen_folder(str(d))
            made[key] = str(d)
        return made[key]
    return get
