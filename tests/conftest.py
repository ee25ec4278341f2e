import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here: the engine has no CPU path")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the tiny configurations with random weights, made once per session in
    a temporary folder: {(name, storage): path}."""
    from helpers import make_model_dir
    made = {}

    def get(name: str, storage: str = "float32") -> str:
        key = (name, storage)
        if key not in made:
            made[key] = make_model_dir(str(tmp_path_factory.mktemp(f"{name}_{storage}")), name, storage)
        return made[key]

    return get
