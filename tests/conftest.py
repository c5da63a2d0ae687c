import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders (config.json + model.safetensors, random bf16 weights) of
    the tiny configurations, made once in a temporary folder."""
    from helpers import TINY, make_model_folder
    root = tmp_path_factory.mktemp("models")
    return {name: make_model_folder(str(root / name), name) for name in TINY}
