import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """The tiny models, written once per session into a temporary folder."""
    import tiny_models

    root = tmp_path_factory.mktemp("models")
    return {name: tiny_models.write_model(root / name, name) for name in tiny_models.CONFIGS}


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    """(weights, config) of the plain implementation for every tiny model."""
    import plain_gemma

    return {name: (plain_gemma.load_weights(d), plain_gemma.read_config(d)) for name, d in model_dirs.items()}
