from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for path in (str(ROOT), str(ROOT / "tests")):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu); everything else runs on the CPU")


def pytest_collection_modifyitems(config, items):
    """A test marked ``gpu`` is skipped where no GPU is visible."""

    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders of the tiny configurations, random weights stored in
    float32, in a temporary place: ``{"a": (folder, block_size), "b": ..., "c": ...}``."""

    from helpers import TINY, make_model_folder

    base = tmp_path_factory.mktemp("models")
    folders = {}
    for seed, (name, (make_config, block_size)) in enumerate(TINY.items()):
        folders[name] = (make_model_folder(base / name, make_config(), seed=11 + seed), block_size)
    return folders
