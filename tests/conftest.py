import os
import sys
from pathlib import Path

import pytest

REPO_ROOT = Path(__file__).resolve().parents[1]
if str(REPO_ROOT) not in sys.path:
    sys.path.insert(0, str(REPO_ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu on an MI355X)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders (config.json + model.safetensors, random weights) of the tiny configurations,
    made once per session in a temporary folder."""
    from tests.configs import TINY_CONFIGS
    from clockwork_amd.weights.random_init import write_random_model

    from tests.replay import sharpen

    root = tmp_path_factory.mktemp("models")
    dirs = {name: write_random_model(root / name, cfg, seed) for name, (cfg, seed, _) in TINY_CONFIGS.items()}
    # the same models with peaked attention: a wrong key shows in their logits
    for name in ("A", "B"):
        dirs[name + "_peaked"] = sharpen(dirs[name], root / (name + "_peaked"))
    return dirs
