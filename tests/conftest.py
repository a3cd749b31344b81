import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the GPU box)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session by the random-weights mode.  The
    norms' scales lie well away from 1, so that a norm's weight taken from the wrong tensor, or not at all,
    changes the logits."""
    from tiny_configs import TINY
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config

    root = tmp_path_factory.mktemp("models")
    folders = {}
    for name, (raw, seed) in TINY.items():
        folder = str(root / name)
        ta.write_random_model(Qwen2Config.from_dict(raw), seed, folder, norm_spread=0.3)
        folders[name] = folder
    return folders
