import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real GPU (run with -m gpu on an MI355X)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders (random weights) of the two tiny configurations, made once per session in a temp folder."""
    import tiny
    out = {}
    for name, raw, seed, norm_std in (("A", tiny.tiny_a(), 101, 0.1), ("B", tiny.tiny_b(), 202, 0.0)):
        d = tmp_path_factory.mktemp(f"tiny_{name}")
        tiny.write_model(raw, str(d), seed, norm_std=norm_std)
        out[name] = str(d)
    return out
