import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this machine")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders (config.json + model.safetensors) of the tiny configurations,
    written once per session into a temporary folder, in float32."""
    from tiny_configs import TINY, write_tiny

    root = tmp_path_factory.mktemp("models")
    return {name: write_tiny(name, str(root / name), torch.float32) for name in TINY}


@pytest.fixture(scope="session")
def model_dirs_bf16(tmp_path_factory):
    from tiny_configs import TINY, write_tiny

    root = tmp_path_factory.mktemp("models_bf16")
    return {name: write_tiny(name, str(root / name), torch.bfloat16) for name in TINY}


@pytest.fixture(scope="session")
def wide_model_dir_f32(tmp_path_factory):
    """The two-layer model at serving widths in float32 (about 6 GB: written once for all tests that use it)."""
    from tiny_configs import write_tiny

    return write_tiny("W", str(tmp_path_factory.mktemp("models_wide_f32") / "W"), torch.float32)


@pytest.fixture(scope="session")
def many_experts_model_dir_f32(tmp_path_factory):
    """128 experts on the second of two layers at serving widths, in float32 (about 3.6 GB, written once)."""
    from tiny_configs import write_tiny

    return write_tiny("M", str(tmp_path_factory.mktemp("models_many_experts_f32") / "M"), torch.float32)
