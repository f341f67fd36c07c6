"""Test configuration: import paths, the `gpu` marker and per-test context hygiene."""

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT, ROOT / "nanovllm-voxcpm_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run on the MI355X box with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no ROCm GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _clean_lora_state():
    from nanovllm_voxcpm_amd.lora import set_backend_for_testing
    from nanovllm_voxcpm_amd.utils.context import reset_lora_context

    reset_lora_context()
    set_backend_for_testing(None)
    yield
    reset_lora_context()
    set_backend_for_testing(None)
    # environment changes of the test are undone by now: let the library drop what it read
    from nanovllm_voxcpm_amd import _hip

    if _hip.load_error() is None:
        _hip.reload_knobs()
