import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _have_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _decoder_switches_restored():
    """Tests flip the decoders' class-level switches (fused element-wise launches, gate placement); a failing test must not
    leave them flipped for the tests after it."""
    yield
    mods = sys.modules
    if "trimkv_amd.decoder_ops" in mods:
        mods["trimkv_amd.decoder_ops"].enabled = True
    if "trimkv_amd.qwen3" in mods:
        attn = mods["trimkv_amd.qwen3"].TrimKVQwen3Attention
        attn.fold_gate, attn.gate_on_side_stream = True, False
