"""Shared pytest set-up: the ``gpu`` marker and the import path of the repository root."""
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> folder of a tiny random-weight model (written once per session, in a temporary folder)."""
    import tiny_models

    root = tmp_path_factory.mktemp("models")
    return {name: tiny_models.write(name, root) for name in tiny_models.CONFIGS}


@pytest.fixture
def cpu_ops(monkeypatch):
    """Patch the CPU stand-ins of ``tests/emulated_ops.py`` over the HIP entry points, so that
    host logic can run without a GPU.  Never used by GPU tests."""
    import emulated_ops
    from torchlet_amd.kernels import ops

    for name in ("attention_tile_tokens", "load", "embedding", "add_rmsnorm", "linear", "rope_cache_write",
                 "paged_attention", "swiglu", "sample", "interleave_gate_up", "linear_swiglu",
                 "prefill_attention_tile_tokens", "paged_attention_prefill", "linear_partials", "linear_partials_pay", "linear_rope_cache_write"):
        monkeypatch.setattr(ops, name, getattr(emulated_ops, name))
    return ops
