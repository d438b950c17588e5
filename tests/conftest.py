"""Shared test plumbing: markers, import paths, small synthetic models."""
from __future__ import annotations

import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
for p in (ROOT, ROOT / "oracle"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

from __graft_entry__ import load_package  # noqa: E402

load_package()

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: takes more than a few seconds on CPU")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _restore_shape():
    """Tests re-point LlamaConfig at reduced shapes; put the default back afterwards."""
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig

    yield
    LlamaConfig.set_shape(LLAMA_3_2_1B)


@pytest.fixture(scope="session")
def small_model():
    """Llama-1B layer geometry, 2 layers, vocabulary 2048: weights + prompt (CPU tensors)."""
    from qimeng_megakernel_amd import synthetic

    shape = synthetic.reduced_shape(num_layers=2, vocab_size=2048)
    weights = synthetic.random_weights(shape, seed=11, max_positions=96)
    prompt = synthetic.random_prompt(shape, seed=11, length=5)
    return shape, weights, prompt
