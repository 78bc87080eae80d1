"""Shared test configuration: the `gpu` marker, repo-root imports and tiny helpers."""
import pathlib
import sys

import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def has_gpu() -> bool:
    return torch.cuda.is_available() and torch.cuda.device_count() > 0


@pytest.fixture(scope="session")
def device():
    if not has_gpu():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


def rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    """max|out - ref| / max|ref|, the metric of the reference's own MoE tests (tests/test_moe.py:49)."""
    return ((out.double() - ref.double()).abs().max() / ref.double().abs().max()).item()
