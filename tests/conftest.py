import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")


def attn_close(got: torch.Tensor, ref: torch.Tensor, max_abs: float, mean_rel: float):
    """The acceptance bar for attention outputs: max-abs error and mean relative error
    (sum |err| / sum |ref|) against the fp32 oracle."""
    got, ref = got.float().cpu(), ref.float().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert torch.isfinite(got).all(), "non-finite values in the kernel output"
    err = (got - ref).abs()
    ma = err.max().item()
    mr = (err.sum() / ref.abs().sum().clamp_min(1e-30)).item()
    assert ma <= max_abs and mr <= mean_rel, f"max_abs={ma:.4g} (<= {max_abs}), mean_rel={mr:.4g} (<= {mean_rel})"
    return ma, mr
