import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _gpu_tests_compare_with_the_gpu_statistic_order(request, monkeypatch):
    """The reference's quantisers run on the GPU, where torch reduces a 32-element group in a fixed tree order;
    the oracle restates that order (``std_mean_gpu_tree``) and every GPU test compares against it, so the std /
    mean of the 1-bit normal-quantile class are held to bit equality like everything else."""
    if request.node.get_closest_marker("gpu") is not None:
        from oracle import hqe_oracle as O
        monkeypatch.setattr(O, "NORMAL1_STAT_ORDER", "gpu_tree")
