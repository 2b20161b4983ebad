"""pytest configuration: `gpu` marker and import paths.

`-m "not gpu"` covers the oracle against the reference's golden vectors, the host
logic and the C-ABI surface; `-m gpu` are the parity tests proper and call the
HIP kernels through the C ABI.
"""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "sparse-attention-hub_amd"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels)")


@pytest.fixture(scope="session")
def cuda():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from sparse_attention_hub_amd import _native

    _native.lib()  # a missing library is an error, not a skip
    return torch.device("cuda:0")
