import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with `-m gpu` on the GPU box)")


@pytest.fixture
def key_tiles():
    """Every attention call runs key tiles: a decoder step of up to four rows a KV head has a kernel of its own
    (tests/test_gpu_decode.py), and the modules that pin the tile kernel's program (its splits, its grouped tiles,
    its cache reads) against the tile program's restatement keep their small cases on it."""
    import svod_amd

    svod_amd.tune_decode(0)
    yield
    svod_amd.tune_decode(svod_amd.DECODE_ROWS_DEFAULT)


@pytest.fixture(scope="session")
def device():
    """cuda:0 on a box whose device has kernels; the GPU tests fail, not skip, when the
    library is missing or does not recognise the device."""
    import torch

    import svod_amd

    assert torch.cuda.is_available(), "the gpu-marked tests need a GPU"
    svod_amd.load_library()
    assert svod_amd.supported(), "the current device is not a gfx950 this library has kernels for"
    # Outputs the harness allocates start as NaN: an element a kernel leaves unwritten fails its comparison.
    import svod_amd.ops

    svod_amd.ops.POISON = True
    return torch.device("cuda:0")
