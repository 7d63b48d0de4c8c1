import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_lib():
    import oracle
    return oracle.load()


@pytest.fixture(scope="session")
def ref_lib():
    """The reference's own sources compiled in place, or None where they were
    not built (the GPU box has no reference tree)."""
    import oracle
    return oracle.load_ref()


@pytest.fixture(params=["by_size", "streaming", "streaming_4x4x1", "tiled"])
def linear_kernel_choice(request):
    """A Linear layer goes to the one-launch kernel for small layers, to the streaming
    kernels (up to 32 samples) or to the tiled kernel depending on the size of its
    weight matrix. "by_size" leaves that choice as shipped; "streaming" sends every
    layer whose batch fits to the streaming kernels and "tiled" every layer to the
    tiled kernel, so that the small test shapes reach each of them. The streaming forward
    is the 16-wide kernel for every batch as shipped; "streaming_4x4x1" sends the forward
    to the 4x4x1 kernels the library keeps for up to 16 samples."""
    from cutagi_amd import capi
    if request.param in ("streaming", "streaming_4x4x1"):
        capi.tune("linear.stream_min_weights", 0)
        if request.param == "streaming_4x4x1":
            capi.tune("linear.gemv16.min_batch", 33)
    elif request.param == "tiled":
        capi.tune("linear.stream_min_weights", 2 ** 31 - 1)
    yield request.param
    capi.tune("linear.stream_min_weights", -1)
    capi.tune("linear.gemv16.min_batch", -1)
