import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "slow: long-running parity sweep")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(params=["literal_for_small_tensors", "table_on_the_quotient", "table_always"])
def codec_form(request):
    """Compression has three encoders that must give the same bits: the literal procedure per element for small
    tensors, the fixed table on the quotient x / precision for mid-size ones and the table built for the call's
    precision for the largest.  Tests that use this fixture run once with the library's own choice by size and once
    with each table forced for every size, so the small adversarial inputs exercise all three."""
    from clusternet_amd import _lib as L
    L.lib().cn_host_codec_encoder({"literal_for_small_tensors": 0, "table_on_the_quotient": 2, "table_always": 3}[request.param])
    yield request.param
    L.lib().cn_host_codec_encoder(0)  # back to the library's own choice
