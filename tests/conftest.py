import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, os.path.join(ROOT, "test-burn_amd"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(params=[1, 2, 3], ids=["staged", "lds_direct", "chunk"])
def prefill_variant(request):
    """Runs a GPU test once per prefill kernel variant (fa_set_prefill_variant) and restores the default. 3 = the automatic
    choice with the short-chunk kernel taking every launch it can (at most 64 query rows), whatever the context length."""
    from gpu_util import ctx
    ctx().set_prefill_variant(request.param)
    yield request.param
    ctx().set_prefill_variant(0)
