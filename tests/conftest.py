import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lsa():
    """The product package; the GPU tests call the HIP kernels only through it."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import loongserve_amd
    return loongserve_amd


PREFILL_GEOMETRIES = {
    "library-choice": {},
    "rows128": {"prefill_rows": "128"},
    "rows256-head-major": {"prefill_rows": "256", "prefill_order": "head"},
    "rows256-tile-major": {"prefill_rows": "256", "prefill_order": "tile"},
    "rows256-one-head": {"prefill_rows": "256", "prefill_pack": "off"},
    "rows128-one-head": {"prefill_rows": "128", "prefill_pack": "off"},
    "rows128-four-waves": {"prefill_rows": "half"},
    "rows128-four-waves-one-head": {"prefill_rows": "half", "prefill_pack": "off"},
}


@pytest.fixture
def tuning(lsa):
    """set_tuning of the library for the length of a test: call it with the choices to force; the library's own choices
    come back when the test ends."""
    yield lsa.set_tuning
    lsa.set_tuning()


@pytest.fixture(params=list(PREFILL_GEOMETRIES))
def prefill_geometry(request, tuning):
    """Runs a prefill test once per workgroup shape (128 or 256 query rows; the query heads of a KV head side by side in
    a workgroup, the library's way wherever the group size allows, or one head per workgroup) and grid order (one KV head
    at a time per XCD, or the heaviest query tiles of all KV heads first) of the prefill kernel.  The library picks both from the size
    of the launch; the test shapes alone would leave most combinations to the few large cases."""
    tuning(**PREFILL_GEOMETRIES[request.param])
    return request.param
