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
    "rows128": {"LSATTN_PREFILL_ROWS": "128"},
    "rows256-head-major": {"LSATTN_PREFILL_ROWS": "256", "LSATTN_PREFILL_ORDER": "head"},
    "rows256-tile-major": {"LSATTN_PREFILL_ROWS": "256", "LSATTN_PREFILL_ORDER": "tile"},
    "rows256-one-head": {"LSATTN_PREFILL_ROWS": "256", "LSATTN_PREFILL_PACK": "0"},
    "rows128-one-head": {"LSATTN_PREFILL_ROWS": "128", "LSATTN_PREFILL_PACK": "0"},
    "rows128-four-waves": {"LSATTN_PREFILL_ROWS": "half"},
    "rows128-four-waves-one-head": {"LSATTN_PREFILL_ROWS": "half", "LSATTN_PREFILL_PACK": "0"},
}


@pytest.fixture(params=list(PREFILL_GEOMETRIES))
def prefill_geometry(request, monkeypatch):
    """Runs a prefill test once per workgroup shape (128 or 256 query rows; the query heads of a KV head side by side in
    a workgroup, the library's way wherever the group size allows, or one head per workgroup) and grid order (one KV head
    at a time per XCD, or the heaviest query tiles of all KV heads first) of the prefill kernel.  The library picks both from the size
    of the launch; the test shapes alone would leave most combinations to the few large cases."""
    for name in ("LSATTN_PREFILL_ROWS", "LSATTN_PREFILL_ORDER", "LSATTN_PREFILL_PACK"):
        monkeypatch.delenv(name, raising=False)
    for name, value in PREFILL_GEOMETRIES[request.param].items():
        monkeypatch.setenv(name, value)
    return request.param
