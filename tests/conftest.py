import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def override():
    """override(mr_nseg=4, li_coop=1, ...): pins launch-shape choices of the library (hyena_set_launch_override) so
    that small inputs exercise the multi-segment, non-temporal or cooperative code paths; reset after the test."""
    from vortex_amd import _lib
    used = set()

    def set_(**kv):
        for k, v in kv.items():
            _lib.check(_lib.lib().hyena_set_launch_override(k.encode(), int(v)), "hyena_set_launch_override")
            used.add(k)

    yield set_
    for k in used:
        _lib.lib().hyena_set_launch_override(k.encode(), -1)


@pytest.fixture(autouse=True)
def poisoned_device_buffers(request, monkeypatch):
    """GPU tests: every floating-point tensor that torch.empty / empty_like hands out on the device starts as NaN, so
    an output that a kernel does not write in full cannot pass a comparison on what an earlier call left in the same
    memory (the caching allocator returns a freed block as it is)."""
    if "gpu" not in request.keywords:
        yield
        return
    import torch

    real_empty, real_empty_like = torch.empty, torch.empty_like

    def poison(t):
        if t.is_cuda and t.is_floating_point() and t.numel():
            t.fill_(float("nan"))
        return t

    monkeypatch.setattr(torch, "empty", lambda *a, **k: poison(real_empty(*a, **k)))
    monkeypatch.setattr(torch, "empty_like", lambda *a, **k: poison(real_empty_like(*a, **k)))
    yield
