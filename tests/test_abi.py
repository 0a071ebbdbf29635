"""The C-ABI library loads and exports every symbol include/hyena_mi355x.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    src = open(os.path.join(ROOT, "include", "hyena_mi355x.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(hyena_[a-z0-9_]+)\s*\(", src)))


def test_header_symbols_exported():
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 6
    for n in names:
        assert hasattr(L, n), n
    assert set(_lib.EXPORTS) == set(names)
    assert b"gfx950" in _lib.lib().hyena_version()


def test_argument_errors_are_reported_without_a_gpu():
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = _lib.lib()
    rc = L.hyena_se_fwd(None, None, None, None, None, 0, None, 1, 16, 8, 1, 7, None)
    assert rc == -1 and b"required" in L.hyena_last_error_string()
    with pytest.raises(ValueError):
        _lib.check(rc, "hyena_se_fwd")


def test_cpu_tensors_are_rejected():
    import torch
    import vortex_amd as va
    x = torch.zeros(1, 16, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        va.hyena_se_fwd(x, x, x, torch.zeros(1, 1, 7))
