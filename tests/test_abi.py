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


def test_new_entry_points_validate_before_touching_the_device():
    # every call below is rejected by the argument checks; the dummy non-null pointers are never dereferenced
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = _lib.lib()
    P = 4096                      # aligned, non-null
    cl = _lib.Cl(P, 64, 64)
    ref = ctypes.byref
    assert L.hyena_fir_cl_fwd(ref(cl), ref(cl), ref(cl), P, 0, None, 0, P, None, None, 0, 1, 8, 64, 4, 200, None) == -3
    assert b"K=200" in L.hyena_last_error_string()
    assert L.hyena_fir_cl_fwd(ref(cl), ref(cl), ref(cl), P, 0, None, 0, P, None, None, 0, 1, 8, 24, 3, 4, None) == -3
    assert L.hyena_fir_cl_fwd(ref(cl), None, ref(cl), P, 0, None, 0, P, None, None, 0, 1, 8, 64, 4, 4, None) == -3
    assert L.hyena_fir_cl_fwd(ref(_lib.Cl(P + 2, 64, 64)), None, None, P, 0, None, 0, P, None, None, 0, 1, 8, 64, 4,
                              4, None) == -2
    assert L.hyena_fir_cl_fwd(ref(cl), None, None, P, 0, None, 2, P, None, None, 0, 1, 8, 64, 4, 4, None) == -1
    pj = _lib.ProjFwd(P, 192, 192, P, None, 5, 0, 64, 0, 64, 1)
    assert L.hyena_fir_layer_fwd(ref(pj), P, 0, None, 0, P, None, 0, 1, 8, 64, 4, 7, None) == -3      # 5-tap featurizer
    pj = _lib.ProjFwd(P, 192, 192, P, None, 3, 0, 64, 0, 80, 1)
    assert L.hyena_fir_layer_fwd(ref(pj), P, 0, None, 0, P, None, 0, 1, 8, 64, 4, 7, None) == -1      # map past 3D
    ps = _lib.ProjStep(P, 192, P, 0, 0, P, None, 64, 0, 64, 1, 0)
    assert L.hyena_fir_layer_step(ref(ps), P, 6, 64, 0, P, None, 0, P, 64, 1, 64, 4, None) == -1          # empty cache
    ps = _lib.ProjStep(P, 192, P, 2, 0, P, None, 4, 12, 4, 1, 0)
    assert L.hyena_fir_layer_step(ref(ps), P, 6, 64, 0, P, None, 0, P, 64, 1, 64, 4, None) == -3          # head_dim 4
    assert L.hyena_iir_layer_step(None, P, P, P, 0, P, 0, P, 0, 64, 1, 64, 64, 16, None) == -1
    # ring positions in device memory: the pointer is required, and a position on the device lifts the host range check
    assert L.hyena_fir_step_dpos(P, None, None, 64, P, 6, 64, None, P, None, 0, P, 64, 1, 64, 4, None) == -1
    assert L.hyena_fir_layer_step_dpos(ref(ps), P, 6, 64, None, P, None, 0, P, 64, 1, 64, 4, None) == -1
    # cache layout: the channel block is D or a multiple of 512 that divides D
    assert L.hyena_fir_step_dpos(P, None, None, 1024, P, 6, 256, P, P, None, 0, P, 1024, 1, 1024, 64, None) == -1
    assert L.hyena_fir_step_dpos(P, None, None, 1536, P, 6, 1024, P, P, None, 0, P, 1536, 1, 1536, 96, None) == -1
    assert L.hyena_fir_step_dpos(P, None, None, 1536, P, 6, 512, P, P, None, 0, P, 1536, 0, 1536, 96, None) == 0
    # far-sum FIR step: deep caches only, the far buffer is required, the counter runs to lcm(window, R)
    per = L.hyena_fir_far_period(127)
    assert per % 127 == 0 and per // 127 == L.hyena_fir_far_period(1) and L.hyena_fir_far_period(0) == 0
    assert L.hyena_fir_far_bytes(64, 4096) == 64 * L.hyena_fir_far_period(1) * 4096 * 4
    assert L.hyena_fir_step_far(P, None, None, 512, P, 127, 512, 0, None, None, 0, P, None, 0, P, 512, 1, 512, 32, None) == -1
    assert L.hyena_fir_step_far(P, None, None, 512, P, 6, 512, 0, None, P, 0, P, None, 0, P, 512, 1, 512, 32, None) == -3
    assert L.hyena_fir_step_far(P, None, None, 512, P, 127, 512, per, None, P, 0, P, None, 0, P, 512, 1, 512, 32, None) == -1
    assert L.hyena_fir_step_far(P, None, None, 512, P, 127, 512, per - 1, None, P, 1, P, None, 0, P, 512, 0, 512, 32, None) == 0
    assert L.hyena_fir_layer_step_far(None, P, 127, 512, 0, None, P, 0, P, None, 0, P, 512, 1, 512, 32, None) == -1
    # gate-fused featurizer: descriptor checks as in the layer call, both outputs, column count a multiple of 8
    pj = _lib.ProjFwd(P, 192, 192, P, None, 3, 0, 64, 0, 64, 1)
    assert L.hyena_featurizer_gates_fwd(None, P, P, 8, 1, 8, 64, 0, None) == -1
    assert L.hyena_featurizer_gates_fwd(ref(pj), P, None, 8, 1, 8, 64, 0, None) == -1
    assert L.hyena_featurizer_gates_fwd(ref(pj), P, P, 8, 1, 5, 64, 0, None) == -2     # 5 columns
    assert L.hyena_featurizer_gates_fwd(ref(pj), P, P, 16, 1, 5, 64, 8, None) == -1    # front_pad above 7
    assert L.hyena_featurizer_gates_fwd(ref(pj), P, P, 8, 0, 5, 64, 3, None) == 0      # B = 0: no launch
    assert L.hyena_featurizer_gates_fwd(ref(pj), P, P, 8, 1, 16, 64, 0, None) == -1    # rows 8 apart for 16 columns
    assert L.hyena_featurizer_gates_fwd(ref(pj), P, P, 20, 1, 16, 64, 0, None) == -2   # row stride not a multiple of 8
    pj5 = _lib.ProjFwd(P, 192, 192, P, None, 5, 0, 64, 0, 64, 1)
    assert L.hyena_featurizer_gates_fwd(ref(pj5), P, P, 8, 1, 8, 64, 0, None) == -3    # 5-tap featurizer
    pjs = _lib.ProjFwd(P, 192, 192, P, None, 3, 0, 4, 12, 4, 1)
    assert L.hyena_featurizer_gates_fwd(ref(pjs), P, P, 8, 1, 8, 64, 0, None) == -3    # heads of 4 channels: no 16-byte pieces
    # windowed modal step: 16 states and B*D of 65536 and more, all three window buffers, the counter inside the window
    W = L.hyena_iir_window_tokens()
    assert W >= 2 and L.hyena_iir_window_supported(64, 4096, 16, 0) == 1 and L.hyena_iir_window_supported(64, 4096, 16, 1) == 1
    assert L.hyena_iir_window_supported(64, 4096, 8, 0) == 0 and L.hyena_iir_window_supported(8, 4096, 16, 0) == 0
    assert L.hyena_iir_window_supported(64, 4100, 16, 0) == 0
    iw = lambda *a: ref(_lib.IirWindow(*a))
    win_args = lambda w, B=64, D=4096, S=16: (P, P, P, D, P, P, P, 0, P, 0, P, 0, D, B, D, D, S, w, None)
    assert L.hyena_iir_step_win(*win_args(None)) == -1
    assert L.hyena_iir_step_win(*win_args(iw(P, None, P, 0, None, 0, 0))) == -1          # no far buffer
    assert L.hyena_iir_step_win(*win_args(iw(P, P, P, W, None, 0, 0))) == -1             # counter past the window
    assert L.hyena_iir_step_win(*win_args(iw(P, P, P, 0, None, -1, 0))) == -1            # warm below zero
    assert L.hyena_iir_step_win(*win_args(iw(P, P, P, 0, None, 0, 0), S=8)) == -3
    assert L.hyena_iir_step_win(*win_args(iw(P, P, P, 0, None, 0, 0), B=4)) == -3
    assert L.hyena_iir_layer_step_win(None, P, P, P, 0, P, 0, P, 0, 64, 64, 4096, 4096, 16, iw(P, P, P, 0, None, 0, 0),
                                      None) == -1
    assert L.hyena_iir_window_flush(P, P, P, 0, 64, 4096, 4096, 16, None, None) == -1
    assert L.hyena_iir_window_flush(P, P, P, 0, 64, 4096, 4096, 16, iw(None, None, None, 0, None, 1, 0), None) == -1
    assert L.hyena_ring_advance(None, P, 4, None) == -1 and L.hyena_ring_advance(P, P, -1, None) == -1
    assert L.hyena_ring_advance(P, P, 0, None) == 0
    ps = _lib.ProjStep(P, 192, P, 2, 5, P, None, 64, 0, 64, 1, 0, None)
    assert L.hyena_fir_layer_step(ref(ps), P, 6, 64, 0, P, None, 0, P, 64, 0, 64, 4, None) == -1           # pos 5 of 2
    ps = _lib.ProjStep(P, 192, P, 2, 5, P, None, 64, 0, 64, 1, 0, P)
    assert L.hyena_fir_layer_step(ref(ps), P, 6, 64, 0, P, None, 0, P, 64, 0, 64, 4, None) == 0            # B = 0: no launch
    # modal state sizes
    assert L.hyena_li_plan_bytes(4, 16) == L.hyena_li_plan_bytes(4, 2) == 4 * 1536 * 4
    assert L.hyena_li_plan_bytes(4, 17) == 0 and L.hyena_li_plan_bytes(4, 0) == 0
    assert L.hyena_iir_step(P, P, P, 64, P, P, P, 0, P, 0, P, 0, 64, 1, 64, 64, 12, None) == -3          # not a power of two
    assert L.hyena_iir_step(P, P, P, 64, P, P, P, 0, P, 0, P, 0, 64, 0, 64, 64, 2, None) == 0            # B = 0


def test_missing_library_fails_loudly(monkeypatch):
    # no CPU or PyTorch fallback: without the built library every operator raises
    from vortex_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libhyena_mi355x.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_fused_layer_tail_limit_is_checked_before_launch():
    # with the featurizer fused in, bx_out is the cache tail: more than K-1 rows is refused
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = _lib.lib()
    P = 4096
    pj = _lib.ProjFwd(P, 192, 192, P, None, 3, 0, 64, 0, 64, 1)
    assert L.hyena_fir_layer_fwd(ctypes.byref(pj), P, 0, None, 0, P, P, 100, 1, 200, 64, 4, 7, None) == -3
    assert b"cache tail" in L.hyena_last_error_string()


def test_bad_row_descriptors_are_rejected_by_every_prefill_entry_point():
    # a channel map that would divide by zero or wrap in the kernels' 32-bit arithmetic is an argument error
    # (no launch): ch_inner = 0, ch_inner >= 2^31, negative ch_outer, B*D >= 2^31
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = _lib.lib()
    P = 4096
    ref = ctypes.byref
    good = _lib.Rows(P, 64 * 16, 64, 16, 16)
    bad = [_lib.Rows(P, 64 * 16, 64, 0, 16), _lib.Rows(P, 64 * 16, 64, 1 << 32, 16), _lib.Rows(P, 64 * 16, 64, 16, -3)]
    for r in bad:
        for args in ((r, good, good), (good, r, good), (good, good, r)):
            x1, x2, v = (ref(a) for a in args)
            assert L.hyena_se_fwd(x1, x2, v, P, None, 0, P, 1, 16, 64, 1, 7, None) == -1
            assert L.hyena_mr_fwd(x1, x2, v, P, 0, None, 0, P, 1, 16, 64, 1, 128, None) == -1
            assert b"channel map" in L.hyena_last_error_string()
            assert L.hyena_li_fwd(x1, x2, v, P, None, 1, P, None, None, 1, 16, 64, 1, 16, None) == -1
            assert b"channel map" in L.hyena_last_error_string()
    g = ref(good)
    assert L.hyena_mr_fwd(g, g, g, P, 0, None, 0, P, 1 << 20, 1 << 12, 64, 1, 128, None) == -1
    assert L.hyena_li_fwd(g, g, g, P, None, 1, P, None, None, 1 << 20, 1 << 12, 64, 1, 16, None) == -1


def test_li_row_length_limit_is_checked_before_launch():
    # the long-convolution kernel addresses a row with 32-bit byte offsets: rows beyond 2^30 - 2^16 samples are refused
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = _lib.lib()
    P = 4096
    big = (1 << 30) - (1 << 16) + 8
    g = ctypes.byref(_lib.Rows(P, 16 * big, big, 16, 16))
    assert L.hyena_li_fwd(g, g, g, P, None, 1, P, None, None, 1, 16, big, 1, 16, None) == -3
    assert b"2^30" in L.hyena_last_error_string()
    taps = P
    assert L.hyena_li_layer_fwd(g, g, g, taps, 3, P, None, 1, P, None, 1, 16, big, 1, 16, None) == -3


def test_launch_override_names():
    from vortex_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built in this tree")
    L = _lib.lib()
    for n in (b"mr_nseg", b"cl_nseg", b"li_xcd", b"se_nt", b"mr_nt", b"li_nt", b"cl_nt", b"li_cpw", b"li_coop"):
        assert L.hyena_set_launch_override(n, 1) == 0 and L.hyena_set_launch_override(n, -1) == 0
    assert L.hyena_set_launch_override(b"HYENA_MR_NSEG", 1) == -1
    assert L.hyena_set_launch_override(None, 1) == -1
