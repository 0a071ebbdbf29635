"""ctypes binding of libhyena_mi355x.so (the C ABI declared in include/hyena_mi355x.h).

There is no fallback: if the library is missing, every operator raises.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhyena_mi355x.so")

HYENA_BIAS_NONE, HYENA_BIAS_ADD, HYENA_BIAS_GATED_FP32, HYENA_BIAS_ADD_FP32, HYENA_BIAS_GATED_BF16 = 0, 1, 2, 3, 4
HYENA_DTYPE_BF16, HYENA_DTYPE_F16, HYENA_DTYPE_F32 = 0, 1, 2

EXPORTS = [
    "hyena_version", "hyena_last_error_string", "hyena_se_fwd", "hyena_mr_fwd",
    "hyena_fir_step", "hyena_iir_step", "hyena_li_plan_bytes", "hyena_li_plan", "hyena_li_fwd", "hyena_li_layer_fwd", "hyena_fir_layer_fwd_rows", "hyena_li_fwd_static", "hyena_featurizer_fwd", "hyena_set_launch_override",
    "hyena_fir_layer_step", "hyena_iir_layer_step", "hyena_fir_cl_fwd", "hyena_fir_cl_fwd_dtype", "hyena_fir_layer_fwd",
    "hyena_featurizer_gates_fwd",
    "hyena_fir_step_dpos", "hyena_fir_layer_step_dpos", "hyena_ring_advance",
    "hyena_fir_far_period", "hyena_fir_far_bytes", "hyena_fir_step_far", "hyena_fir_layer_step_far",
    "hyena_iir_window_tokens", "hyena_iir_window_supported", "hyena_iir_step_win", "hyena_iir_layer_step_win",
    "hyena_iir_window_flush",
]


class Rows(Structure):
    _fields_ = [("ptr", c_void_p), ("batch_stride", c_int64), ("row_stride", c_int64),
                ("ch_inner", c_int64), ("ch_outer", c_int64)]


class ProjStep(Structure):
    """hyena_proj_step: the featurizer decode step a layer step evaluates on the fly."""
    _fields_ = [("u", c_void_p), ("u_batch_stride", c_int64), ("ring", c_void_p), ("Rf", c_int64), ("pos", c_int64),
                ("w", c_void_p), ("bias", c_void_p), ("ch_inner", c_int64), ("ch_outer", c_int64),
                ("gate_stride", c_int64), ("ch_stride", c_int64), ("flip_x1x2", c_int), ("pos_dev", c_void_p)]


class IirWindow(Structure):
    """hyena_iir_window: the buffers and counters of the windowed modal step."""
    _fields_ = [("hist", c_void_p), ("far", c_void_p), ("g", c_void_p), ("cnt", c_int64), ("cnt_dev", c_void_p),
                ("warm", c_int), ("reserved", c_int)]


class Cl(Structure):
    """hyena_cl: a channel-last [B, L, D] operand."""
    _fields_ = [("ptr", c_void_p), ("batch_stride", c_int64), ("time_stride", c_int64)]


class ProjFwd(Structure):
    """hyena_proj_fwd: the featurizer a fused prefill layer evaluates on the fly."""
    _fields_ = [("u", c_void_p), ("u_batch_stride", c_int64), ("u_time_stride", c_int64), ("w", c_void_p),
                ("bias", c_void_p), ("Ks", c_int), ("flip_x1x2", c_int), ("ch_inner", c_int64), ("ch_outer", c_int64),
                ("gate_stride", c_int64), ("ch_stride", c_int64)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `python -m vortex_amd.build` (hipcc, gfx950). "
            "There is no CPU or PyTorch fallback for the Hyena kernels.")
    L = ctypes.CDLL(LIB_PATH)
    L.hyena_version.restype = c_char_p
    L.hyena_last_error_string.restype = c_char_p
    R = POINTER(Rows)
    L.hyena_se_fwd.argtypes = [R, R, R, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_int64,
                               c_int, c_void_p]
    L.hyena_mr_fwd.argtypes = [R, R, R, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64,
                               c_int64, c_int, c_void_p]
    L.hyena_fir_step.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                 c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]
    L.hyena_iir_step.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                                 c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64,
                                 c_void_p]
    L.hyena_li_plan_bytes.argtypes = [c_int64, c_int64]
    L.hyena_li_plan.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]
    L.hyena_li_fwd.argtypes = [R, R, R, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                               c_int64, c_int64, c_int64, c_void_p]
    L.hyena_fir_layer_fwd_rows.argtypes = [R, R, R, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64,
                                           c_int64, c_int64, c_int64, c_int, c_void_p]
    L.hyena_li_layer_fwd.argtypes = [R, R, R, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int64,
                                     c_int64, c_int64, c_int64, c_int64, c_void_p]
    L.hyena_li_fwd_static.argtypes = [R, R, R, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64,
                                      c_int64, c_int64, c_int64, c_int64, c_void_p]
    L.hyena_featurizer_fwd.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_int64,
                                       c_int64, c_int64, c_int64, c_int, c_int, c_void_p]
    L.hyena_set_launch_override.argtypes = [c_char_p, c_int64]
    P = POINTER(ProjStep)
    L.hyena_fir_layer_step.argtypes = [P, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_int64,
                                       c_int64, c_int64, c_int64, c_void_p]
    L.hyena_iir_layer_step.argtypes = [P, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                       c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p]
    L.hyena_fir_step_dpos.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]
    L.hyena_fir_layer_step_dpos.argtypes = [P, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                            c_int64, c_int64, c_int64, c_int64, c_void_p]
    L.hyena_ring_advance.argtypes = [c_void_p, c_void_p, c_int64, c_void_p]
    WN = POINTER(IirWindow)
    L.hyena_iir_window_tokens.argtypes = []
    L.hyena_iir_window_supported.argtypes = [c_int64, c_int64, c_int64, c_int]
    L.hyena_iir_step_win.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                                     c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64,
                                     WN, c_void_p]
    L.hyena_iir_layer_step_win.argtypes = [P, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                           c_int64, c_int64, c_int64, c_int64, c_int64, WN, c_void_p]
    L.hyena_iir_window_flush.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, WN,
                                         c_void_p]
    L.hyena_fir_far_period.argtypes = [c_int64]
    L.hyena_fir_far_bytes.argtypes = [c_int64, c_int64]
    L.hyena_fir_step_far.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                     c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64,
                                     c_int64, c_void_p]
    L.hyena_fir_layer_step_far.argtypes = [P, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p,
                                           c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]
    C = POINTER(Cl)
    L.hyena_fir_cl_fwd.argtypes = [C, C, C, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64,
                                   c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]
    L.hyena_fir_cl_fwd_dtype.argtypes = [C, C, C, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64,
                                         c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p]
    L.hyena_featurizer_gates_fwd.argtypes = [POINTER(ProjFwd), c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]
    L.hyena_fir_layer_fwd.argtypes = [POINTER(ProjFwd), c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int64,
                                      c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]
    for name in EXPORTS:
        fn = getattr(L, name)
        if name not in ("hyena_version", "hyena_last_error_string"):
            fn.restype = c_int64 if name in ("hyena_li_plan_bytes", "hyena_fir_far_period", "hyena_fir_far_bytes", "hyena_iir_window_tokens") else c_int
    _lib = L
    return L


class launch_override:
    """Context manager pinning one launch-shape choice of the library (hyena_set_launch_override) for its body.

    Tests use it to force the multi-segment, non-temporal or cooperative code paths on small inputs."""

    def __init__(self, **kv):
        self.kv = kv

    def __enter__(self):
        for k, v in self.kv.items():
            check(lib().hyena_set_launch_override(k.encode(), int(v)), "hyena_set_launch_override")
        return self

    def __exit__(self, *exc):
        for k in self.kv:
            lib().hyena_set_launch_override(k.encode(), -1)
        return False


_probe = None
PROBE_PATH = os.path.join(_HERE, "libhyena_probe.so")


def copy_probe():
    """hyena_copy_probe(src, dst, nbytes, stream) of libhyena_probe.so: a plain 16-bytes-per-lane device copy, the
    calibration launch for traffic counters and the bandwidth yardstick of the benchmark (not an operator)."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_PATH):
            raise RuntimeError(f"{PROBE_PATH} is not built; run `python -m vortex_amd.build`")
        P = ctypes.CDLL(PROBE_PATH)
        P.hyena_copy_probe.argtypes = [c_void_p, c_void_p, c_int64, c_void_p]
        P.hyena_copy_probe.restype = c_int
        _probe = P
    return _probe.hyena_copy_probe


def check(rc, what):
    """Turns a non-zero return code into the exception TORCH_CHECK would have raised."""
    if rc == 0:
        return
    msg = lib().hyena_last_error_string().decode()
    if rc == -3:
        raise NotImplementedError(msg or what)
    if rc < 0:
        raise ValueError(msg or what)
    raise RuntimeError(msg or f"{what}: hipError {rc}")
