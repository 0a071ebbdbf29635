"""`hyena_ops.kernel_utils`: the kernel configuration dataclasses vortex's callers import
(vortex/ops/hyena_se/kernel_utils.py:326-343).  The HIP kernels have fixed tiles; the fields are accepted and ignored."""
from .interface import BwdKernelConfig, FwdKernelConfig  # noqa: F401

__all__ = ["FwdKernelConfig", "BwdKernelConfig"]
