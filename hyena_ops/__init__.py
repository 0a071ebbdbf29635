"""`hyena_ops`: the import name vortex uses for its Hyena operator package
(vortex/ops/conv/setup.py:56-64, vortex/model/layers.py:18-21), provided here by the
gfx950 kernels of vortex_amd.

    from hyena_ops import hyena_se_fwd, hyena_mr_fwd, hyena_li_fwd
"""
from vortex_amd.ops import hyena_li_fwd, hyena_mr_fwd, hyena_se_fwd  # noqa: F401

from . import interface, kernel_utils, utils  # noqa: F401

__all__ = ["hyena_se_fwd", "hyena_mr_fwd", "hyena_li_fwd", "interface", "kernel_utils", "utils"]
