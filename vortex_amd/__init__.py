"""vortex_amd: MI355X-native (gfx950) Hyena operator hot path behind vortex's own operator API."""
from . import _lib  # noqa: F401
from .ops import (DecodeLayerSet, FirRing, FirStepper, IirStepper, LayerStepper, ModalPlan, fir_step, hyena_li_fwd, hyena_mr_fwd, hyena_se_fwd, iir_step)  # noqa: F401

__all__ = ["hyena_se_fwd", "hyena_mr_fwd", "hyena_li_fwd", "fir_step", "iir_step", "FirRing", "ModalPlan", "FirStepper", "IirStepper", "DecodeLayerSet", "LayerStepper"]
