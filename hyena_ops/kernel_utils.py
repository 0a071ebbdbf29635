"""`hyena_ops.kernel_utils`: the kernel configuration records vortex's callers build and pass to the operator
(vortex/ops/hyena_se/kernel_utils.py:282-343).

The reference's Triton kernels are tuned through these fields (chunk size, block width, warps, stages, TMA).
The gfx950 kernels have fixed tiles chosen for the hardware, so every tuning field is accepted, validated the
way the reference validates it, and otherwise ignored; the three RETURN_* flags of the forward record are the
only ones with an effect (they select the by-products `two_pass_fwd_grouped` hands back).
"""
import warnings
from dataclasses import dataclass, fields

_SCHEDULES = ("default", "persistent")
_SWIZZLES = ("row", "col")


@dataclass
class KernelConfig:
    """Common part (kernel_utils.py:282-324).  schedule / CHUNK_SIZE / BLOCK_D / THREADBLOCK_SWIZZLE are required
    by the reference; they have defaults here so that a bare FwdKernelConfig() is also accepted."""
    schedule: str = "default"
    CHUNK_SIZE: int = 128
    BLOCK_D: int = 32
    THREADBLOCK_SWIZZLE: str = "row"
    USE_TMA: bool = False
    FLUSH_TMA: bool = False
    NUM_PIPELINE_STAGES: int = 0
    CHUNK_TILES_PER_PROGRAM: int = 1
    num_warps: int = 4
    num_stages: int = 3
    num_ctas: int = 1
    maxnreg: int = None
    autotune: bool = False          # not a field of the reference record; older callers pass it, so it is taken too

    def __post_init__(self):
        if self.schedule not in _SCHEDULES:
            raise AssertionError(f"schedule must be one of {_SCHEDULES}")
        if self.THREADBLOCK_SWIZZLE not in _SWIZZLES:
            raise AssertionError(f"THREADBLOCK_SWIZZLE must be one of {_SWIZZLES}")
        if not 0 <= self.NUM_PIPELINE_STAGES < 2:
            raise AssertionError("NUM_PIPELINE_STAGES must be 0 or 1")
        if self.schedule == "default" and self.NUM_PIPELINE_STAGES:
            warnings.warn("NUM_PIPELINE_STAGES is reset to 0: the default schedule has no pipeline")
            self.NUM_PIPELINE_STAGES = 0

    def _key(self):
        return tuple(getattr(self, f.name) for f in fields(self))

    def __eq__(self, other):
        return self._key() == other._key() if isinstance(other, KernelConfig) else NotImplemented

    def __hash__(self):
        return hash(self._key())

    def __str__(self):
        return type(self).__name__ + ": " + ", ".join(f"{f.name}={getattr(self, f.name)}" for f in fields(self))


@dataclass(eq=False)
class FwdKernelConfig(KernelConfig):
    """kernel_utils.py:326-335."""
    name: str = "fwd"
    version: str = "v2"
    RETURN_TOEPLITZ: bool = True
    RETURN_Y2: bool = True
    RETURN_BX_LAG: bool = True


@dataclass(eq=False)
class BwdKernelConfig(KernelConfig):
    """kernel_utils.py:337-343; carried for signature compatibility only (this build is forward only)."""
    name: str = "bwd"
    version: str = "v2"
    LOAD_TOEPLITZ: bool = True
    LOAD_BX_LAG: bool = True


__all__ = ["KernelConfig", "FwdKernelConfig", "BwdKernelConfig"]
