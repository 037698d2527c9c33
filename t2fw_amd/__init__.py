"""MI355X-native kernels for the decaying-fast-weight recurrence (drop-in for T2FW's
``LFWFunction`` / ``DFWFunction`` autograd functions)."""
from .functional_lfw import LFWFunction, lfw_step, DEFAULT_CKPT_INTERVAL  # noqa: F401
from .functional_dfw import DFWFunction  # noqa: F401
from .state_cache import FastWeightState  # noqa: F401

__all__ = ["LFWFunction", "DFWFunction", "FastWeightState", "lfw_step", "DEFAULT_CKPT_INTERVAL"]
