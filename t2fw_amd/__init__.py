"""MI355X-native kernels for the decaying-fast-weight recurrence (drop-in for T2FW's
``LFWFunction`` / ``DFWFunction`` autograd functions)."""
from .functional_lfw import (LFWFunction, LFWGatedFunction, LFWHeadsFunction, sigmoid_gates, lfw_step,  # noqa: F401
                             lfw_apply_16bit, lfw_apply_padded, DEFAULT_CKPT_INTERVAL)
from .functional_dfw import DFWFunction  # noqa: F401
from .state_cache import FastWeightState  # noqa: F401

__all__ = ["LFWFunction", "LFWGatedFunction", "LFWHeadsFunction", "DFWFunction", "FastWeightState", "sigmoid_gates", "lfw_step", "lfw_apply_16bit", "lfw_apply_padded",
           "DEFAULT_CKPT_INTERVAL"]
