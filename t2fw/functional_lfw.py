"""Alias module: same import path as the reference's t2fw/functional_lfw.py."""
from t2fw_amd.functional_lfw import LFWFunction, lfw_step  # noqa: F401
