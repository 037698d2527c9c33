"""Alias module: same import path as the reference's t2fw/functional_dfw.py."""
from t2fw_amd.functional_dfw import DFWFunction  # noqa: F401
