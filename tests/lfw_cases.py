"""Input generators of the LFW tests: the package's synthetic-input module."""
from t2fw_amd.synthetic import (err_stats, make_config_inputs, make_reference_test_inputs,  # noqa: F401
                                reference_shape_grid, uniform_gate_logits)
