from .moe import (ExpertMLP, LinearExperts2D, get_non_linearized_moes, linearize_moe,  # noqa: F401
                  moe_calibration_context)
