from .moe import (ExpertMLP, LinearExperts2D, Llama4LinearExperts, get_non_linearized_moes,  # noqa: F401
                  linearize_moe, moe_calibration_context)
