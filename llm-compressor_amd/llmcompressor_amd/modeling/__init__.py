from .moe import ExpertMLP, LinearExperts2D, moe_calibration_context  # noqa: F401
