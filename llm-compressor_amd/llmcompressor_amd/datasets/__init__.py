from .utils import (
    DataCollatorWithTruncation,
    LengthAwareSampler,
    format_calibration_data,
    get_calibration_dataloader,
)

__all__ = ["get_calibration_dataloader", "format_calibration_data", "DataCollatorWithTruncation",
           "LengthAwareSampler"]
