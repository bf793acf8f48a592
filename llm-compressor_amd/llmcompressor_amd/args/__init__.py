"""The arguments of ``oneshot`` that this path reads, as one typed record (reference: args/dataset_arguments.py).

``oneshot`` takes them as keyword arguments; ``DatasetArguments`` names them with the reference's defaults for
callers that build a pipeline call themselves (``pipeline(model, dataloader, dataset_args)``)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, List, Optional, Union

__all__ = ["DatasetArguments"]


@dataclass
class DatasetArguments:
    dataset: Any = None
    splits: Union[None, str, list, dict] = None
    text_column: str = "text"
    remove_columns: Union[None, str, List[str]] = None
    preprocessing_func: Optional[Callable] = None
    batch_size: int = 1
    data_collator: Union[str, Callable] = "truncation"
    max_seq_length: Optional[int] = None
    num_calibration_samples: Optional[int] = 512
    shuffle_calibration_samples: bool = True
    pad_to_max_length: bool = True
    dataloader_num_workers: int = 0
    moe_calibrate_all_experts: bool = True
    moe_grouped_calibration: bool = False  # this build's own: grouped expert launches in observed passes too
    pipeline: Optional[str] = "independent"
    propagate_error: bool = True  # sequential pipeline: feed the next layer the compressed layer's outputs
    sequential_targets: Optional[List[str]] = None
    sequential_targets_per_subgraph: int = 1
    sequential_offload_device: Optional[str] = None  # None: activations stay in HBM (the reference defaults to "cpu")
    tracing_ignore: List[str] = field(default_factory=list)
