"""Per-module compression log line: time, error, peak device memory (reference: utils/metric_logging.py:18-64)."""
from __future__ import annotations

import logging
import time

import torch

logger = logging.getLogger("llmcompressor_amd")
METRIC = 25
logging.addLevelName(METRIC, "METRIC")

__all__ = ["CompressionLogger", "METRIC"]


class CompressionLogger:
    def __init__(self, module: torch.nn.Module):
        self.module = module
        self.start_tick = None
        self.loss = None
        self.name = None

    def set_results(self, name: str, loss: float):
        self.name, self.loss = name, loss

    def __enter__(self):
        self.start_tick = time.time()
        return self

    def __exit__(self, _exc_type, _exc_val, _exc_tb):
        dt = time.time() - self.start_tick
        logger.log(METRIC, f"time {dt:.2f}s")
        if self.loss is not None:
            logger.log(METRIC, f"error {self.loss:.2f}")
        if torch.cuda.is_available():
            logger.log(METRIC, f"peak device memory {torch.cuda.max_memory_allocated() / 2**30:.2f} GiB")
