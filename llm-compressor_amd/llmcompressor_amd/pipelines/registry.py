"""``from llmcompressor.pipelines.registry import CalibrationPipeline`` (reference: pipelines/registry.py)."""
from . import CalibrationPipeline  # noqa: F401

__all__ = ["CalibrationPipeline"]
