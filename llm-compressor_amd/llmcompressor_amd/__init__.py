"""MI355X-native calibration-time quantization hot path (GPTQ, observers, packing)."""
__version__ = "0.1.0"
