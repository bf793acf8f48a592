"""Save-time integration with transformers models (reference: src/llmcompressor/transformers/)."""
