"""MI355X-native quantized weight-matmul path for jitLLM (Q8_0 / Q4_0 / Q4_K)."""
from .ggml import GGMLType  # noqa: F401

__all__ = ["GGMLType"]
