from .builder import Qwen3Builder

__all__ = ["Qwen3Builder"]
