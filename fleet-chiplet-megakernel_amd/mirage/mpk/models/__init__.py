"""Model graph builders; importing the package registers them (reference: python/mirage/mpk/models/__init__.py)."""
from .graph_builder import GraphBuilder, MirageModelConfig
from .qwen3 import builder as _qwen3_builder  # noqa: F401  (registers Qwen3Builder)

__all__ = ["GraphBuilder", "MirageModelConfig"]
