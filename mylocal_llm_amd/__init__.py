"""MI355X-native packed-weight decode path (drop-in for MyLocal_LLM's packed operators)."""
from .quantized_weight import BLOCK_FORMATS, PackedGGUFWeight  # noqa: F401

__all__ = ["BLOCK_FORMATS", "PackedGGUFWeight"]
