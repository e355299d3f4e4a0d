from . import kofipel, qwen3, rupezen   # noqa: F401  (registers the architecture)
from .decoder import Decoder

__all__ = ["Decoder"]
