from . import qwen3   # noqa: F401  (registers the architecture)
from .decoder import Decoder

__all__ = ["Decoder"]
