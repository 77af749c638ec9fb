from . import fefulorn, kofipel, qwen3, rupezen, safilorn   # noqa: F401  (registers the architecture)
from .decoder import Decoder

__all__ = ["Decoder"]
