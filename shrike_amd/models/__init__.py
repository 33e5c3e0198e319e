from . import mofarax, qwen2  # noqa: F401  (register Mofarax and Qwen2ForCausalLM)
from .decoder import DecoderModel

__all__ = ["DecoderModel", "mofarax", "qwen2"]
