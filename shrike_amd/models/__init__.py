from . import minilorn, mofarax, qwen2  # noqa: F401  (register Minilorn, Mofarax and Qwen2ForCausalLM)
from .decoder import DecoderModel

__all__ = ["DecoderModel", "minilorn", "mofarax", "qwen2"]
