from . import ligipel, minilorn, mofarax, qwen2  # noqa: F401  (register Ligipel, Minilorn, Mofarax and Qwen2ForCausalLM)
from .decoder import DecoderModel

__all__ = ["DecoderModel", "ligipel", "minilorn", "mofarax", "qwen2"]
