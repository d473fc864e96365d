from . import ligipel, minilorn, mofarax, poresun, qwen2  # noqa: F401  (register Ligipel, Minilorn, Mofarax, Poresun and Qwen2ForCausalLM)
from .decoder import DecoderModel

__all__ = ["DecoderModel", "ligipel", "minilorn", "mofarax", "poresun", "qwen2"]
