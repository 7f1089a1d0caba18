from . import dedelorn, kegozen, qwen2, tilivik, tosisun  # noqa: F401  (register the architectures)
from .model import DecoderModel, expected_weights

__all__ = ["DecoderModel", "expected_weights", "dedelorn", "kegozen", "qwen2", "tilivik", "tosisun"]
