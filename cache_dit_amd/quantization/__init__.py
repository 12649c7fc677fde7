from .backend import QuantizeBackend
from .config import QuantizeConfig
from .dispatch import load
from .dispatch import quantize
from .dispatch import remove_quantization_stats

__all__ = ["QuantizeBackend", "QuantizeConfig", "load", "quantize", "remove_quantization_stats"]
