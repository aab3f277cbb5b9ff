"""v2 float quantizers (aimet_torch/v2/quantization/float/__init__.py)."""
from .encoding import FloatEncoding
from .quantizer import FloatQuantizeDequantize, QuantizeDequantize

__all__ = ['FloatEncoding', 'FloatQuantizeDequantize', 'QuantizeDequantize']
