"""Float fake-cast quantizers (counterpart of aimet_torch.quantization.float)."""

from .encoding import FloatEncoding  # noqa: F401
from .quantizer import FloatQuantizeDequantize, QuantizeDequantize, float_quantize_dequantize  # noqa: F401
