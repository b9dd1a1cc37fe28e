"""Base classes shared by the quantizer modules."""

from aimet_amd.quantization.base.encoding import EncodingBase  # noqa: F401
from aimet_amd.quantization.base.quantizer import QuantizerBase  # noqa: F401
