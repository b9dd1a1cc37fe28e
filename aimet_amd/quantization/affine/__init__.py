"""Affine quantization: functional API, backend registry and quantizer modules."""

from aimet_amd.quantization.affine.backends import (  # noqa: F401
    quantize,
    quantize_dequantize,
    dequantize,
    set_backend,
    get_backend,
    add_backend,
)
from aimet_amd.quantization.affine.encoding import AffineEncoding, GroupedBlockEncoding, VectorEncoding  # noqa: F401,E402
from aimet_amd.quantization.affine.quantizer import (  # noqa: F401,E402
    AffineQuantizerBase,
    MinMaxQuantizer,
    ScaleOffsetQuantizer,
    Quantize,
    QuantizeDequantize,
    Dequantize,
    GroupedBlockQuantizeDequantize,
)
