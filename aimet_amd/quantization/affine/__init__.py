"""Affine quantization: functional API, backend registry and quantizer modules."""

from aimet_amd.quantization.affine.backends import (  # noqa: F401
    quantize,
    quantize_dequantize,
    dequantize,
    set_backend,
    get_backend,
    add_backend,
)
