"""aimet_amd.quantization: MI355X-native counterpart of aimet_torch.quantization for the fake-quant hot path."""

from aimet_amd.quantization.affine.backends.utils import set_backend, get_backend, add_backend  # noqa: F401
from aimet_amd.quantization import affine  # noqa: F401
