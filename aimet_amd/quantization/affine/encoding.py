"""Affine encodings: the (scale, offset, grid) description attached to quantizer outputs.

Counterpart of aimet_torch/quantization/affine/encoding.py:33-740, including the export of an encoding to the
dictionary formats "0.6.1", "1.0.0", "2.0.0" and "2.1.0" (`to_qnn_encoding_dict`), the way back from a per-tensor
2.0.0 / 2.1.0 dictionary, the vector-quantization encoding (a record of its extra fields) and the reading of a
blockwise encoding as a grouped one.
"""

from __future__ import annotations

import math
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from aimet_amd.quantization.base.encoding import EncodingBase
from aimet_amd.quantization.affine._utils import _GridMixin
from aimet_amd.quantization.affine.backends import quantize, dequantize, quantize_dequantize, _derive_qmin_qmax

__all__ = ["AffineEncoding", "VectorEncoding", "GroupedBlockEncoding"]


class AffineEncoding(EncodingBase, _GridMixin):
    """AffineEncoding(scale, offset, qmin, qmax, symmetry=False, block_size=None, zero_point_shift=None) or
    AffineEncoding(scale, offset, bitwidth, signed=False, symmetry=False, block_size=None, zero_point_shift=None)."""

    def __init__(self, scale: torch.Tensor, offset: torch.Tensor, *args, **kwargs):
        self.scale = scale
        self.offset = offset
        self._input_shape_hint = None
        pos = tuple(args) + (None,) * (5 - len(args))
        first = kwargs.pop("qmin", kwargs.pop("bitwidth", pos[0]))
        second = kwargs.pop("qmax", kwargs.pop("signed", pos[1]))
        symmetry = kwargs.pop("symmetry", pos[2])
        block_size = kwargs.pop("block_size", pos[3])
        zero_point_shift = kwargs.pop("zero_point_shift", pos[4])
        self.producer = kwargs.pop("producer", None)
        if kwargs:
            raise TypeError(f"{type(self).__qualname__}.__init__ got unexpected keyword argument: {', '.join(kwargs)}")
        if first is None:
            raise TypeError("expected (qmin, qmax) or (bitwidth[, signed]) after scale and offset")
        if second is None or isinstance(second, bool):
            qmin, qmax = _derive_qmin_qmax(bitwidth=first, signed=bool(second))
        else:
            qmin, qmax = first, second
        if qmin >= qmax:
            raise ValueError(f"qmax should be strictly larger than qmin. Got qmax={qmax}, qmin={qmin}")
        self.qmin = qmin
        self.qmax = qmax
        self._symmetry = bool(symmetry)
        self.block_size = block_size
        self._zero_point_shift = zero_point_shift or 0.0
        if self._zero_point_shift not in (0.0, 0.5):
            raise ValueError(f"zero_point_shift should be 0.0 or 0.5. Got {self._zero_point_shift}")

    @property
    def mapping(self) -> str:
        return "affine"

    @property
    def granularity(self) -> str:
        if self.scale.dim() == 0:
            return "pertensor"
        if self.block_size is not None:
            return "blockwise"
        non_singleton = [d for d in self.scale.shape if d > 1]
        if len(non_singleton) <= 1:
            return "perchannel"
        return "unknown"

    @property
    def num_steps(self) -> int:
        return self.qmax - self.qmin

    @property
    def min(self) -> torch.Tensor:
        return (self.offset + self.qmin) * self.scale

    @property
    def max(self) -> torch.Tensor:
        return (self.offset + self.qmax) * self.scale

    @property
    def symmetry(self) -> bool:
        return self._symmetry

    @property
    def zero_point_shift(self) -> float:
        return self._zero_point_shift

    @property
    def bitwidth(self) -> int:
        return self._get_bitwidth()

    @property
    def signed(self) -> bool:
        return self._get_signed()

    @property
    def dtype(self) -> torch.dtype:
        """The narrowest of uint8, int8, int16, int32 that holds the grid (encoding.py:178-192)."""
        if 0 <= self.qmin < self.qmax < 2 ** 8:
            return torch.uint8
        if -(2 ** 7) <= self.qmin < self.qmax < 2 ** 7:
            return torch.int8
        if -(2 ** 15) <= self.qmin < self.qmax < 2 ** 15:
            return torch.int16
        return torch.int32

    def to(self, *args, **kwargs):
        """Same encoding with scale/offset moved to another device and/or floating-point dtype."""
        scale = self.scale.to(*args, **kwargs)
        if scale is self.scale:
            return self
        if not scale.dtype.is_floating_point:
            raise RuntimeError(f"Cannot change encoding data dtype to {scale.dtype}, must be a floating point dtype")
        return self._rebuilt(scale, self.offset.to(*args, **kwargs))

    def _rebuilt(self, scale, offset):
        return AffineEncoding(scale, offset, self.qmin, self.qmax, self._symmetry, self.block_size,
                              self._zero_point_shift, producer=self.producer)

    # ------------------------------------------------------------------------------------------------ export --
    def _hint_input_shape(self, input_shape: Tuple[int, ...]) -> "AffineEncoding":
        """Shape of the tensor this encoding quantizes; needed to tell channel axes from block axes
        (aimet_torch/quantization/base/encoding.py:130-140)."""
        self._input_shape_hint = tuple(input_shape)
        return self

    def _safe_get_channel_and_block_axis(self):
        """(channel axis, block axis) as negative indices into the scale's dimensions, None where there is none
        (base/encoding.py:142-213).  An axis with several blocks of more than one element is a block axis; an axis
        with several blocks of one element is a channel axis."""
        from aimet_amd.quantization._utils import concretize_block_size

        if self._input_shape_hint is None:
            raise RuntimeError("Could not safely infer channel and block axes because input shape hint is not provided. "
                               "Call `_hint_input_shape` before calling this function.")
        concrete = concretize_block_size(self._input_shape_hint, self.scale.shape, self.block_size or ())
        channel_axes, block_axes = [], []
        for axis, (n_blocks, blk) in enumerate(zip(self.scale.shape, concrete)):
            if n_blocks > 1:
                (block_axes if blk > 1 else channel_axes).append(axis)
        if len(block_axes) > 1:
            raise RuntimeError(f"Multiple non-trivial block axes found: {block_axes}. Cannot determine a unique block axis.")
        block_axis = block_axes[0] if block_axes else None
        if not channel_axes and block_axis is not None:
            # a singleton dimension is still the channel axis when its block size is 1
            channel_axes = [axis for axis, blk in enumerate(concrete) if blk == 1]
        if len(channel_axes) > 1:
            raise RuntimeError(f"Multiple non-trivial channel axes found: {channel_axes}. "
                               "Cannot determine a unique channel axis.")
        channel_axis = channel_axes[0] if channel_axes else None
        if channel_axis is None and block_axis is not None:
            raise RuntimeError(f"Block axis {block_axis} found without a corresponding channel axis. "
                               "Cannot determine a unique channel axis.")
        nd = self.scale.dim()
        return (None if channel_axis is None else channel_axis - nd, None if block_axis is None else block_axis - nd)

    def _get_export_dtype(self) -> str:
        nbits = math.ceil(math.log2(self.qmax - self.qmin + 1))
        return f"int{nbits}" if self.qmin < 0 <= self.qmax else f"uint{nbits}"

    def _to_legacy_format(self) -> List[Dict]:
        """One dictionary per encoding; the offset counts from qmin (encoding.py:333-357)."""
        offset = self.offset.flatten() + self.qmin
        out = []
        for mn, mx, sc, off in zip(self.min.flatten(), self.max.flatten(), self.scale.flatten(), offset):
            enc = {"min": float(mn), "max": float(mx), "scale": float(sc), "offset": int(off),
                   "bitwidth": self.bitwidth, "dtype": "int", "is_symmetric": str(self.symmetry)}
            if self.zero_point_shift:
                enc["zero_point_shift"] = self.zero_point_shift
            out.append(enc)
        return out

    def _get_additional_properties(self) -> Dict[str, Any]:
        """Fields a subclass adds to the exported dictionaries (encoding.py:359-360)."""
        return {}

    @classmethod
    def _from_qnn_encoding_dict(cls, encoding_dict, version=None) -> "AffineEncoding":
        """A per-tensor encoding from its 2.0.0 / 2.1.0 dictionary (encoding.py:460-497)."""
        if version is None:
            version = "2.0.0" if "y_scale" in encoding_dict or "per_block_int_scale" in encoding_dict else "unknown"
        if version not in ("2.0.0", "2.1.0"):
            raise NotImplementedError(f"Only 2.0.0 and 2.1.0 encodings are supported; got {version}")
        if "per_block_int_scale" in encoding_dict or "axis" in encoding_dict:
            raise NotImplementedError("Only per-tensor encodings are supported")
        unsigned, bw = encoding_dict["output_dtype"].split("int")
        bw = int(bw)
        if unsigned:
            qmin, qmax = 0, 2 ** bw - 1
        else:
            qmin, qmax = -(2 ** (bw - 1)), 2 ** (bw - 1) - 1
        offset = -encoding_dict.get("y_zero_point", 0)
        return AffineEncoding(scale=torch.tensor(encoding_dict["y_scale"], dtype=torch.float32),
                              offset=torch.tensor(offset, dtype=torch.float32), qmin=qmin, qmax=qmax,
                              symmetry=(not unsigned) and offset == 0)

    def to_qnn_encoding_dict(self, encoding_version=None) -> Union[List, Dict]:
        """The encoding as a dictionary of the given format version (encoding.py:362-458)."""
        if encoding_version == "0.6.1":
            return self._to_legacy_format()

        if encoding_version == "1.0.0":
            offset = self.offset
            if self.signed:
                offset = offset - 2 ** (self.bitwidth - 1)
            enc = {"dtype": "INT", "bw": self.bitwidth, "is_sym": self.symmetry,
                   "scale": self.scale.flatten().tolist(), "offset": offset.to(torch.int).flatten().tolist()}
            if self.zero_point_shift != 0.0:
                assert self.zero_point_shift == 0.5 and self.symmetry
                enc["zero_point_shift"] = [self.zero_point_shift] * len(enc["offset"])
            granularity = self.granularity
            assert granularity != "unknown"
            if granularity == "pertensor":
                enc["enc_type"] = "PER_TENSOR"
            elif granularity == "perchannel":
                enc["enc_type"] = "PER_CHANNEL"
            else:
                _, block_axis = self._safe_get_channel_and_block_axis()
                enc["enc_type"] = "PER_BLOCK"
                enc["block_size"] = self.block_size[block_axis]
                if enc["block_size"] == -1:
                    raise NotImplementedError("Exporting encodings to 1.0.0 format with block size -1 is not supported yet. "
                                              "Export using sim.export() instead.")
            return enc

        if encoding_version in ("2.0.0", "2.1.0"):
            y_scale = self.scale
            if self.symmetry:
                y_zero_point = torch.full_like(y_scale, self._get_centroid(), dtype=torch.int32)
            else:
                y_zero_point = -self.offset.to(torch.int32)
            if self.zero_point_shift:
                y_zero_point = y_zero_point - self.zero_point_shift
            channel_axis = block_axis = block_size = None
            if self.granularity != "pertensor":
                channel_axis, block_axis = self._safe_get_channel_and_block_axis()
            if block_axis is not None:
                axis = block_axis
                block_size = self.block_size[block_axis]
            elif channel_axis is not None:
                axis = channel_axis
                y_scale, y_zero_point = y_scale.flatten(), y_zero_point.flatten()
            else:
                axis = None
                y_scale, y_zero_point = y_scale.squeeze(), y_zero_point.squeeze()
            ret = {"output_dtype": self._get_export_dtype(), "y_scale": y_scale.tolist()}
            if not bool(torch.all(y_zero_point == 0)):
                ret["y_zero_point"] = y_zero_point.tolist()
            if axis is not None:
                ret["axis"] = axis
            if block_size is not None:
                ret["block_size"] = block_size
            return ret

        raise AssertionError(f"Export encoding version {encoding_version} not supported."
                             "Expected one of: ['0.6.1', '1.0.0', '2.0.0', '2.1.0']")

    def quantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        return quantize(input, self.scale, self.offset, self.qmin, self.qmax, block_size=self.block_size)

    def dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        return dequantize(input, self.scale, self.offset, block_size=self.block_size)

    def quantize_dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        return quantize_dequantize(input, self.scale, self.offset, self.qmin, self.qmax, block_size=self.block_size,
                                   zero_point_shift=self._zero_point_shift)


class VectorEncoding(AffineEncoding):
    """Affine encoding of a vector-quantized tensor (encoding.py:500-575): the codebook geometry travels with it into
    the legacy and 1.0.0 dictionaries."""

    _FIELDS = ("rows_per_block", "cols_per_block", "vector_dim", "vector_stride", "index_bw")

    def __init__(self, scale: torch.Tensor, offset: torch.Tensor, bitwidth: int, signed=False, symmetry=False,
                 block_size: Optional[Tuple[int, ...]] = None, **kwargs):
        extra = {k: kwargs.pop(k) for k in self._FIELDS}  # all five are required
        super().__init__(scale, offset, bitwidth, signed, symmetry, block_size, **kwargs)
        for k, v in extra.items():
            setattr(self, k, v)

    def _get_additional_properties(self) -> Dict[str, Any]:
        return {k: getattr(self, k) for k in self._FIELDS}

    def _to_legacy_format(self) -> List[Dict]:
        encoding = super()._to_legacy_format()
        for e in encoding:
            e.update(self._get_additional_properties())
        return encoding

    def to_qnn_encoding_dict(self, encoding_version=None):
        encodings = super().to_qnn_encoding_dict(encoding_version)
        if encoding_version == "1.0.0":
            encodings.update(self._get_additional_properties())
            encodings["enc_type"] = "VECTOR"
        return encodings

    def _rebuilt(self, scale, offset):
        return VectorEncoding(scale, offset, self.bitwidth, self.signed, self._symmetry, self.block_size,
                              producer=self.producer, **self._get_additional_properties())


class GroupedBlockEncoding(AffineEncoding):
    """Blockwise encoding whose block scales are integer multiples of a per-channel scale (LPBQ)."""

    def __init__(self, scale, offset, bitwidth: int, signed=False, symmetry=False,
                 block_size: Optional[Tuple[int, ...]] = None, block_grouping: Optional[Tuple[int, ...]] = None,
                 decompressed_bw: Optional[int] = None, per_channel_scale: Optional[torch.Tensor] = None, **kwargs):
        super().__init__(scale, offset, bitwidth, signed, symmetry, block_size, **kwargs)
        self.block_grouping = block_grouping
        self.decompressed_bw = decompressed_bw
        self.per_channel_scale = per_channel_scale

    @property
    def per_block_int_scale(self) -> torch.Tensor:
        """Integer multipliers m with scale = m * per_channel_scale (1 <= m <= 2^(decompressed_bw - bitwidth))."""
        return quantize(self.scale, scale=self.per_channel_scale, offset=torch.zeros_like(self.per_channel_scale),
                        qmin=1, qmax=2 ** (self.decompressed_bw - self.bitwidth), block_size=self.block_grouping)

    def to_qnn_encoding_dict(self, encoding_version=None) -> Union[List, Dict]:
        """encoding.py:621-684: the per-block integer multipliers and the per-channel float scale replace the
        blockwise scale, unless no blocks are grouped or the legacy format is asked for."""
        enc = super().to_qnn_encoding_dict(encoding_version)
        if all(g == 1 for g in self.block_grouping) or encoding_version == "0.6.1":
            return enc
        if encoding_version == "1.0.0":
            enc["bw"] = self.decompressed_bw
            enc["compressed_bw"] = self.bitwidth
            enc["scale"] = self.per_channel_scale.flatten().tolist()
            enc["offset"] = [-(2 ** (self.decompressed_bw - 1)) for _ in enc["scale"]]
            enc["enc_type"] = "LPBQ"
            enc["per_block_int_scale"] = self.per_block_int_scale.to(torch.int32).flatten().tolist()
            return enc
        y_zero_point = enc.pop("y_zero_point", None)
        if y_zero_point is not None and bool(torch.any(torch.tensor(y_zero_point) != 0)):
            raise RuntimeError(f"LPBQ only supports symmetric quantization; got non-zero y_zero_point {y_zero_point}")
        output_dtype = f"int{self.bitwidth}" if self.signed else f"uint{self.bitwidth}"
        int_scale = self.per_block_int_scale.to(torch.int32).tolist()
        if encoding_version == "2.0.0":
            del enc["y_scale"]
            del enc["output_dtype"]
            enc.update({"per_block_int_scale": int_scale, "per_channel_float_scale": self.per_channel_scale.tolist(),
                        "output_dtype": output_dtype})
        else:
            channel_axis, _ = self._safe_get_channel_and_block_axis()
            enc.update({"y_scale": {"x": int_scale, "x_scale": self.per_channel_scale.flatten().tolist(),
                                    "axis": channel_axis},
                        "output_dtype": output_dtype})
        return enc

    @classmethod
    def _from_affine_encoding(cls, encoding: AffineEncoding) -> "GroupedBlockEncoding":
        """A symmetric blockwise encoding read as a grouped one (encoding.py:686-735): the groups run along the block
        axis, the block scales expand to twice the bitwidth, and the reading is accepted if snapping the scales to
        integer multiples of the per-channel scale leaves them where they are."""
        from aimet_amd.quantization.affine.quantizer import GroupedBlockQuantizeDequantize

        if isinstance(encoding, GroupedBlockEncoding):
            return encoding
        if not isinstance(encoding, AffineEncoding):
            raise ValueError(f"Only AffineEncoding can be converted to GroupedBlockEncoding; got {type(encoding)}")
        if encoding.block_size is None:
            raise ValueError("Only blockwise AffineEncodings can be converted to GroupedBlockEncoding; "
                             f"got block_size={encoding.block_size}")
        if not encoding.symmetry:
            raise ValueError("Only symmetric AffineEncodings can be converted to GroupedBlockEncoding; "
                             "asymmetric encodings are not supported")
        _, block_axis = encoding._safe_get_channel_and_block_axis()
        ndim = encoding.scale.dim()
        block_grouping = tuple(d if block_axis in (axis, axis - ndim) else 1
                               for axis, d in enumerate(encoding.scale.shape))
        qtzr = GroupedBlockQuantizeDequantize(shape=encoding.scale.shape, bitwidth=encoding.bitwidth,
                                              symmetric=encoding.symmetry, decompressed_bw=encoding.bitwidth * 2,
                                              block_size=encoding.block_size, block_grouping=block_grouping)
        qtzr.to(encoding.scale.device)
        with torch.no_grad():
            qtzr.min.copy_(encoding.min)
            qtzr.max.copy_(encoding.max)
        lpbq = qtzr.get_encodings()
        if torch.allclose(encoding.scale, lpbq.scale):
            if encoding._input_shape_hint is not None:
                lpbq._hint_input_shape(encoding._input_shape_hint)
            return lpbq
        raise ValueError("Failed to interpret encoding as GroupedBlockEncoding.")

    def _rebuilt(self, scale, offset):
        return GroupedBlockEncoding(scale, offset, self.bitwidth, self.signed, self._symmetry, self.block_size,
                                    self.block_grouping, self.decompressed_bw,
                                    self.per_channel_scale.to(device=scale.device, dtype=scale.dtype),
                                    zero_point_shift=self._zero_point_shift, producer=self.producer)
