"""Export of affine encodings to the dictionary formats (host code, no GPU): the parameter table and the assertions of
the reference's test_affine_encoding_schema_2_0_0 (test_affine_quantizer.py:2210-2315), plus the 1.0.0 and legacy
formats checked against their definitions (encoding.py:333-403)."""

import itertools

import numpy as np
import pytest
import torch

from aimet_amd.quantization.affine import AffineEncoding, QuantizeDequantize

LAYOUTS = [
    ((), None, None),
    ((10, 1, 1, 1), None, 0),
    ((1, 10, 1, 1), None, 1),
    ((10, 1), None, 0),
    ((1, 10), None, 1),
    ((10, 2, 1, 1), (1, 5, 1, 1), 1),
    ((2, 10, 1, 1), (5, 1, 1, 1), 0),
    ((10, 2), (1, 5), 1),
    ((2, 10), (5, 1), 0),
]
GRIDS = [
    (-2, 1, True, 0, "int2"), (0, 3, False, -2, "uint2"), (-8, 7, True, 0, "int4"), (-8, 7, False, -5, "int4"),
    (-8, 7, False, 0, "int4"), (0, 15, True, -8, "uint4"), (0, 15, False, -5, "uint4"), (0, 15, False, 0, "uint4"),
    (-128, 127, True, 0, "int8"), (-128, 127, False, -5, "int8"), (-128, 127, False, 0, "int8"),
    (0, 255, True, -128, "uint8"), (0, 255, False, -5, "uint8"), (0, 255, False, 0, "uint8"),
    (-(2 ** 15), 2 ** 15 - 1, True, 0, "int16"), (-(2 ** 15), 2 ** 15 - 1, False, -5, "int16"),
    (-(2 ** 15), 2 ** 15 - 1, False, 0, "int16"), (0, 2 ** 16 - 1, True, -(2 ** 15), "uint16"),
    (0, 2 ** 16 - 1, False, -5, "uint16"), (0, 2 ** 16 - 1, False, 0, "uint16"),
    (-(2 ** 31), 2 ** 31 - 1, True, 0, "int32"), (-(2 ** 31), 2 ** 31 - 1, False, 0, "int32"),
]


@torch.no_grad()
@pytest.mark.parametrize("shape,block_size,axis", LAYOUTS)
@pytest.mark.parametrize("qmin,qmax,symmetric,offset,output_dtype", GRIDS)
def test_affine_encoding_schema_2_0_0(shape, block_size, axis, qmin, qmax, symmetric, offset, output_dtype):
    input_shape = tuple([10] * len(shape))
    scale = torch.arange(1, int(np.prod(shape)) + 1).view(shape) * 0.001
    offset = torch.full_like(scale, offset)
    qtzr = QuantizeDequantize(shape=shape, qmin=qmin, qmax=qmax, symmetric=symmetric, block_size=block_size).to(torch.float64)
    qtzr.set_range(scale * (qmin + offset), scale * (qmax + offset))
    encoding = qtzr.get_encodings()._hint_input_shape(input_shape).to_qnn_encoding_dict("2.0.0")

    assert torch.allclose(torch.tensor(encoding["y_scale"]).view_as(scale), scale)
    if torch.all(offset == 0):
        assert "y_zero_point" not in encoding
    else:
        assert torch.equal(torch.tensor(encoding["y_zero_point"]).view_as(offset), -offset)
    if axis is None:
        assert "axis" not in encoding
    else:
        assert encoding["axis"] in (axis, axis - len(shape))
    if block_size is None:
        assert "block_size" not in encoding
    else:
        assert encoding["block_size"] == next(iter(blk for blk in block_size if blk != 1))
    assert encoding["output_dtype"] == output_dtype


@torch.no_grad()
@pytest.mark.parametrize("shape,block_size,axis", LAYOUTS)
@pytest.mark.parametrize("bitwidth,signed,symmetric", [(8, False, False), (8, True, True), (4, True, True), (16, False, False)])
def test_schema_1_0_0_and_legacy(shape, block_size, axis, bitwidth, signed, symmetric):
    n = int(np.prod(shape))
    scale = torch.arange(1, n + 1, dtype=torch.float32).view(shape) * 0.01
    qmin = -(2 ** (bitwidth - 1)) if signed else 0
    qmax = qmin + 2 ** bitwidth - 1
    off_val = -3.0 if not symmetric else float(-round((qmin + qmax) / 2))
    offset = torch.full_like(scale, off_val)
    enc = AffineEncoding(scale, offset, qmin, qmax, symmetric, block_size)._hint_input_shape(tuple([10] * len(shape)))

    d = enc.to_qnn_encoding_dict("1.0.0")
    assert d["dtype"] == "INT" and d["bw"] == bitwidth and d["is_sym"] == symmetric
    assert np.allclose(d["scale"], scale.flatten().tolist())
    # the 1.0.0 offset counts from the lowest code of the *unsigned* grid
    expect = int(off_val) - (2 ** (bitwidth - 1) if signed else 0)
    assert d["offset"] == [expect] * n
    if shape == ():
        assert d["enc_type"] == "PER_TENSOR" and "block_size" not in d
    elif block_size is None:
        assert d["enc_type"] == "PER_CHANNEL" and "block_size" not in d
    else:
        assert d["enc_type"] == "PER_BLOCK" and d["block_size"] == 5

    legacy = enc.to_qnn_encoding_dict("0.6.1")
    assert isinstance(legacy, list) and len(legacy) == n
    for i, e in enumerate(legacy):
        s = float(scale.flatten()[i])
        assert e["bitwidth"] == bitwidth and e["dtype"] == "int" and e["is_symmetric"] == str(symmetric)
        assert e["offset"] == int(off_val) + qmin
        assert e["scale"] == pytest.approx(s)
        assert e["min"] == pytest.approx((off_val + qmin) * s) and e["max"] == pytest.approx((off_val + qmax) * s)


def test_zero_point_shift_and_errors():
    scale = torch.tensor([0.5, 0.25]).view(2, 1)
    enc = AffineEncoding(scale, torch.full_like(scale, -2.0), -2, 1, True, None, 0.5)._hint_input_shape((2, 8))
    d = enc.to_qnn_encoding_dict("2.0.0")
    assert d["y_zero_point"] == [-0.5, -0.5] and d["axis"] in (0, -2) and d["output_dtype"] == "int2"
    assert enc.to_qnn_encoding_dict("1.0.0")["zero_point_shift"] == [0.5, 0.5]
    assert all(e["zero_point_shift"] == 0.5 for e in enc.to_qnn_encoding_dict("0.6.1"))
    with pytest.raises(AssertionError):
        enc.to_qnn_encoding_dict("3.0.0")
    with pytest.raises(RuntimeError, match="input shape hint"):
        AffineEncoding(scale, torch.zeros_like(scale), 0, 255).to_qnn_encoding_dict("2.0.0")
    two_block_axes = AffineEncoding(torch.ones(2, 2), torch.zeros(2, 2), 0, 255, False, (5, 5))._hint_input_shape((10, 10))
    with pytest.raises(RuntimeError, match="Multiple non-trivial block axes"):
        two_block_axes.to_qnn_encoding_dict("2.0.0")


def test_from_qnn_encoding_dict():
    """Reference expectation: test_affine_quantizer.py:2788-2826."""
    e = AffineEncoding._from_qnn_encoding_dict({"y_scale": 0.1, "output_dtype": "int8"}, version="2.0.0")
    assert e.scale == 0.1 and e.offset == 0 and e.symmetry and (e.qmin, e.qmax) == (-128, 127)
    e = AffineEncoding._from_qnn_encoding_dict({"y_scale": 0.1, "output_dtype": "uint8"}, version="2.0.0")
    assert e.scale == 0.1 and e.offset == 0 and not e.symmetry and (e.qmin, e.qmax) == (0, 255)
    e = AffineEncoding._from_qnn_encoding_dict({"y_scale": 0.1, "y_zero_point": 0, "output_dtype": "int8"}, version="2.0.0")
    assert e.scale == 0.1 and e.offset == 0 and e.symmetry
    e = AffineEncoding._from_qnn_encoding_dict({"y_scale": 0.1, "y_zero_point": 128, "output_dtype": "uint8"}, version="2.0.0")
    assert e.scale == 0.1 and e.offset == -128 and not e.symmetry
    # the version is recognised from the keys; everything but per-tensor 2.x dictionaries is refused
    assert AffineEncoding._from_qnn_encoding_dict({"y_scale": 0.5, "output_dtype": "uint4"}).qmax == 15
    with pytest.raises(NotImplementedError):
        AffineEncoding._from_qnn_encoding_dict({"scale": [0.1], "bw": 8}, version=None)
    with pytest.raises(NotImplementedError):
        AffineEncoding._from_qnn_encoding_dict({"y_scale": [0.1, 0.2], "axis": 0, "output_dtype": "int8"}, version="2.1.0")
    # and a per-tensor encoding survives the round trip
    src = AffineEncoding(torch.tensor(0.25), torch.tensor(-3.0), 0, 255)
    back = AffineEncoding._from_qnn_encoding_dict(src.to_qnn_encoding_dict("2.0.0"), version="2.0.0")
    assert back.scale == src.scale and back.offset == src.offset and (back.qmin, back.qmax) == (0, 255)


def test_encoding_dtype_is_the_narrowest_integer_type_that_holds_the_grid():
    """encoding.py:178-192."""
    one, zero = torch.tensor(1.0), torch.tensor(0.0)
    assert AffineEncoding(one, zero, 0, 255).dtype == torch.uint8
    assert AffineEncoding(one, zero, 0, 15).dtype == torch.uint8
    assert AffineEncoding(one, zero, -128, 127).dtype == torch.int8
    assert AffineEncoding(one, zero, -8, 7).dtype == torch.int8
    assert AffineEncoding(one, zero, 0, 256).dtype == torch.int16
    assert AffineEncoding(one, zero, -32768, 32767).dtype == torch.int16
    assert AffineEncoding(one, zero, 0, 65535).dtype == torch.int32
    assert AffineEncoding(one, zero, -(2 ** 31), 2 ** 31 - 1).dtype == torch.int32


def test_vector_encoding_carries_its_codebook_geometry():
    """encoding.py:500-575."""
    from aimet_amd.quantization.affine import VectorEncoding

    geometry = dict(rows_per_block=64, cols_per_block=2, vector_dim=2, vector_stride=1, index_bw=8)
    e = VectorEncoding(torch.tensor([0.5, 0.25]), torch.zeros(2), 8, signed=True, symmetry=True, **geometry)
    assert e._get_additional_properties() == geometry
    legacy = e.to_qnn_encoding_dict("0.6.1")
    assert len(legacy) == 2 and all(all(entry[k] == v for k, v in geometry.items()) for entry in legacy)
    v1 = e._hint_input_shape((2, 8)).to_qnn_encoding_dict("1.0.0")
    assert v1["enc_type"] == "VECTOR" and all(v1[k] == v for k, v in geometry.items())
    assert "rows_per_block" not in e.to_qnn_encoding_dict("2.0.0")
    moved = e.to(torch.float64)
    assert isinstance(moved, VectorEncoding) and moved.scale.dtype == torch.float64
    assert moved._get_additional_properties() == geometry
    assert AffineEncoding(torch.tensor(1.0), torch.tensor(0.0), 0, 255)._get_additional_properties() == {}
    with pytest.raises(KeyError):
        VectorEncoding(torch.tensor(1.0), torch.tensor(0.0), 8, rows_per_block=1)
