"""TEST INFRASTRUCTURE ONLY: ctypes access to libdlq_ref.so, the plain-C restatement of the DlQuantization CPU path
(oracle/dlq_ref.c).  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module."""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdlq_ref.so")
PDF_SIZE = 1536
_lib = None

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")


def lib():
    global _lib
    if _lib is None:
        src = os.path.join(_HERE, "dlq_ref.c")
        if not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
            subprocess.run(["make", "-s", "-C", _HERE], check=True)
        L = ctypes.CDLL(_LIB_PATH)
        L.dlq_qdq.argtypes = [_f32p, ctypes.c_uint64] + [ctypes.c_double] * 4 + [_f32p]
        L.dlq_qdq.restype = None
        L.dlq_qdq_broadcast.argtypes = [_f32p, _f32p, _i64p, ctypes.c_int, _i64p, ctypes.c_int, _f64p]
        L.dlq_qdq_broadcast.restype = ctypes.c_int
        L.dlq_fp8_qdq.argtypes = [_f32p, ctypes.c_uint64, ctypes.c_double, ctypes.c_int, ctypes.c_int, ctypes.c_double, _f32p]
        L.dlq_fp8_qdq.restype = None
        L.dlq_minmax.argtypes = [_f32p, ctypes.c_uint64, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
        L.dlq_minmax.restype = None
        L.dlq_computed_encodings.argtypes = [ctypes.c_int, ctypes.c_double, ctypes.c_double, ctypes.c_int, ctypes.c_int,
                                             ctypes.c_int, ctypes.c_double, _f64p]
        L.dlq_computed_encodings.restype = ctypes.c_int
        L.dlq_minmax_encoding.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_double, _f64p]
        L.dlq_minmax_encoding.restype = ctypes.c_int
        L.dlq_pdf_sizeof.restype = ctypes.c_uint64
        for name in ("dlq_pdf_init", "dlq_pdf_reset"):
            getattr(L, name).argtypes = [ctypes.c_void_p]
            getattr(L, name).restype = None
        L.dlq_pdf_update.argtypes = [ctypes.c_void_p, _f32p, ctypes.c_uint64, _u32p]
        L.dlq_pdf_update.restype = None
        L.dlq_tfe_compute_encoding.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               _f64p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.dlq_tfe_compute_encoding.restype = None
        L.dlq_percentile_compute_encoding.argtypes = [ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_int,
                                                      ctypes.c_int, ctypes.c_int, _f64p]
        L.dlq_percentile_compute_encoding.restype = None
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).reshape(-1))


def qdq(x, enc):
    """enc = (min, max, delta, offset); x any float array-like -> float32 array of the same shape."""
    x = np.asarray(x, dtype=np.float32)
    out = np.empty(x.size, dtype=np.float32)
    lib().dlq_qdq(_f32(x), x.size, float(enc[0]), float(enc[1]), float(enc[2]), float(enc[3]), out)
    return out.reshape(x.shape)


def qdq_broadcast(x, enc_shape, encs):
    """encs: [E][4] = min, max, delta, offset in row-major order of enc_shape."""
    x = np.asarray(x, dtype=np.float32)
    out = np.empty(x.size, dtype=np.float32)
    ts = np.asarray(x.shape, dtype=np.int64)
    es = np.asarray(list(enc_shape), dtype=np.int64)
    e = np.ascontiguousarray(np.asarray(encs, dtype=np.float64).reshape(-1, 4))
    rc = lib().dlq_qdq_broadcast(_f32(x), out, ts, len(ts), es, len(es), e)
    if rc:
        raise RuntimeError("Cannot interpret tensor and encoding dimensions as broadcastable")
    return out.reshape(x.shape)


def fp8_spec(exponent_bits, mantissa_bits, finite, unsigned_zero):
    """QuantizationType::Float(exponentBits, mantissaBits, finite, unsignedZero) (QuantizationType.hpp:85-128):
    returns (bitwidth, mantissa_bits, exponent_min, max_value)."""
    bias = (1 << (exponent_bits - 1)) - 1 + (1 if unsigned_zero else 0)
    unit = 2.0 ** -mantissa_bits
    if unsigned_zero:
        max_exp, max_man = (1 << exponent_bits) - 1 - bias, 2.0 - unit
    elif finite:
        max_exp, max_man = (1 << exponent_bits) - 1 - bias, 2.0 - 2.0 * unit
    else:
        max_exp, max_man = (1 << exponent_bits) - 2 - bias, 2.0 - unit
    return 1 + exponent_bits + mantissa_bits, mantissa_bits, 1 - bias, max_man * 2.0 ** max_exp


FP8_E4M3FN = fp8_spec(4, 3, True, False)
FP8_E5M2 = fp8_spec(5, 2, False, False)


def fp8_qdq(x, delta, spec):
    x = np.asarray(x, dtype=np.float32)
    out = np.empty(x.size, dtype=np.float32)
    lib().dlq_fp8_qdq(_f32(x), x.size, float(delta), spec[1], spec[2], float(spec[3]), out)
    return out.reshape(x.shape)


def fp8_qdq_broadcast(x, enc_shape, deltas, spec):
    """quantizeDequantizeFp8Broadcast (trim_functions.cpp:791-900): every block with its own scale."""
    x = np.asarray(x, dtype=np.float32)
    ts = list(x.shape)
    es = [1] * (len(ts) - len(enc_shape)) + list(enc_shape)
    split, enc_axes, blk_axes = [], [], []
    for d, e in zip(ts, es):
        enc_axes.append(len(split))
        split.append(e)
        blk_axes.append(len(split))
        split.append(d // e)
    perm = enc_axes + blk_axes
    blocks = block_view(x, enc_shape)
    out = np.stack([fp8_qdq(blocks[e], deltas[e], spec) for e in range(blocks.shape[0])])
    out = out.reshape([split[a] for a in perm]).transpose(np.argsort(perm))
    return np.ascontiguousarray(out).reshape(x.shape)


def fp8_encoding(computed, observed, spec):
    """The FP8 branch of BlockTensorQuantizer::computeEncodings (TensorQuantizer.cpp:182-224).  computed: the
    analyzer's (min, max, ...); observed: (min, max) statistics where the analyzer keeps them (min/max scheme),
    else None.  Returns (min, max, delta, offset, bw)."""
    amax = max(abs(float(computed[0])), abs(float(computed[1])))
    if observed is not None:
        seen = max(abs(float(observed[0])), abs(float(observed[1])))
        if seen > 0.0:
            amax = seen
    if not amax > 0:
        raise ValueError("FP8 amax must be positive")
    scale = amax / spec[3]
    return (-scale * spec[3], scale * spec[3], scale, 0.0, spec[0])


def minmax(x):
    mn, mx = ctypes.c_float(), ctypes.c_float()
    x = _f32(x)
    lib().dlq_minmax(x, x.size, ctypes.byref(mn), ctypes.byref(mx))
    return np.float32(mn.value), np.float32(mx.value)


def computed_encodings(bw, mn, mx, symmetric, strict=False, unsigned_sym=False, zps=0.0):
    out = np.zeros(5)
    if lib().dlq_computed_encodings(bw, float(mn), float(mx), int(symmetric), int(strict), int(unsigned_sym), zps, out):
        raise RuntimeError("zero_point_shift is not supported in this mode")
    return out


def minmax_encoding(stat_min, stat_max, bw, symmetric, strict=False, unsigned_sym=False, zps=0.0):
    out = np.zeros(5)
    if lib().dlq_minmax_encoding(float(stat_min), float(stat_max), bw, int(symmetric), int(strict), int(unsigned_sym),
                                 zps, out):
        raise RuntimeError("zero_point_shift is not supported in this mode")
    return out


def block_view(x, enc_shape):
    """Rows of `x` gathered per encoding block (what withContiguousBlocks hands to the per-block analyzers):
    returns an array [E][block_numel]."""
    x = np.asarray(x)
    ts = list(x.shape)
    es = [1] * (len(ts) - len(enc_shape)) + list(enc_shape)
    split, enc_axes, blk_axes = [], [], []
    for d, e in zip(ts, es):
        if d < e or d % e:
            raise RuntimeError("Cannot interpret tensor and encoding dimensions as broadcastable")
        enc_axes.append(len(split))
        split.append(e)
        blk_axes.append(len(split))
        split.append(d // e)
    v = x.reshape(split).transpose(enc_axes + blk_axes)
    E = int(np.prod(es)) if es else 1
    return np.ascontiguousarray(v.reshape(E, -1))


class Pdf:
    """One TF-enhanced analyzer's statistics (TfEnhancedEncodingAnalyzer with its PDF)."""

    def __init__(self):
        self._buf = ctypes.create_string_buffer(int(lib().dlq_pdf_sizeof()))
        lib().dlq_pdf_init(self._buf)

    def reset(self):
        lib().dlq_pdf_reset(self._buf)

    def update(self, x):
        x = _f32(x)
        hist = np.zeros(PDF_SIZE, dtype=np.uint32)
        lib().dlq_pdf_update(self._buf, x, x.size, hist)
        return hist

    def load(self, xleft, pdf, iterations=1):
        """Replace the statistics by a given table of left edges and probabilities (tests build such tables by hand)."""
        buf = np.frombuffer(self._buf, dtype=np.float64, count=2 * PDF_SIZE, offset=0)
        buf[:PDF_SIZE] = np.asarray(xleft, dtype=np.float64)
        buf[PDF_SIZE:] = np.asarray(pdf, dtype=np.float64)
        meta = np.frombuffer(self._buf, dtype=np.int32, count=3, offset=16 * PDF_SIZE)
        meta[:] = (int(iterations), 1, 1)

    @property
    def xleft(self):
        return np.frombuffer(self._buf, dtype=np.float64, count=PDF_SIZE, offset=0).copy()

    @property
    def pdf(self):
        return np.frombuffer(self._buf, dtype=np.float64, count=PDF_SIZE, offset=8 * PDF_SIZE).copy()

    @property
    def meta(self):
        """(iterations, initialized, stats_updated)"""
        m = np.frombuffer(self._buf, dtype=np.int32, count=3, offset=16 * PDF_SIZE)
        return int(m[0]), int(m[1]), int(m[2])

    def compute_encoding(self, bw, symmetric, strict=False, unsigned_sym=False, with_index=False):
        out = np.zeros(5)
        n, best = ctypes.c_int(), ctypes.c_int()
        lib().dlq_tfe_compute_encoding(self._buf, bw, int(symmetric), int(strict), int(unsigned_sym), out,
                                       ctypes.byref(n), ctypes.byref(best))
        return (out, n.value, best.value) if with_index else out

    def percentile_encoding(self, percentile, bw, symmetric, strict=False, unsigned_sym=False):
        out = np.zeros(5)
        lib().dlq_percentile_compute_encoding(self._buf, float(percentile), bw, int(symmetric), int(strict),
                                              int(unsigned_sym), out)
        return out
