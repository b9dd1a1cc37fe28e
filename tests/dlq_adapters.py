"""The CPU oracle (oracle/dlq_ref.c) and the HIP path behind one BlockTensorQuantizer-shaped interface, so the same
checks (tests/dlq_checks.py) run against both.  Tensors go in and come out as CPU torch tensors."""

import numpy as np
import torch

from oracle import dlq as OD

QUANTIZATION_TF = 0
QUANTIZATION_TF_ENHANCED = 1
QUANTIZATION_PERCENTILE = 3

# floating-point formats as (exponent bits, mantissa bits, finite, unsigned zero); an int stands for an integer grid
FP8_E4M3FN = (4, 3, True, False)
FP8_E5M2 = (5, 2, False, False)


def _widen(x: torch.Tensor) -> np.ndarray:
    return x.detach().to(torch.float32).cpu().numpy()


class OracleQuantizer:
    """BlockTensorQuantizer (TensorQuantizer.cpp) over the plain-C restatement."""

    def __init__(self, shape, bitwidth, scheme):
        self.shape = tuple(shape)
        self.fp8 = OD.fp8_spec(*bitwidth) if isinstance(bitwidth, tuple) else None
        self.bitwidth = self.fp8[0] if self.fp8 else bitwidth
        self.scheme = scheme
        self.E = int(np.prod(self.shape)) if self.shape else 1
        self.strict = False
        self.unsigned = False
        self.zps = 0.0
        self.percentile = 100.0
        self.valid_stats = False
        self.isEncodingValid = False
        self.encodings = None
        self._reset_stats(first=True)

    def _reset_stats(self, first=False):
        if self.scheme == QUANTIZATION_TF:
            self.mn = np.full(self.E, np.finfo(np.float32).max, dtype=np.float32)
            self.mx = np.full(self.E, -np.finfo(np.float32).max, dtype=np.float32)
        elif first:
            self.pdfs = [OD.Pdf() for _ in range(self.E)]
        else:
            for p in self.pdfs:
                p.reset()

    def resetEncodingStats(self):
        self.valid_stats = False
        self.isEncodingValid = False
        self._reset_stats()

    def updateStats(self, x, return_histogram=False):
        self.valid_stats = True
        blocks = OD.block_view(_widen(x), self.shape)  # 16-bit tensors are widened first, as the reference does
        if self.scheme == QUANTIZATION_TF:
            if blocks.size == 0:
                return None
            for e in range(self.E):
                mn, mx = OD.minmax(blocks[e])
                self.mn[e] = min(self.mn[e], mn)
                self.mx[e] = max(self.mx[e], mx)
            return None
        hists = [self.pdfs[e].update(blocks[e]) for e in range(self.E)]
        return torch.from_numpy(np.stack(hists).astype(np.int32)) if return_histogram else None

    def computeEncodings(self, symmetric):
        if not self.valid_stats:
            raise RuntimeError("Cannot compute encodings before updating stats")
        if self.fp8:
            fp8, self.fp8 = self.fp8, None
            try:
                computed = self.computeEncodings(symmetric)
            finally:
                self.fp8 = fp8
            seen = list(zip(self.mn, self.mx)) if self.scheme == QUANTIZATION_TF else [None] * self.E
            return [OD.fp8_encoding(c, o, fp8) for c, o in zip(computed, seen)]
        if self.scheme == QUANTIZATION_TF:
            return [tuple(OD.minmax_encoding(self.mn[e], self.mx[e], self.bitwidth, symmetric, self.strict, self.unsigned,
                                             self.zps)) for e in range(self.E)]
        if self.zps != 0.0:
            raise RuntimeError("Non-zero zeroPointShift is only supported for min-max quant scheme.")
        if self.scheme == QUANTIZATION_PERCENTILE:
            return [tuple(p.percentile_encoding(self.percentile, self.bitwidth, symmetric, self.strict, self.unsigned))
                    for p in self.pdfs]
        out = []
        self.last_best = []
        for p in self.pdfs:
            enc, n, best = p.compute_encoding(self.bitwidth, symmetric, self.strict, self.unsigned, with_index=True)
            out.append(tuple(enc))
            self.last_best.append((best, n))
        return out

    def load_pdf(self, xleft, pdf, iterations=1):
        """Put hand-built statistics ([E][1536] left edges and probabilities) in place of observed ones."""
        xleft, pdf = np.asarray(xleft, dtype=np.float64).reshape(self.E, -1), np.asarray(pdf, dtype=np.float64).reshape(self.E, -1)
        for e, p in enumerate(self.pdfs):
            p.load(xleft[e], pdf[e], iterations)
        self.valid_stats = True

    def setEncodings(self, encodings):
        if len(encodings) != self.E:
            raise RuntimeError("Length of encoding vector did not match BlockTensorQuantizer shape")
        self.encodings = [tuple(e) for e in encodings]
        self.isEncodingValid = True
        self.bitwidth = int(self.encodings[0][4])

    def quantizeDequantize(self, x):
        if not self.isEncodingValid:
            raise RuntimeError("Cannot perform quantization before computing encodings")
        encs = [[e[0], e[1], e[2], e[3]] for e in self.encodings]
        if self.fp8:
            if x.dtype != torch.float32:
                raise RuntimeError("BlockTensorQuantizer FP8 QDQ currently supports float tensors only")
            xf = x.numpy()
            if self.E == 1:
                return torch.from_numpy(OD.fp8_qdq(xf, encs[0][2], self.fp8))
            return torch.from_numpy(OD.fp8_qdq_broadcast(xf, self.shape, [e[2] for e in encs], self.fp8))
        xf = _widen(x)
        y = OD.qdq(xf, encs[0]) if self.E == 1 else OD.qdq_broadcast(xf, self.shape, encs)
        return torch.from_numpy(y).to(x.dtype)  # static_cast<DTYPE>(val): round to nearest even

    def setStrictSymmetric(self, v):
        self.isEncodingValid = False
        self.strict = bool(v)

    def setUnsignedSymmetric(self, v):
        self.isEncodingValid = False
        self.unsigned = bool(v)

    def setZeroPointShift(self, v):
        self.zps = float(v)

    def setPercentileValue(self, v):
        self.percentile = float(np.float32(v))

    def stats(self):
        """(min, max) arrays or (xleft, pdf, meta) arrays, for comparisons between implementations."""
        if self.scheme == QUANTIZATION_TF:
            return self.mn.copy(), self.mx.copy()
        return (np.stack([p.xleft for p in self.pdfs]), np.stack([p.pdf for p in self.pdfs]),
                np.array([p.meta for p in self.pdfs], dtype=np.int32))


class HipQuantizer:
    """aimet_amd.dlq.BlockTensorQuantizer with CPU tensors in and out."""

    def __init__(self, shape, bitwidth, scheme, device="cuda:0"):
        from aimet_amd import dlq

        self.dev = torch.device(device)
        if isinstance(bitwidth, tuple):
            bitwidth = dlq.QuantizationType.Float(*bitwidth)
        self.q = dlq.BlockTensorQuantizer(shape, bitwidth, scheme, device=self.dev)
        self.scheme = scheme

    @property
    def isEncodingValid(self):
        return self.q.isEncodingValid

    def resetEncodingStats(self):
        self.q.resetEncodingStats()

    def updateStats(self, x, return_histogram=False):
        h = self.q.updateStats(x.to(self.dev), return_histogram=return_histogram)
        return None if h is None else h.cpu()

    def computeEncodings(self, symmetric):
        encs = self.q.computeEncodings(symmetric)
        if self.scheme == QUANTIZATION_TF_ENHANCED:
            self.last_best = [tuple(r) for r in self.q._last_best.cpu().tolist()]
        return [tuple(e) for e in encs]

    def load_pdf(self, xleft, pdf, iterations=1):
        q = self.q
        E = q._xleft.shape[0]
        q._xleft.copy_(torch.from_numpy(np.asarray(xleft, dtype=np.float64).reshape(E, -1)))
        q._pdf.copy_(torch.from_numpy(np.asarray(pdf, dtype=np.float64).reshape(E, -1)))
        q._meta.zero_()
        q._meta[:, 0] = int(iterations)
        q._meta[:, 1] = 1
        q._meta[:, 2] = 1
        q._validStats = True
        q._all_initialized = True

    def setEncodings(self, encodings):
        self.q.setEncodings(encodings)

    def quantizeDequantize(self, x):
        return self.q.quantizeDequantize(x.to(self.dev)).cpu()

    def setStrictSymmetric(self, v):
        self.q.setStrictSymmetric(v)

    def setUnsignedSymmetric(self, v):
        self.q.setUnsignedSymmetric(v)

    def setZeroPointShift(self, v):
        self.q.setZeroPointShift(v)

    def setPercentileValue(self, v):
        self.q.setPercentileValue(v)

    def stats(self):
        if self.scheme == QUANTIZATION_TF:
            return self.q._min.cpu().numpy(), self.q._max.cpu().numpy()
        return self.q._xleft.cpu().numpy(), self.q._pdf.cpu().numpy(), self.q._meta[:, :3].cpu().numpy()
