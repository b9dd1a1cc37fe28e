"""Adapters that expose the CPU oracle and the HIP path behind the interface tests/golden_checks.py expects."""

import torch

from oracle import torch_ref as O


class OracleImpl:
    name = "oracle"

    def quantize(self, x, scale, offset, qmin, qmax, block):
        return O.quantize_forward(x, scale, offset, qmin, qmax, block)[0]

    def dequantize(self, codes, scale, offset, block):
        return O.dequantize_forward(codes, scale, offset, block)

    def qdq(self, x, scale, offset, qmin, qmax, block, zps):
        return O.qdq_v2_forward(x, scale, offset, qmin, qmax, block, zps).y

    def qdq_backward(self, g, x, scale, offset, qmin, qmax, block, zps):
        return O.qdq_v2_backward(g, x, scale, offset, qmin, qmax, block, zps)

    def quantize_backward(self, g, x, scale, offset, qmin, qmax, block):
        return O.quantize_backward(g, x, scale, offset, qmin, qmax, block)[0]

    def minmax_encodings(self, x, num_steps, symmetric):
        mn, mx = O.reduce_minmax(x, ())
        return O.minmax_encodings(mn, mx, num_steps, symmetric)

    def hist_observer(self, num_bins):
        obs = O.HistObserver((), num_bins)

        class _Obs:
            def update(self, x):
                obs.update(x)

            def stat(self):
                s = obs.stats[0]
                return s.histogram, s.bin_edges, s.min, s.max

        return _Obs()

    def sqnr(self, batches, num_steps, symmetric, num_bins=2048, asymmetric_delta_candidates=17,
             symmetric_delta_candidates=101, offset_candidates=21, gamma=3.0):
        obs = O.HistObserver((1,), num_bins)
        for b in batches:
            obs.update(b)
        lo, hi, *_ = O.sqnr_encodings(obs.stats, (1,), num_steps, symmetric, asym_deltas=asymmetric_delta_candidates,
                                      sym_deltas=symmetric_delta_candidates, num_offsets=offset_candidates,
                                      gamma=float(gamma))
        return lo, hi

    def percentile(self, batches, shape, num_bins, percentile, num_steps, symmetric):
        obs = O.HistObserver(shape, num_bins)
        for b in batches:
            obs.update(b)
        lo, hi = O.percentile_encodings(obs.stats, shape, percentile, num_steps, symmetric)
        return lo, hi, [s.histogram for s in obs.stats], [s.bin_edges for s in obs.stats]


class HipImpl:
    """The product path on cuda:0, results brought back to the CPU."""

    name = "hip"

    def __init__(self, device):
        self.dev = device

    def _d(self, t, grad=False):
        return t.to(self.dev).requires_grad_(grad)

    def quantize(self, x, scale, offset, qmin, qmax, block):
        from aimet_amd.quantization import affine
        return affine.quantize(self._d(x), self._d(scale), self._d(offset), qmin, qmax, block_size=block).cpu()

    def dequantize(self, codes, scale, offset, block):
        from aimet_amd.quantization import affine
        return affine.dequantize(self._d(codes), self._d(scale), self._d(offset), block_size=block).cpu()

    def qdq(self, x, scale, offset, qmin, qmax, block, zps):
        from aimet_amd.quantization import affine
        # scale requires grad so that the composed autograd arithmetic is selected, as in the reference's tests
        return affine.quantize_dequantize(self._d(x), self._d(scale, True), self._d(offset), qmin, qmax,
                                          block_size=block, zero_point_shift=zps).detach().cpu()

    def qdq_backward(self, g, x, scale, offset, qmin, qmax, block, zps):
        from aimet_amd.quantization import affine
        xd, sd, od = self._d(x, True), self._d(scale, True), self._d(offset, True)
        y = affine.quantize_dequantize(xd, sd, od, qmin, qmax, block_size=block, zero_point_shift=zps)
        y.backward(self._d(g))
        return xd.grad.cpu(), sd.grad.cpu(), od.grad.cpu()

    def quantize_backward(self, g, x, scale, offset, qmin, qmax, block):
        from aimet_amd.quantization import affine
        xd = self._d(x, True)
        affine.quantize(xd, self._d(scale), self._d(offset), qmin, qmax, block_size=block).backward(self._d(g))
        return xd.grad.cpu()

    def minmax_encodings(self, x, num_steps, symmetric):
        from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer
        an = MinMaxEncodingAnalyzer(())
        an.update_stats(self._d(x))
        lo, hi = an.compute_encodings(num_steps, symmetric)
        return lo.cpu(), hi.cpu()

    def hist_observer(self, num_bins):
        from aimet_amd.quantization.encoding_analyzer import _HistogramObserver
        obs = _HistogramObserver((), num_bins=num_bins)
        dev = self.dev

        class _Obs:
            def update(self, x):
                obs.update(x.to(dev))

            def stat(self):
                s = obs.get_stats()[0]
                return s.histogram.cpu(), s.bin_edges.cpu(), s.min.cpu(), s.max.cpu()

        return _Obs()

    def sqnr(self, batches, num_steps, symmetric, **kw):
        from aimet_amd.quantization.encoding_analyzer import SqnrEncodingAnalyzer
        an = SqnrEncodingAnalyzer((1,), **kw)
        for b in batches:
            an.update_stats(self._d(b))
        lo, hi = an.compute_encodings(num_steps, symmetric)
        return lo.cpu(), hi.cpu()

    def percentile(self, batches, shape, num_bins, percentile, num_steps, symmetric):
        from aimet_amd.quantization.encoding_analyzer import PercentileEncodingAnalyzer
        an = PercentileEncodingAnalyzer(shape, num_bins=num_bins, percentile=percentile)
        for b in batches:
            an.update_stats(self._d(b))
        lo, hi = an.compute_encodings(num_steps, symmetric)
        stats = an.observer.get_stats()
        return lo.cpu(), hi.cpu(), [s.histogram.cpu() for s in stats], [s.bin_edges.cpu() for s in stats]
