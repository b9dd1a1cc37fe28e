"""Encoding analyzers: observe tensors on the GPU and turn the statistics into (min, max) encodings.

Same classes, constructor signatures and methods as aimet_torch/quantization/encoding_analyzer.py:
``MinMaxEncodingAnalyzer``, ``PercentileEncodingAnalyzer``, ``SqnrEncodingAnalyzer``, ``TfEnhancedEncodingAnalyzer``
(``update_stats``, ``reset_stats``, ``compute_encodings``, ``compute_encodings_from_stats``,
``compute_dynamic_encodings``, ``.observer.shape``).  Every pass over a tensor (min/max, histogram binning) and the
SQNR candidate search run in HIP kernels; only arithmetic on encoding-shaped tensors is left to torch ops on the
device, where each operation is a single IEEE operation and therefore reproduces the reference bit for bit.
"""

# pylint: disable=redefined-builtin, missing-docstring

from __future__ import annotations

import functools
import math
import contextlib
import warnings
from abc import ABC, abstractmethod
from dataclasses import dataclass
from collections.abc import Sequence
from typing import Generic, List, Optional, Tuple, TypeVar

import torch

from aimet_amd import _lib
from aimet_amd._lib import HipLibraryError
from aimet_amd.quantization._utils import StatisticsNotFoundError, _get_minimum_scale, _is_expandable, true_divide
from aimet_amd.quantization._stats import reduce_min_max, _check_reducible
from aimet_amd.quantization.affine.backends.hip import _prepare


class _MinMaxRange:
    """The reference's ``_MinMaxRange(min, max)`` (encoding_analyzer.py:46-50).  A single encoding's statistics may
    still lie in the per-workgroup slots of the streaming kernel (``from_slots``): ``min`` / ``max`` fold them when they
    are first read, and a consumer that takes slots (MinMaxEncodingAnalyzer.compute_encodings_from_stats, the end of
    a quantizer's calibration) folds them inside its own launch, so that nothing is launched for statistics nobody
    reads."""

    __slots__ = ("_min", "_max", "_slots", "_of")

    def __init__(self, min: Optional[torch.Tensor] = None, max: Optional[torch.Tensor] = None):
        self._min, self._max, self._slots, self._of = min, max, None, None

    @classmethod
    def from_slots(cls, slots: torch.Tensor, dtype, device, shape) -> "_MinMaxRange":
        r = cls()
        r._slots, r._of = slots, (dtype, device, tuple(shape))
        return r

    def unfolded(self):
        """(dtype, device, shape, slot buffer) while the statistics have not been folded, else None."""
        return (*self._of, self._slots) if self._slots is not None else None

    def adopt(self, mn: torch.Tensor, mx: torch.Tensor) -> None:
        """The folded statistics, from the launch of a consumer that formed them on its way."""
        self._min, self._max, self._slots = mn, mx, None

    def _fold(self) -> None:
        if self._slots is None:
            return
        dtype, device, shape = self._of
        mn = torch.empty(shape, dtype=dtype, device=device)
        mx = torch.empty(shape, dtype=dtype, device=device)
        _lib.check(_lib.load().ahq_minmax_slots_read(_lib.DTYPE_CODE[dtype], self._slots.data_ptr(), mn.data_ptr(),
                                                     mx.data_ptr(), _lib.current_stream(device)),
                   "ahq_minmax_slots_read")
        self.adopt(mn, mx)

    @property
    def min(self) -> Optional[torch.Tensor]:
        self._fold()
        return self._min

    @min.setter
    def min(self, value):
        self._fold()
        self._min = value

    @property
    def max(self) -> Optional[torch.Tensor]:
        self._fold()
        return self._max

    @max.setter
    def max(self, value):
        self._fold()
        self._max = value

    def is_empty(self) -> bool:
        """Nothing observed (without folding anything)."""
        return self._slots is None and self._min is None and self._max is None

    def __eq__(self, other):
        return isinstance(other, _MinMaxRange) and self.min is other.min and self.max is other.max

    __hash__ = None

    def __repr__(self):
        return f"_MinMaxRange(min={self.min!r}, max={self.max!r})"

    def __getstate__(self):
        self._fold()
        return (self._min, self._max)

    def __setstate__(self, state):
        self._min, self._max = state
        self._slots = self._of = None


@dataclass
class _Histogram:
    histogram: torch.Tensor = None
    bin_edges: torch.Tensor = None
    min: Optional[torch.Tensor] = None
    max: Optional[torch.Tensor] = None


class _HistogramList(Sequence):
    """``List[_Histogram]`` (one entry per encoding, what the reference's observer returns) as a view over the stacked
    device tensors: entries are built when they are asked for.  A per-channel or blockwise observer has thousands of
    slots, and materialising a Python object with four tensor views for each of them on every batch costs
    milliseconds to seconds of host time that nothing reads during a calibration pass."""

    def __init__(self, hist, edges, minmax, dtype, count: Optional[int] = None, make=None):
        self._hist, self._edges, self._minmax, self._dtype = hist, edges, minmax, dtype
        self._typed_minmax = None
        # forms (counts, edges, min/max) when they are first asked for (see _HistogramObserver.update)
        self._make = make
        self._count = int(count) if count is not None else hist.shape[0]

    def __len__(self) -> int:
        return self._count

    def _counts(self):
        if self._hist is None and self._make is not None:
            (self._hist, self._edges, self._minmax), self._make = self._make(), None
        return self._hist

    def stacked(self):
        """(hist [S, B], bin edges [S, B + 1], min/max [S, 2] in float32, dtype the reference keeps min/max in)."""
        hist = self._counts()
        return hist, self._edges, self._minmax, self._dtype

    def _entry(self, i: int) -> _Histogram:
        if self._counts() is None:
            return _Histogram()
        if self._typed_minmax is None:
            self._typed_minmax = self._minmax if self._dtype == torch.float32 else self._minmax.to(self._dtype)
        mm = self._typed_minmax
        return _Histogram(self._hist[i], self._edges[i], mm[i, 0], mm[i, 1])

    def __getitem__(self, i):
        if isinstance(i, slice):
            return [self._entry(k) for k in range(*i.indices(self._count))]
        if i < 0:
            i += self._count
        if not 0 <= i < self._count:
            raise IndexError("histogram index out of range")
        return self._entry(i)

    def __iter__(self):
        return (self._entry(i) for i in range(self._count))


_Statistics = TypeVar("_Statistics", _MinMaxRange, _Histogram)


class _Observer(Generic[_Statistics], ABC):
    """Observes tensors and accumulates statistics of a given shape."""

    def __init__(self, shape, block_size=None):
        if isinstance(shape, int):
            shape = (shape,)
        self.shape = tuple(shape)
        self.block_size = block_size

    @abstractmethod
    def collect_stats(self, input_tensor: torch.Tensor) -> _Statistics: ...

    @abstractmethod
    def merge_stats(self, stats: _Statistics): ...

    @abstractmethod
    def reset_stats(self): ...

    @abstractmethod
    def get_stats(self) -> _Statistics: ...


class _MinMaxObserver(_Observer[_MinMaxRange]):
    """Running per-encoding minimum and maximum (reference: encoding_analyzer.py:69-118).  One fused kernel reads the
    tensor once for both extrema and folds them into the running statistics."""

    def __init__(self, shape, block_size=None):
        super().__init__(shape, block_size)
        self.stats = _MinMaxRange()
        # A single encoding keeps its running extrema as one slot per workgroup of the streaming kernel
        # (ahq_minmax_accumulate): one launch per batch, no launch that folds a batch's partials.  The batch's own
        # extrema come back as slots of their own (a _MinMaxRange that folds them if they are read), and `stats`
        # becomes a view of the running slots when somebody asks for it (get_stats), folded at the latest before the
        # next batch changes the slots.  Any other way of adding statistics (merge_stats, tensors the streaming
        # kernel does not take) folds the slots into `stats` and takes over.
        self._single = math.prod(self.shape) == 1 and not block_size
        self._slots = None         # the slot buffer, kept across reset_stats()
        self._slots_of = None      # (dtype, device) of the tensors accumulated while the slots are live, else None
        self._slots_dirty = False  # the slots hold more than `stats`

    def _stats_view_live(self) -> bool:
        """`stats` is an unfolded view of the running slots."""
        u = self.stats.unfolded()
        return u is not None and u[3] is self._slots

    def _fold_slots(self):
        """`stats` = everything the slots hold, as tensors."""
        if self._slots_of is not None and self._slots_dirty:
            self.stats = _MinMaxRange.from_slots(self._slots, *self._slots_of, self.shape)
            self._slots_dirty = False
        if self._stats_view_live():
            self.stats._fold()  # pylint: disable=protected-access

    def live_slots(self):
        """(dtype, device, slot buffer) while the running extrema lie in the slots and nowhere else, else None."""
        if self._slots_of is not None and (self._slots_dirty or self._stats_view_live()):
            return (*self._slots_of, self._slots)
        return None

    def _leave_slots(self):
        """`stats` becomes the one place the running extrema live in."""
        self._fold_slots()
        self._slots_of = None

    def _takes_slots(self, x: torch.Tensor) -> bool:
        return (self._single and x.is_cuda and x.dtype in _lib.DTYPE_CODE and x.is_contiguous() and x.numel() > 0
                and len(self.shape) <= x.dim())

    def _accumulate(self, x: torch.Tensor, copy_to: Optional[torch.Tensor], want_batch: bool):
        """One launch: the batch folded into the running slots, its copy written if asked for, its own extrema left
        in slots of their own if asked for.  False when the running statistics do not lie in slots of this dtype and
        device (the caller then takes the general route)."""
        of = (x.dtype, x.device)
        first = self._slots_of is None and self.stats.is_empty()
        if not (first or self._slots_of == of):
            return False
        if self._stats_view_live():
            self.stats._fold()  # pylint: disable=protected-access  (a view handed out earlier keeps what it saw)
        if self._slots is None or self._slots.device != x.device:
            self._slots = torch.empty(_lib.MINMAX_SLOTS_BYTES, dtype=torch.uint8, device=x.device)
        batch = torch.empty(_lib.MINMAX_SLOTS_BYTES, dtype=torch.uint8, device=x.device) if want_batch else None
        status = _lib.load().ahq_minmax_accumulate(_lib.DTYPE_CODE[x.dtype], x.data_ptr(), x.numel(),
                                                   None if copy_to is None else copy_to.data_ptr(),
                                                   self._slots.data_ptr(), None if batch is None else batch.data_ptr(),
                                                   1 if first else 0, _lib.current_stream(x.device))
        if status:
            _lib.check(status, "ahq_minmax_accumulate")
        self._slots_of = of
        self._slots_dirty = True
        return _MinMaxRange.from_slots(batch, x.dtype, x.device, self.shape) if want_batch else True

    @torch.no_grad()
    def collect_stats(self, input_tensor: torch.Tensor) -> _MinMaxRange:
        mn, mx = reduce_min_max(input_tensor, self.shape, self.block_size)
        return _MinMaxRange(mn, mx)

    @torch.no_grad()
    def merge_stats(self, stats: _MinMaxRange):
        self._leave_slots()
        self.__dict__["_stats_shared"] = False  # new tensors below
        new_min, new_max = self.stats.min, self.stats.max
        if stats.min is not None:
            new_min = stats.min.clone() if new_min is None else torch.minimum(new_min, stats.min)
        if stats.max is not None:
            new_max = stats.max.clone() if new_max is None else torch.maximum(new_max, stats.max)
        self.stats = _MinMaxRange(new_min, new_max)

    @torch.no_grad()
    def update(self, input_tensor: torch.Tensor, copy_to: Optional[torch.Tensor] = None) -> _MinMaxRange:
        """collect + merge in one launch: the running fold happens where the reduction finishes.  ``copy_to``
        receives a copy of the input from the same pass (what pass-through calibration returns)."""
        x = input_tensor
        if self._takes_slots(x) and (copy_to is None or (copy_to.dtype == x.dtype and copy_to.device == x.device
                                                         and copy_to.shape == x.shape and copy_to.is_contiguous())):
            batch = self._accumulate(x.detach(), copy_to, True)
            if batch is not False:
                return batch
        self._leave_slots()
        cur = self.stats
        if cur.min is None and cur.max is None:
            # the first batch: its extrema ARE the running statistics.  The two objects share their tensors until
            # somebody is about to write into the running ones (_own_stats), so a calibration on one batch -- every
            # weight -- makes no copies
            mn, mx = reduce_min_max(input_tensor, self.shape, self.block_size, copy_to=copy_to)
            self.stats = _MinMaxRange(mn, mx)
            self.__dict__["_stats_shared"] = True
            return _MinMaxRange(mn, mx)
        fused = (
            cur.min is not None and cur.max is not None
            and cur.min.dtype == input_tensor.dtype and cur.min.device == input_tensor.device
            and cur.min.is_contiguous() and cur.max.is_contiguous()
        )
        if fused:
            cur = self._own_stats()
            mn, mx = reduce_min_max(input_tensor, self.shape, self.block_size, running=(cur.min, cur.max),
                                    copy_to=copy_to)
            return _MinMaxRange(mn, mx)
        mn, mx = reduce_min_max(input_tensor, self.shape, self.block_size, copy_to=copy_to)
        new = _MinMaxRange(mn, mx)
        self.merge_stats(new)
        return new

    def _own_stats(self) -> _MinMaxRange:
        """The running statistics as tensors nobody else holds: whoever writes into them in place asks here first."""
        if self.__dict__.get("_stats_shared"):
            cur = self.stats
            self.stats = _MinMaxRange(None if cur.min is None else cur.min.clone(),
                                      None if cur.max is None else cur.max.clone())
            self.__dict__["_stats_shared"] = False
        return self.stats

    @torch.no_grad()
    def observe_and_clone(self, input_tensor: torch.Tensor) -> torch.Tensor:
        """update() for a caller that throws the batch's own statistics away and wants a copy of the input (the
        pass-through calibration of a whole model: hundreds of these per forward pass).  Once the running statistics
        exist, everything that does not change from call to call -- layout, workspace, the two tensors the batch's
        extrema are written to -- is kept, and a call is one allocation (the copy) and one library call."""
        x = input_tensor
        if self._takes_slots(x) and not x.requires_grad:
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
            if self._accumulate(x, out, False) is not False:
                return out
        self._leave_slots()
        fast = self.__dict__.get("_fast")
        cur = self.stats
        key = (x.shape, x.dtype, x.device)
        if (fast is None or fast[0] != key or fast[1] is not cur.min or fast[2] is not cur.max or not x.is_contiguous()
                or x.requires_grad):
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
            self.update(x, copy_to=out)  # (the batch's own extrema are dropped here, so nobody shares the tensors)
            self.__dict__["_stats_shared"] = False
            cur = self.stats
            self.__dict__["_fast"] = None
            if (x.is_contiguous() and x.is_cuda and cur.min is not None and cur.min.dtype == x.dtype
                    and cur.min.device == x.device and cur.min.is_contiguous() and cur.max.is_contiguous()):
                lib = _lib.load()
                _, layout = _prepare(x.detach(), self.shape, self.block_size)
                nbytes = lib.ahq_minmax_workspace_bytes(layout)
                ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
                bmin, bmax = torch.empty_like(cur.min), torch.empty_like(cur.max)
                # plain data only: the observer is deep-copied and pickled with its quantizer, and a ctypes function
                # pointer can be neither
                self.__dict__["_fast"] = (key, cur.min, cur.max, layout, ws, nbytes, bmin, bmax, _lib.DTYPE_CODE[x.dtype])
            return out
        _, rmin, rmax, layout, ws, nbytes, bmin, bmax, code = fast
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        status = _lib.load().ahq_minmax_copy(code, layout, x.data_ptr(), out.data_ptr(), bmin.data_ptr(),
                                             bmax.data_ptr(), rmin.data_ptr(), rmax.data_ptr(), 0, ws.data_ptr(), nbytes,
                                             _lib.current_stream(x.device))
        if status:
            _lib.check(status, "ahq_minmax_copy")
        return out

    def reset_stats(self):
        self.stats = _MinMaxRange()
        self._slots_of = None
        self._slots_dirty = False
        self.__dict__["_fast"] = None

    def get_stats(self) -> _MinMaxRange:
        if self._slots_of is not None and self._slots_dirty:
            # a view of the running slots: folded when it is read, or inside the launch of a consumer that takes
            # slots, and at the latest before the next batch changes them
            self.stats = _MinMaxRange.from_slots(self._slots, *self._slots_of, self.shape)
            self._slots_dirty = False
        return self.stats


class _HistogramObserver(_Observer[_Histogram]):
    """Running per-encoding histograms (reference: encoding_analyzer.py:121-338).

    State lives in fp32 device tensors: ``hist [S, B]``, ``edges [S, B+1]``, ``minmax [S, 2]``, ``limits [S, 2]``.
    One library call per batch produces the batch's own histogram and folds the batch into the running one."""

    def __init__(self, shape, *, block_size=None, num_bins: int, growth_limit: Optional[float] = None):
        super().__init__(shape, block_size)
        self.num_bins = num_bins
        self.num_slots = int(math.prod(self.shape))
        if growth_limit is None:
            growth_limit = float("inf")
        if growth_limit < 1.0:
            raise RuntimeError(f"Growth limit must be at least 1.0. Got {growth_limit}")
        self.growth_limit = growth_limit
        self._state = None          # dict of device tensors
        self._has_stats = False
        self._stat_dtype = None     # dtype of stats.min / stats.max as the reference would hold them
        self._stats_cache = None

    # ---------------------------------------------------------------------------------------------- internals --
    def _alloc(self, device) -> dict:
        S, B = self.num_slots, self.num_bins
        f = dict(dtype=torch.float32, device=device)
        return {
            "hist": torch.zeros(S, B, **f), "edges": torch.zeros(S, B + 1, **f),
            "minmax": torch.zeros(S, 2, **f), "limits": torch.zeros(S, 2, **f),
        }

    def _run(self, x: torch.Tensor, state: dict, first: bool, batch_hist: bool = True, batch_stats: bool = True):
        """One ahq_hist_update call.  Returns (new_hist, new_edges, new_minmax): the batch's own counts if
        ``batch_hist``, its own edges and min / max if ``batch_stats`` (None otherwise)."""
        batch_stats = batch_stats or batch_hist
        _lib.require_device(x, "input tensor")
        if x.dtype not in _lib.DTYPE_CODE:
            raise HipLibraryError(f"histogram statistics support float32, float16 and bfloat16; got {x.dtype}")
        try:
            _check_reducible(x, self.shape, self.block_size)
        except RuntimeError as e:
            raise RuntimeError(f"Shape {self.shape} is incompatible with input of shape {x.shape}") from e
        if x.numel() == 0:
            raise RuntimeError("cannot observe an empty tensor")
        lib = _lib.load()
        S, B = self.num_slots, self.num_bins
        xd, layout = _prepare(x.detach(), self.shape, self.block_size)
        f = dict(dtype=torch.float32, device=x.device)
        new_hist = torch.empty(S, B, **f) if batch_hist else None
        new_edges = torch.empty(S, B + 1, **f) if batch_stats else None
        new_minmax = torch.empty(S, 2, **f) if batch_stats else None
        st = _lib.HistState()
        st.num_slots, st.num_bins, st.growth_limit = S, B, self.growth_limit
        st.hist, st.edges = state["hist"].data_ptr(), state["edges"].data_ptr()
        st.minmax, st.limits = state["minmax"].data_ptr(), state["limits"].data_ptr()
        st.new_hist = new_hist.data_ptr() if batch_hist else None
        st.new_edges = new_edges.data_ptr() if batch_stats else None
        st.new_minmax = new_minmax.data_ptr() if batch_stats else None
        code = _lib.DTYPE_CODE[x.dtype]
        nbytes = lib.ahq_hist_update_workspace_bytes(code, layout, B)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        _lib.check(
            lib.ahq_hist_update(code, layout, xd.data_ptr(), st, 1 if first else 0, ws.data_ptr(), nbytes,
                                _lib.current_stream(x.device)),
            "ahq_hist_update",
        )
        return new_hist, new_edges, new_minmax

    @staticmethod
    def _as_list(hist, edges, minmax, dtype) -> "_HistogramList":
        return _HistogramList(hist, edges, minmax, dtype)

    # --------------------------------------------------------------------------------------------------- API --
    @torch.no_grad()
    def collect_stats(self, input_tensor: torch.Tensor) -> List[_Histogram]:
        scratch = self._alloc(input_tensor.device)
        h, e, mm = self._run(input_tensor, scratch, first=True)
        return self._as_list(h, e, mm, input_tensor.dtype)

    @torch.no_grad()
    def update(self, input_tensor: torch.Tensor) -> List[_Histogram]:
        """collect_stats + merge_stats with a single binning pass over the tensor.

        After the first batch, the returned batch statistics are formed when they are first read, from the tensor
        that was passed in: the running histogram only needs to know whether the batch reaches beyond the running
        range (reference: merge_stats, encoding_analyzer.py:260-331, bins the tensor itself onto the running range),
        a calibration loop discards the batch statistics, and without them a batch inside the running range is read
        once instead of twice, with one histogram update per element instead of two.  The returned object keeps the
        tensor alive until then; a caller that modifies the tensor in place before reading the statistics gets those
        of the modified tensor."""
        first = not self._has_stats
        if first or self._state["hist"].device != input_tensor.device:
            if not first:
                raise RuntimeError("histogram statistics live on a different device than the input")
            self._state = self._alloc(input_tensor.device)
        h, e, mm = self._run(input_tensor, self._state, first, batch_hist=first, batch_stats=first)
        # the reference keeps the first batch's min/max in the tensor dtype; after a merge they are float32
        self._stat_dtype = input_tensor.dtype if first else torch.promote_types(self._stat_dtype, torch.float32)
        self._has_stats = True
        self._stats_cache = None
        if first:
            return self._as_list(h, e, mm, input_tensor.dtype)
        held = input_tensor.detach()

        def collect():
            return self._run(held, self._alloc(held.device), first=True)

        return _HistogramList(None, None, None, input_tensor.dtype, count=self.num_slots, make=collect)

    @torch.no_grad()
    def merge_stats(self, new_stats_list: List[_Histogram], input_tensor: torch.Tensor):  # pylint: disable=arguments-differ
        # the fused update recomputes the batch statistics while it bins the batch onto the running range
        del new_stats_list
        self.update(input_tensor)

    def reset_stats(self):
        self._state = None
        self._has_stats = False
        self._stat_dtype = None
        self._stats_cache = None

    def get_stats(self) -> List[_Histogram]:
        if not self._has_stats:
            return _HistogramList(None, None, None, None, count=self.num_slots)
        if self._stats_cache is None:
            s = self._state
            self._stats_cache = self._as_list(s["hist"], s["edges"], s["minmax"], self._stat_dtype)
        return self._stats_cache

    @property
    def stats(self) -> List[_Histogram]:
        return self.get_stats()


class EncodingAnalyzer(Generic[_Statistics], ABC):
    """Gathers statistics of input data and computes encodings from them."""

    def __init__(self, observer: _Observer):
        self.observer = observer

    @torch.no_grad()
    def update_stats(self, input_tensor: torch.Tensor):
        """Update the running statistics with ``input_tensor``; returns the statistics of this tensor alone."""
        return self.observer.update(input_tensor)

    def reset_stats(self):
        self.observer.reset_stats()

    def compute_encodings(self, num_steps: int, is_symmetric: bool):
        """(min, max) of the encoding for a grid of ``num_steps`` steps."""
        return self.compute_encodings_from_stats(self.observer.get_stats(), num_steps, is_symmetric)

    def compute_dynamic_encodings(self, input_tensor: torch.Tensor, num_steps: int, is_symmetric: bool):
        return self.compute_encodings_from_stats(self.observer.collect_stats(input_tensor), num_steps, is_symmetric)

    @abstractmethod
    def compute_encodings_from_stats(self, stats, num_steps: int, is_symmetric: bool): ...


class MinMaxEncodingAnalyzer(EncodingAnalyzer[_MinMaxRange]):
    """Min-max calibration: the encoding range is [min(input), max(input)], widened to contain zero and to be
    representable (reference: encoding_analyzer.py:397-481)."""

    def __init__(self, shape, block_size=None):
        super().__init__(_MinMaxObserver(shape, block_size))

    @torch.no_grad()
    def update_stats_and_clone(self, input_tensor: torch.Tensor):
        """update_stats(input) and input.clone() with one read of the tensor.  Returns (batch statistics, clone)."""
        out = torch.empty(input_tensor.shape, dtype=input_tensor.dtype, device=input_tensor.device)
        return self.observer.update(input_tensor, copy_to=out), out

    def observe_and_clone(self, input_tensor: torch.Tensor) -> torch.Tensor:
        """update_stats(input) whose result nobody reads, and input.clone(), with one read of the tensor."""
        return self.observer.observe_and_clone(input_tensor)

    @torch.no_grad()
    def compute_encodings_from_stats(self, stats: _MinMaxRange, num_steps: int, is_symmetric: bool):
        if num_steps <= 0:
            raise ValueError("The number of quantization bins cannot be less than or equal to 0.")
        if stats.is_empty() or (stats.unfolded() is None and (stats.min is None or stats.max is None)):
            raise StatisticsNotFoundError("No statistics present to compute encodings.")

        fused = self._fused_encodings(stats, num_steps, is_symmetric)
        if fused is not None:
            return fused

        tiny = _get_minimum_scale(num_steps)
        lo = torch.clamp(stats.min, max=0)
        hi = torch.clamp(stats.max, min=0)
        # ranges narrower than the minimum scale are widened by it (this fp32 term promotes 16-bit statistics)
        widen = tiny * (true_divide(hi - lo, num_steps) < tiny)
        if is_symmetric:
            pos, neg = math.floor(num_steps / 2), math.ceil(num_steps / 2)
            hi = hi + pos * widen
            lo = lo - neg * widen
            # a 2-bit signed grid would waste a level on the negative side: calibrate as if it had one more
            extra = 1 if num_steps == 3 else 0
            delta = torch.maximum(true_divide(hi, pos + extra), true_divide(-lo, neg))
            lo = (-1 * neg) * delta
            hi = pos * delta
        else:
            hi = hi + num_steps * widen
        hi = torch.clamp(hi, max=torch.finfo(stats.min.dtype).max).to(stats.min.dtype)
        lo = torch.clamp(lo, min=torch.finfo(stats.max.dtype).min).to(stats.max.dtype)
        return lo, hi


    @staticmethod
    def _fused_encodings(stats: _MinMaxRange, num_steps: int, is_symmetric: bool):
        """The arithmetic below in one kernel launch (ahq_minmax_to_encodings); None when the statistics are not a
        pair of same-shaped 16/32-bit float tensors, in which case the elementwise formulation runs.  Statistics that
        still lie in the streaming kernel's slots are folded by the same launch (ahq_minmax_slots_to_encodings)."""
        slots = stats.unfolded()
        if slots is not None and 0 < num_steps <= (1 << 24) and num_steps == int(num_steps):
            dt, device, shape, buf = slots
            num_steps = int(num_steps)
            consts = _scalar_constants(dt, _get_minimum_scale(num_steps))
            out = torch.empty((4,) + tuple(shape), dtype=dt, device=device)  # lo, hi and the folded statistics
            flags = torch.zeros(2, dtype=torch.int32, device=device)
            base, step = out.data_ptr(), out.element_size()
            status = _lib.load().ahq_minmax_slots_to_encodings(
                _lib.DTYPE_CODE[dt], buf.data_ptr(), num_steps, 1 if is_symmetric else 0, consts[0], consts[1],
                consts[2], consts[3], base, base + step, base + 2 * step, base + 3 * step, flags.data_ptr(),
                _lib.current_stream(device))
            if status:
                _lib.check(status, "ahq_minmax_slots_to_encodings")
            lo, hi = out[0], out[1]
            stats.adopt(out[2], out[3])
            lo._ahq_range_flags = hi._ahq_range_flags = flags  # pylint: disable=protected-access
            return lo, hi
        mn, mx = stats.min, stats.max
        if (mn.dtype not in _lib.DTYPE_CODE or mx.dtype != mn.dtype or mn.shape != mx.shape or not mn.is_cuda
                or num_steps > (1 << 24) or num_steps != int(num_steps)):
            return None
        num_steps = int(num_steps)  # callers may hand over 2.0 ** bitwidth - 1
        dt = mn.dtype
        tiny = _get_minimum_scale(num_steps)
        consts = _scalar_constants(dt, tiny)
        mn, mx = mn.contiguous(), mx.contiguous()
        lo, hi = torch.empty_like(mn), torch.empty_like(mx)
        flags = torch.zeros(2, dtype=torch.int32, device=mn.device)
        lib = _lib.load()
        _lib.check(lib.ahq_minmax_to_encodings(_lib.DTYPE_CODE[dt], mn.data_ptr(), mx.data_ptr(), mn.numel(), num_steps,
                                               1 if is_symmetric else 0, consts[0], consts[1], consts[2], consts[3],
                                               lo.data_ptr(), hi.data_ptr(), flags.data_ptr(),
                                               _lib.current_stream(mn.device)), "ahq_minmax_to_encodings")
        lo._ahq_range_flags = hi._ahq_range_flags = flags  # pylint: disable=protected-access
        return lo, hi


@functools.lru_cache(maxsize=256)
def _scalar_constants(dtype: torch.dtype, tiny: float):
    """(minimum scale as `dtype` sees it, as float32, finfo(dtype).max, the near-overflow threshold in `dtype`)."""
    big = torch.finfo(dtype).max
    return (float(torch.tensor(tiny, dtype=dtype)), float(torch.tensor(tiny, dtype=torch.float32)), float(big),
            float(torch.tensor(1e-8 + 0.05 * big, dtype=dtype)))


_deferred_range_flags = None  # list of device flag pairs while deferred_range_warnings() is active
_deferred_shared_flags = None  # device -> int32[2] that kernels OR into while it is active


@contextlib.contextmanager
def deferred_range_warnings():
    """Inside this context the non-finite / near-overflow checks of every quantizer are gathered on the device and
    read back once on exit, instead of one host synchronisation per quantizer (a whole-model calibration ends
    hundreds of quantizer contexts at once).  The same warnings are issued, at the end."""
    global _deferred_range_flags, _deferred_shared_flags  # pylint: disable=global-statement
    if _deferred_range_flags is not None:
        yield
        return
    _deferred_range_flags = []
    _deferred_shared_flags = {}
    try:
        yield
    finally:
        flags, _deferred_range_flags = _deferred_range_flags, None
        shared, _deferred_shared_flags = _deferred_shared_flags, None
        flags += [f != 0 for f in shared.values()]
        if flags:
            by_device = {}
            for f in flags:
                by_device.setdefault(f.device, []).append(f)
            for group in by_device.values():
                _warn_range_flags(*torch.stack(group).any(dim=0).tolist())


def _range_flags_buffer(device):
    """(int32[2] on ``device`` for a kernel to OR its range flags into, whether the caller has to report it itself).
    Inside deferred_range_warnings() all kernels on a device share one buffer, read back when the context ends."""
    if _deferred_shared_flags is not None:
        buf = _deferred_shared_flags.get(device)
        if buf is None:
            buf = _deferred_shared_flags[device] = torch.zeros(2, dtype=torch.int32, device=device)
        return buf, False
    return torch.zeros(2, dtype=torch.int32, device=device), True


def _report_range_flags(flags: torch.Tensor):
    _warn_range_flags(*(v != 0 for v in flags.tolist()))  # one device-to-host read, no launch


def _warn_range_flags(nonfinite: bool, extreme: bool):
    if nonfinite:
        warnings.warn("Infinite or NaN values detected within input! This may skew the associated encodings")
    if extreme:
        warnings.warn("Extreme values detected within input! This may skew the associated encodings")


def _flag_extreme_min_max(curr_min, curr_max):
    """Warn about non-finite or near-overflow encodings (reference: encoding_analyzer.py:484-498)."""
    flags = getattr(curr_min, "_ahq_range_flags", None)
    if flags is not None and getattr(curr_max, "_ahq_range_flags", None) is flags:
        # already evaluated by the kernel that produced this pair
        if _deferred_range_flags is not None:
            _deferred_range_flags.append(flags != 0)
            return
        _report_range_flags(flags)
        return
    big = torch.finfo(curr_min.dtype).max
    both = torch.stack([curr_min.reshape(-1), curr_max.reshape(-1)]).abs()
    nonfinite = ~torch.isfinite(both).all()
    # torch.isclose(|x|, big, rtol=0.05) with its default atol of 1e-8: | |x| - big | <= 1e-8 + 0.05 * big
    extreme = ((both - big).abs() <= 1e-8 + 0.05 * big).any()
    flags = torch.stack([nonfinite, extreme])
    if _deferred_range_flags is not None:
        _deferred_range_flags.append(flags)
        return
    _warn_range_flags(*flags.tolist())  # both answers in one device-to-host read


def adjust_min_max(curr_min, curr_max, num_steps, is_symmetric):
    """Make a (min, max) pair contain zero, finite and at least minimum_scale wide; symmetric grids are re-centred
    (reference: encoding_analyzer.py:501-534).  Works on tensors of any shape."""
    tiny = _get_minimum_scale(num_steps)
    curr_min = torch.minimum(curr_min, torch.zeros_like(curr_min))
    curr_max = torch.maximum(curr_max, torch.zeros_like(curr_max))
    curr_min = curr_min.clamp(min=torch.finfo(curr_max.dtype).min, max=0)
    curr_max = curr_max.clamp(min=0, max=torch.finfo(curr_max.dtype).max)
    narrow = true_divide(curr_max - curr_min, num_steps) < tiny
    if is_symmetric:
        curr_min = torch.where(narrow, curr_min - tiny * math.ceil(num_steps / 2), curr_min)
        curr_max = torch.where(narrow, curr_max + tiny * math.floor(num_steps / 2), curr_max)
        pos, neg = math.floor(num_steps / 2), math.ceil(num_steps / 2)
        delta = torch.maximum(true_divide(curr_max, pos), true_divide(-curr_min, neg))
        curr_min = (-1 * neg) * delta
        curr_max = pos * delta
    else:
        curr_max = torch.where(narrow, curr_max + tiny * num_steps, curr_max)
    return curr_min, curr_max


class _HistogramAnalyzer(EncodingAnalyzer[_Histogram]):
    def _stack(self, stats: List[_Histogram]):
        """(hist [S,B], edges [S,B+1], minmax [S,2] fp32, dtype of min/max) from a list of per-slot statistics."""
        obs = self.observer
        if stats is obs.get_stats() and obs._has_stats:  # pylint: disable=protected-access
            s = obs._state  # pylint: disable=protected-access
            return s["hist"], s["edges"], s["minmax"], obs._stat_dtype  # pylint: disable=protected-access
        if isinstance(stats, _HistogramList) and stats.stacked()[0] is not None:
            return stats.stacked()
        hist = torch.stack([s.histogram for s in stats]).contiguous()
        edges = torch.stack([s.bin_edges for s in stats]).contiguous()
        dtype = stats[0].min.dtype
        mm = torch.stack([torch.stack((s.min, s.max)) for s in stats]).to(torch.float32).contiguous()
        return hist, edges, mm, dtype


class PercentileEncodingAnalyzer(_HistogramAnalyzer):
    """Percentile calibration: clip (100 - p)% of the largest and smallest observed values
    (reference: encoding_analyzer.py:538-650)."""

    def __init__(self, shape, num_bins: int = 2048, percentile: float = 100, block_size=None):
        if num_bins <= 0:
            raise ValueError("Number of bins cannot be less than or equal to 0.")
        super().__init__(_HistogramObserver(shape=shape, num_bins=num_bins, block_size=block_size))
        self.set_percentile(percentile)

    def set_percentile(self, percentile):
        if percentile < 50 or percentile > 100:
            raise ValueError("Percentile value must be within 50-100 range")
        self.percentile = percentile

    @torch.no_grad()
    def compute_encodings_from_stats(self, stats: List[_Histogram], num_steps: int, is_symmetric: bool):
        if num_steps <= 0:
            raise ValueError("The number of quantization bins cannot be less than or equal to 0.")
        if stats[0].histogram is None:
            raise StatisticsNotFoundError("No statistics present to compute encodings.")
        hist, edges, _, dtype = self._stack(stats)
        B = hist.shape[1]
        if self.percentile == 100:
            lo, hi = edges[:, 0], edges[:, B]
        else:
            cs = torch.cumsum(hist, dim=1)
            total = cs[:, -1:]
            hi_i = torch.searchsorted(cs, total * self.percentile / 100).clamp_(max=B)
            lo_i = torch.searchsorted(cs, total * (1 - self.percentile / 100)).clamp_(max=B)
            lo = torch.gather(edges, 1, lo_i).squeeze(1)
            hi = torch.gather(edges, 1, hi_i).squeeze(1)
        lo, hi = adjust_min_max(lo, hi, num_steps, is_symmetric)
        return lo.to(dtype).reshape(self.observer.shape), hi.to(dtype).reshape(self.observer.shape)


class _LpNormEncodingAnalyzer(_HistogramAnalyzer):
    """Searches (delta, offset) candidates for the lowest expected p-norm quantization + gamma * clipping noise
    over the histogram (reference: encoding_analyzer.py:653-899).  The whole search is one library call."""

    def __init__(self, shape, num_bins: int, *, p: float, asymmetric_delta_candidates: int,
                 symmetric_delta_candidates: int, offset_candidates: int, max_parallelism: int, gamma: float,
                 histogram_growth_limit: Optional[float] = None, block_size=None):
        if num_bins <= 0:
            raise ValueError("Number of bins cannot be less than or equal to 0.")
        super().__init__(_HistogramObserver(shape=shape, num_bins=num_bins, growth_limit=histogram_growth_limit,
                                            block_size=block_size))
        self.p = p
        self.asym_delta_candidates = asymmetric_delta_candidates
        self.sym_delta_candidates = symmetric_delta_candidates
        self.num_offset_candidates = offset_candidates
        self.gamma = gamma
        self.max_parallelism = max_parallelism  # kept for signature compatibility; the kernel needs no chunking
        self._offset_grid_cache = {}
        self.last_search = None

    def _offset_grid(self, num_steps: int, device) -> torch.Tensor:
        """round(arange(-num_steps, step, step)) evaluated on the CPU (torch.arange computes in double there),
        then kept on the device."""
        key = (num_steps, self.num_offset_candidates, str(device))
        grid = self._offset_grid_cache.get(key)
        if grid is None:
            n_off = min(num_steps + 2, self.num_offset_candidates)
            step = num_steps / (n_off - 2)
            grid = torch.round(torch.arange(start=-num_steps, end=step, step=step, dtype=torch.float32)).to(device)
            self._offset_grid_cache[key] = grid
        return grid

    @torch.no_grad()
    def compute_encodings_from_stats(self, stats: List[_Histogram], num_steps: int, is_symmetric: bool):
        if stats[0].histogram is None:
            raise StatisticsNotFoundError("No statistics present to compute encodings.")
        if num_steps <= 0:
            raise ValueError("The number of quantization bins cannot be less than or equal to 0.")
        num_steps = int(num_steps)
        hist, edges, minmax, dtype = self._stack(stats)
        device = hist.device
        lib = _lib.load()
        S, B = hist.shape
        prm = _lib.SqnrParams()
        prm.num_slots, prm.num_bins = S, B
        prm.symmetric = 1 if is_symmetric else 0
        prm.stat_dtype = _lib.DTYPE_CODE[dtype]
        prm.num_steps = num_steps
        prm.minimum_scale = _get_minimum_scale(num_steps)
        prm.gamma, prm.p = float(self.gamma), float(self.p)
        grid = None
        if is_symmetric:
            prm.num_deltas, prm.num_offsets = self.sym_delta_candidates, 1
        else:
            grid = self._offset_grid(num_steps, device)
            prm.num_deltas, prm.num_offsets = self.asym_delta_candidates, grid.numel() + 1
        D, O = prm.num_deltas, prm.num_offsets
        f = dict(dtype=torch.float32, device=device)
        noise = torch.empty(S, D, O, **f)
        deltas = torch.empty(S, D, O, **f)
        offsets = torch.empty(S, D, O, **f)
        out = torch.empty(S, 4, **f)
        best = torch.empty(S, dtype=torch.int64, device=device)
        _lib.check(
            lib.ahq_sqnr_search(prm, hist.data_ptr(), edges.data_ptr(), minmax.data_ptr(), _lib.ptr(grid),
                                noise.data_ptr(), deltas.data_ptr(), offsets.data_ptr(), out.data_ptr(),
                                best.data_ptr(), _lib.current_stream(device)),
            "ahq_sqnr_search",
        )
        self.last_search = {"noise": noise, "deltas": deltas, "offsets": offsets, "best_index": best,
                            "best_delta": out[:, 0], "best_offset": out[:, 1]}
        shape = self.observer.shape
        return out[:, 2].to(dtype).view(shape), out[:, 3].to(dtype).view(shape)


class SqnrEncodingAnalyzer(_LpNormEncodingAnalyzer):
    """SQNR calibration (p = 2) (reference: encoding_analyzer.py:902-953)."""

    def __init__(self, shape, num_bins: int = 2048, *, asymmetric_delta_candidates=17, symmetric_delta_candidates=101,
                 offset_candidates=21, max_parallelism=64, gamma=3.0, histogram_growth_limit: Optional[float] = None,
                 block_size=None):
        super().__init__(shape=shape, num_bins=num_bins, p=2.0,
                         asymmetric_delta_candidates=asymmetric_delta_candidates,
                         symmetric_delta_candidates=symmetric_delta_candidates, offset_candidates=offset_candidates,
                         max_parallelism=max_parallelism, gamma=gamma, histogram_growth_limit=histogram_growth_limit,
                         block_size=block_size)


class TfEnhancedEncodingAnalyzer(SqnrEncodingAnalyzer):
    """SQNR analyzer with the fixed hyper-parameters of the legacy tf-enhanced scheme: 512 bins, 17 / 101 delta
    candidates, 21 offsets, gamma 3, histogram range limited to 3x the first input's range
    (reference: encoding_analyzer.py:956-1002)."""

    _V1_HISTOGRAM_NUM_BINS = 512
    _V1_ASYMMETRIC_DELTA_CANDIDATES = 17
    _V1_SYMMETRIC_DELTA_CANDIDATES = 101
    _V1_OFFSET_CANDIDATES = 21
    _V1_GAMMA = 3.0
    _V1_HISTOGRAM_MAX_GROWTH_RATE = 3.0

    def __init__(self, shape, block_size=None):
        super().__init__(shape=shape, num_bins=self._V1_HISTOGRAM_NUM_BINS,
                         asymmetric_delta_candidates=self._V1_ASYMMETRIC_DELTA_CANDIDATES,
                         symmetric_delta_candidates=self._V1_SYMMETRIC_DELTA_CANDIDATES,
                         offset_candidates=self._V1_OFFSET_CANDIDATES, gamma=self._V1_GAMMA,
                         histogram_growth_limit=self._V1_HISTOGRAM_MAX_GROWTH_RATE, block_size=block_size)

    @classmethod
    def set_growth_limit(cls, growth_limit: float):
        if growth_limit < 1.0:
            raise RuntimeError(f"Growth limit must be at least 1.0. Got {growth_limit}")
        cls._V1_HISTOGRAM_MAX_GROWTH_RATE = growth_limit
