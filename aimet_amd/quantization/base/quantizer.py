"""Quantizer base class: parameter registration with "has this parameter been initialised" tracking.

Counterpart of aimet_torch/quantization/base/quantizer.py:30-306.  A quantization parameter counts as initialised
once it has been written to (its tensor version changed) or replaced; the flags travel in the module's extra state so
that checkpoints restore them.
"""

from __future__ import annotations

import abc
import contextlib
import copy
import warnings
import weakref
from collections import OrderedDict
from typing import Optional

import torch
from torch import nn

__all__ = ["QuantizerBase"]


class QuantizerBase(abc.ABC, torch.nn.Module):
    """Quantizer base class"""

    def __init__(self):
        super().__init__()
        # name -> (weak reference to the parameter object registered first, its version at that time)
        self._initial_parameters = OrderedDict()
        self._is_overwrite_allowed: dict = OrderedDict()

    @abc.abstractmethod
    @contextlib.contextmanager
    def compute_encodings(self):
        """Observe inputs and update quantization parameters based on the input statistics."""

    @abc.abstractmethod
    def get_encodings(self):
        """Return the quantizer's encodings as an encoding object."""

    def get_encoding(self):
        """Deprecated alias of get_encodings() (base/quantizer.py:81-86)."""
        warnings.warn("get_encoding is deprecated: use get_encodings instead", DeprecationWarning, stacklevel=2)
        return self.get_encodings()

    def set_encodings(self, encodings):
        """Set the quantizer's encodings (base/quantizer.py:88-92: not implemented by the reference either)."""
        raise NotImplementedError

    @abc.abstractmethod
    def get_legacy_encodings(self):
        """The encodings as a list of dictionaries, one per channel; None before initialisation."""

    @abc.abstractmethod
    def set_legacy_encodings(self, encodings):
        """Take the encodings from a list in the form get_legacy_encodings() gives."""

    @classmethod
    @abc.abstractmethod
    def from_encodings(cls, encodings):
        """A quantizer that holds the given encoding object's encodings."""

    def register_quantization_parameter(self, name: str, param: Optional[nn.Parameter]):
        self.register_parameter(name, param)
        if param is not None:
            self._initial_parameters[name] = (weakref.ref(param), param._version)  # pylint: disable=protected-access

    def is_initialized(self, name: Optional[str] = None) -> bool:
        """True if every quantization parameter (or the named one) has been given a value."""
        # a quantizer's parameters are its own (no sub-modules hold any): the dictionary is walked directly, which is
        # an order of magnitude cheaper than named_parameters() and this runs several times per forward pass
        params = self._parameters
        if name is not None:
            p = params.get(name)
            return p is None or self._is_initialized(name, p)
        for n, p in params.items():
            if p is not None and not self._is_initialized(n, p):
                return False
        return True

    def _is_initialized(self, param_name: str, current: nn.Parameter) -> bool:
        ref, version = self._initial_parameters.get(param_name, (None, None))
        if ref is None:
            return True
        first = ref()
        if first is None or current is not first:
            return True
        return current._version != version  # pylint: disable=protected-access

    # ------------------------------------------------------------------------------------------ checkpointing --
    def get_extra_state(self):
        return {n: torch.tensor(self._is_initialized(n, p)) for n, p in self.named_parameters()}

    @torch.no_grad()
    def set_extra_state(self, state):
        for name, param in self._parameters.items():
            if name in state:
                self.register_quantization_parameter(name, param)
                if state[name]:
                    param.mul_(1.0)  # bumps the version: marks the parameter as initialised

    def load_state_dict(self, state_dict, *args, **kwargs):  # pylint: disable=arguments-differ
        if "_extra_state" not in state_dict:
            state_dict["_extra_state"] = OrderedDict(
                (n, torch.tensor(True)) for n in state_dict if n in self._parameters
            )
        return super().load_state_dict(state_dict, *args, **kwargs)

    @torch.no_grad()
    def __deepcopy__(self, memo):
        clone = type(self).__new__(type(self))
        clone.__dict__ = copy.deepcopy(self.__dict__, memo)
        clone.set_extra_state(self.get_extra_state())
        return clone

    def __getstate__(self):
        state = self.__dict__.copy()
        state.pop("_initial_parameters")
        state["is_initialized"] = self.get_extra_state()
        return state

    @torch.no_grad()
    def __setstate__(self, state):
        self._initial_parameters = OrderedDict()
        flags = state.pop("is_initialized")
        self.__dict__.update(state)
        self.set_extra_state(flags)

    # ----------------------------------------------------------------------------------------- overwrite flags --
    def allow_overwrite(self, *args, **kwargs):
        """allow_overwrite(mode) sets every flag; allow_overwrite(min=..., max=...) sets the named ones."""
        mode = kwargs.get("mode", args[0] if args else None)
        if mode is not None:
            update = {n: mode for n in self._is_overwrite_allowed}
        else:
            update = dict(kwargs)
        unexpected = sorted(set(update) - set(self._is_overwrite_allowed))
        if unexpected:
            raise RuntimeError(
                f"'allow_overwrite' expected param names {sorted(self._is_overwrite_allowed)};"
                f" got unexpected parameter names {unexpected}"
            )
        self._is_overwrite_allowed.update(update)

    def is_overwrite_allowed(self, name: Optional[str] = None) -> bool:
        if name is None:
            return any(self._is_overwrite_allowed.values())
        return self._is_overwrite_allowed[name]

    @property
    def _allow_overwrite(self) -> bool:
        """Deprecated spelling of is_overwrite_allowed() / allow_overwrite() (base/quantizer.py:293-302)."""
        warnings.warn("_allow_overwrite is deprecated: use is_overwrite_allowed() instead", DeprecationWarning, stacklevel=2)
        return self.is_overwrite_allowed()

    @_allow_overwrite.setter
    def _allow_overwrite(self, mode: bool):
        warnings.warn("_allow_overwrite is deprecated: use allow_overwrite() instead", DeprecationWarning, stacklevel=2)
        self.allow_overwrite(mode)

    @contextlib.contextmanager
    def _precompute_encodings(self, dtype=None):  # pylint: disable=unused-argument
        yield
