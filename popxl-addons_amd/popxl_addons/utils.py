"""Small host-side containers used by the layers: named variables and a validating weight map."""
from collections.abc import MutableMapping

import numpy as np


class Variable:
    """A named device tensor owned by a layer (eager counterpart of a graph variable)."""

    def __init__(self, name, data):
        self.name = name
        self.data = data

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def shape(self):
        return tuple(self.data.shape)

    def __repr__(self):
        return f"Variable({self.name}, {self.dtype}, {self.shape})"


class NamedTensors:
    """Attribute/key access to a layer's variables by name."""

    def __init__(self, **tensors):
        self._tensors = dict(tensors)

    def __getattr__(self, name):
        try:
            return self.__dict__["_tensors"][name]
        except KeyError:
            raise AttributeError(name) from None

    def __getitem__(self, name):
        return self._tensors[name]

    def insert(self, name, value):
        self._tensors[name] = value

    def keys(self):
        return self._tensors.keys()

    def values(self):
        return self._tensors.values()

    def items(self):
        return self._tensors.items()

    def __contains__(self, name):
        return name in self._tensors

    def __len__(self):
        return len(self._tensors)


def _numpy_dtype_of(torch_dtype):
    import torch

    table = {
        torch.float16: np.float16,
        torch.float32: np.float32,
        torch.uint16: np.uint16,
        torch.int16: np.int16,
    }
    return np.dtype(table[torch_dtype])


class WeightsDict(MutableMapping):
    """Maps a layer's `Variable`s to numpy arrays and rejects an item whose dtype or shape differs
    from the variable's (popxl_addons/utils.py:79-99)."""

    def __init__(self, *args, **kwargs):
        self.dict = dict()
        if len(args) + len(kwargs) > 0:
            self.update(*args, **kwargs)

    def __getitem__(self, key):
        return self.dict[key]

    def __setitem__(self, key, value):
        value = np.asarray(value)
        expected = _numpy_dtype_of(key.dtype)
        if expected != value.dtype:
            raise ValueError(f"{key}: tensor and weight dtypes do not equal {expected} != {value.dtype}")
        if key.shape != tuple(value.shape):
            raise ValueError(f"{key}: tensor and weight shapes do not equal {key.shape} != {tuple(value.shape)}")
        self.dict[key] = value

    def __delitem__(self, key):
        del self.dict[key]

    def __len__(self):
        return len(self.dict)

    def __iter__(self):
        return iter(self.dict)
