"""Encoder base class (interface of difflut/encoder/base_encoder.py:18-137)."""
from abc import ABC, abstractmethod

import torch
import torch.nn as nn

DEFAULT_ENCODER_NUM_BITS = 3
DEFAULT_ENCODER_FLATTEN = True


class BaseEncoder(nn.Module, ABC):
    """fit(data) learns the encoding parameters, encode(data) returns 0/1 floats:
    (batch, features * num_bits) when flatten else (batch, features, num_bits)."""

    def __init__(self, num_bits=DEFAULT_ENCODER_NUM_BITS, flatten=DEFAULT_ENCODER_FLATTEN):
        super().__init__()
        assert num_bits > 0, "num_bits must be positive"
        assert isinstance(flatten, bool), "flatten must be a boolean"
        self.num_bits, self.flatten = int(num_bits), flatten
        self._is_fitted = False

    @abstractmethod
    def fit(self, x):
        ...

    @abstractmethod
    def encode(self, x):
        ...

    def forward(self, x):
        return self.encode(x)

    @staticmethod
    def _to_tensor(x):
        return x if isinstance(x, torch.Tensor) else torch.tensor(x)

    def _check_fitted(self):
        if not self._is_fitted:
            raise RuntimeError(f"{self.__class__.__name__} must be fitted before encoding. Call fit() first with "
                               "your training data to compute encoding parameters.")

    @property
    def is_fitted(self):
        return self._is_fitted

    def to(self, device):
        """Encoder parameters are plain tensor attributes (not buffers): move each one."""
        for name, value in list(vars(self).items()):
            if not name.startswith("_") and isinstance(value, torch.Tensor):
                setattr(self, name, value.to(device))
        return self

    def __repr__(self):
        return f"{self.__class__.__name__}(num_bits={self.num_bits}, flatten={self.flatten})"
