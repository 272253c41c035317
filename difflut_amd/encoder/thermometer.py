"""Thermometer encoder (difflut/encoder/thermometer.py:14-128): per feature, num_bits evenly
spaced thresholds strictly between the fitted minimum and maximum; bit j is (x > threshold j)."""
import warnings

import torch

from .. import ops
from ..registry import register_encoder
from .base_encoder import BaseEncoder

DEFAULT_THERMOMETER_NUM_BITS = 1


@register_encoder("thermometer")
class ThermometerEncoder(BaseEncoder):
    def __init__(self, num_bits=DEFAULT_THERMOMETER_NUM_BITS, flatten=True):
        super().__init__(num_bits=num_bits, flatten=flatten)
        self.thresholds = None

    def _compute_thresholds(self, x):
        """(features, num_bits): min + (j + 1) * (max - min) / (num_bits + 1); one-off pass over the data."""
        lo, hi = x.min(dim=0)[0], x.max(dim=0)[0]
        steps = torch.arange(1, self.num_bits + 1, device=x.device)
        return lo.unsqueeze(-1) + steps.unsqueeze(0) * ((hi - lo) / (self.num_bits + 1)).unsqueeze(-1)

    def fit(self, x):
        x = self._to_tensor(x)
        if self.num_bits > 32:
            warnings.warn(f"ThermometerEncoder: Using {self.num_bits} bits will create many features.", UserWarning,
                          stacklevel=2)
        self.thresholds = self._compute_thresholds(x)
        self._is_fitted = True
        return self

    def encode(self, x):
        self._check_fitted()
        x = self._to_tensor(x)
        lead = x.shape[:-1] if x.dim() > 2 else None
        x2 = x.reshape(-1, x.shape[-1]) if x.dim() != 2 else x
        bits = ops.thermometer_encode(x2, self.thresholds.to(x.device))
        if lead is not None:
            bits = bits.view(*lead, x.shape[-1], self.num_bits)
        return bits.reshape(bits.shape[0], -1) if self.flatten else bits

    def binarize(self, x):
        return self.encode(x)

    def get_thresholds(self, x):
        return self._compute_thresholds(x)
