"""GroupSum head (difflut/utils/modules.py:20-163): split the features into k contiguous groups
(zero-padded to a multiple of k), sum each group, divide by tau."""
import warnings

import torch
import torch.nn as nn

from .. import ops
from .warnings import warn_default_value

DEFAULT_GROUPSUM_K = 1
DEFAULT_GROUPSUM_TAU = 1.0
DEFAULT_GROUPSUM_USE_RANDPERM = False


class GroupSum(nn.Module):
    def __init__(self, k=None, tau=None, use_randperm=None):
        super().__init__()
        if k is None:
            k = DEFAULT_GROUPSUM_K
            warn_default_value("k (GroupSum)", k, stacklevel=2)
        if tau is None:
            tau = DEFAULT_GROUPSUM_TAU
            warn_default_value("tau (GroupSum)", tau, stacklevel=2)
        if use_randperm is None:
            use_randperm = DEFAULT_GROUPSUM_USE_RANDPERM
            warn_default_value("use_randperm (GroupSum)", use_randperm, stacklevel=2)
        if not isinstance(k, int) or k <= 0:
            raise ValueError(f"k must be a positive integer, got {k}")
        if not isinstance(tau, (int, float)) or tau <= 0:
            raise ValueError(f"tau must be a positive number, got {tau}")
        self.k, self.tau, self.use_randperm = k, tau, use_randperm

    def forward(self, x):
        if x.dim() != 2:
            raise ValueError(f"GroupSum expects 2D input (batch_size, num_features), but got shape {x.shape} "
                             f"with {x.dim()} dimensions.")
        batch, features = x.shape
        if batch == 0:
            raise ValueError(f"GroupSum requires non-empty batch, got batch_size={batch}")
        if features == 0:
            raise ValueError(f"GroupSum requires non-zero features, got num_features={features}.")
        if features < self.k:
            warnings.warn(f"GroupSum input has fewer features ({features}) than output groups ({self.k}).",
                          UserWarning, stacklevel=2)
        if self.use_randperm:
            x = x[:, torch.randperm(features, device=x.device)]
        if features % self.k != 0:
            warnings.warn(f"GroupSum: Input has {features} features which is not divisible by k={self.k}. Adding "
                          f"{self.k - features % self.k} zero-padded features.", UserWarning, stacklevel=2)
        return ops.group_sum(x, self.k, self.tau)


def cross_entropy(logits, labels):
    """Mean cross-entropy of [batch, classes] logits (e.g. what GroupSum returns) against int64 class labels, loss and
    gradient from one pass on the device: a drop-in for `torch.nn.functional.cross_entropy(logits, labels)` with
    its default mean reduction (no class weights, no label smoothing, no ignore_index)."""
    return ops.cross_entropy(logits, labels)

