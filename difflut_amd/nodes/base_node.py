"""Abstract LUT node: constructor validation, train/eval dispatch, regulariser plumbing.

Interface of difflut/nodes/base_node.py:22-371 - same constructor arguments, attributes
(input_dim, output_dim, num_inputs, num_outputs, regularizers, init_fn, init_kwargs) and
error types - so node subclasses written against the reference keep working.
"""
import itertools
import warnings
from abc import ABC, abstractmethod

import torch
import torch.nn as nn

from ..utils.warnings import warn_default_value

DEFAULT_NODE_INPUT_DIM = 6
DEFAULT_NODE_OUTPUT_DIM = 1
NODE_INPUT_DIM_WARNING_THRESHOLD = 10
NODE_OUTPUT_DIM_WARNING_THRESHOLD = 10


def _positive_int(name, value, example):
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ValueError(f"{name} must be a positive integer, but got {value}. Example: {name}={example}")


class BaseNode(nn.Module, ABC):
    """A node maps (batch, input_dim) to (batch, output_dim)."""

    # layers look at this to decide whether all nodes can run as one fused device call
    fused_kind = None

    def __init__(self, input_dim=None, output_dim=None, regularizers=None, init_fn=None, init_kwargs=None, **kwargs):
        super().__init__()
        if input_dim is None:
            input_dim = DEFAULT_NODE_INPUT_DIM
            warn_default_value("input_dim", input_dim, stacklevel=2)
        if output_dim is None:
            output_dim = DEFAULT_NODE_OUTPUT_DIM
            warn_default_value("output_dim", output_dim, stacklevel=2)
        _positive_int("input_dim", input_dim, 6)
        _positive_int("output_dim", output_dim, 1)
        self.input_dim, self.output_dim = input_dim, output_dim
        if input_dim > NODE_INPUT_DIM_WARNING_THRESHOLD:
            warnings.warn(f"input_dim={input_dim} is quite large: a LUT node stores 2^{input_dim} entries.",
                          UserWarning, stacklevel=2)
        if output_dim > NODE_OUTPUT_DIM_WARNING_THRESHOLD:
            warnings.warn(f"output_dim={output_dim} is quite large.", UserWarning, stacklevel=2)
        if init_fn is not None and not callable(init_fn):
            raise TypeError(f"init_fn must be callable, but got {type(init_fn).__name__}.")
        self.init_fn = init_fn
        self.init_kwargs = {} if init_kwargs is None else init_kwargs
        if not isinstance(self.init_kwargs, dict):
            raise TypeError(f"init_kwargs must be a dict, but got {type(self.init_kwargs).__name__}")
        self.regularizers = self._checked_regularizers(regularizers)

    def __setattr__(self, name, value):
        # a parameter or scalar buffer that a layer keeps in a bank is being replaced: the bank must re-tie
        params = self.__dict__.get("_parameters")
        if params is not None:
            old = params.get(name)
            if old is None:
                old = self.__dict__["_buffers"].get(name)
            bank = getattr(old, "_bank", None) or getattr(old, "_scalar_bank", None)
            if bank is not None:
                bank._stale = True
        super().__setattr__(name, value)

    @property
    def num_inputs(self):
        return self.input_dim

    @property
    def num_outputs(self):
        return self.output_dim

    @staticmethod
    def _checked_regularizers(regs):
        """{"name": [fn(node, **kw) -> scalar, weight, kwargs]}"""
        out = {}
        for name, spec in (regs or {}).items():
            if not isinstance(spec, (list, tuple)):
                raise ValueError(f"Regularizer '{name}' must be a list/tuple of [function, weight, kwargs], "
                                 f"but got {type(spec).__name__}.")
            if len(spec) != 3:
                raise ValueError(f"Regularizer '{name}' must have exactly 3 elements [function, weight, kwargs], "
                                 f"but got {len(spec)} elements.")
            fn, weight, kw = spec
            if not callable(fn):
                raise TypeError(f"Regularizer '{name}' function must be callable, but got {type(fn).__name__}.")
            if not isinstance(weight, (int, float)):
                raise TypeError(f"Regularizer '{name}' weight must be numeric, but got {type(weight).__name__}.")
            if not isinstance(kw, dict):
                raise TypeError(f"Regularizer '{name}' kwargs must be a dict, but got {type(kw).__name__}.")
            out[name] = [fn, weight, kw]
        return out

    def _apply_init_fn(self, param, name="parameter"):
        if self.init_fn is None:
            return
        try:
            self.init_fn(param, **self.init_kwargs)
        except Exception as exc:
            raise RuntimeError(f"Initialization of '{name}' failed with error: {exc}.")

    @abstractmethod
    def forward_train(self, x):
        """(batch, input_dim) -> (batch, output_dim), differentiable."""

    def forward_eval(self, x):
        return (self.forward_train(x) > 0.5).float()

    def forward(self, x):
        return self.forward_train(x) if self.training else self.forward_eval(x)

    def forward_with_mapping(self, x, mapping_indices):
        """x (batch, input_size) and indices (layer_size, input_dim) -> (batch, layer_size, output_dim).

        Default: materialise the mapped inputs and run forward() on them, as base_node.py:293-304.
        """
        rows = torch.arange(x.shape[0], device=x.device).view(-1, 1, 1)
        return self.forward(x[rows, mapping_indices])

    def _builtin_regularization(self):
        params = list(self.parameters())
        return torch.tensor(0.0, device=params[0].device if params else "cpu")

    def regularization(self):
        total = self._builtin_regularization()
        for name, (fn, weight, kw) in self.regularizers.items():
            try:
                total = total + weight * fn(self, **kw)
            except Exception as exc:
                raise RuntimeError(f"Regularizer '{name}' failed with error: {exc}.")
        return total

    def export_bitstream(self):
        """Outputs of forward_eval over all 2^input_dim binary inputs, first input most significant
        in the enumeration order (itertools.product), as base_node.py:347-371."""
        params = list(self.parameters())
        device = params[0].device if params else "cpu"
        combos = torch.tensor(list(itertools.product([0, 1], repeat=self.num_inputs)), dtype=torch.float32,
                              device=device)
        with torch.no_grad():
            out = self.forward_eval(combos)
        return [int(v > 0.5) for v in out.flatten().tolist()]
