"""Probabilistic LUT node: expectation of a sigmoid table under independent Bernoulli inputs.

API of difflut/nodes/probabilistic_node.py:153-335 (`raw_weights` [2^k, output_dim],
`temperature` and `binary_combinations` buffers, `weights` property).  Forward and backward
run in libdifflut_hip.so; the backward is the exact derivative of the forward expression
(what autograd gives the reference's CPU path).
"""
import torch
import torch.nn as nn

from .. import _native, ops
from ..registry import register_node
from .base_node import BaseNode
from .cuda import is_cuda_available
from .dwn_node import _identity_plan

DEFAULT_PROBABILISTIC_TEMPERATURE = 1.0
DEFAULT_PROBABILISTIC_EVAL_MODE = "expectation"
DEFAULT_PROBABILISTIC_USE_CUDA = True

_CUDA_EXT_AVAILABLE = _native.is_built()


def probabilistic_forward(input, raw_weights, temperature):
    """(batch, k), (2^k, output_dim) -> (batch, output_dim); autograd-aware."""
    plan = _identity_plan(input.shape[1], input.device)
    return ops.prob_layer(input, raw_weights.unsqueeze(0), plan, temperature)


@register_node("probabilistic")
class ProbabilisticNode(BaseNode):
    fused_kind = "probabilistic"

    def __init__(self, input_dim=None, output_dim=None, init_fn=None, init_kwargs=None, regularizers=None,
                 temperature=DEFAULT_PROBABILISTIC_TEMPERATURE, eval_mode=DEFAULT_PROBABILISTIC_EVAL_MODE,
                 use_cuda=DEFAULT_PROBABILISTIC_USE_CUDA):
        super().__init__(input_dim=input_dim, output_dim=output_dim, regularizers=regularizers, init_fn=init_fn,
                         init_kwargs=init_kwargs)
        self.register_buffer("temperature", torch.tensor(float(temperature)))
        assert eval_mode in {"expectation", "deterministic", "threshold"}, "Invalid eval_mode"
        self.eval_mode = eval_mode
        self.use_cuda = use_cuda and is_cuda_available()
        # one normal draw per node, then the initialiser (probabilistic_node.py:224-225)
        self.raw_weights = nn.Parameter(torch.randn(2 ** self.input_dim, self.output_dim))
        self._apply_init_fn(self.raw_weights, name="raw_weights")
        addresses = torch.arange(2 ** self.input_dim).unsqueeze(1)
        bits = (addresses >> torch.arange(self.input_dim).unsqueeze(0)) & 1  # input 0 is the LSB
        self.register_buffer("binary_combinations", bits.to(torch.float32))

    @property
    def weights(self):
        return torch.sigmoid(self.raw_weights / self.temperature.clamp(min=1e-6))

    def temperature_value(self):
        key = (self.temperature._version, self.temperature.data_ptr())
        if getattr(self, "_t_key", None) != key:
            self._t, self._t_key = float(self.temperature), key
        return self._t

    def forward_train(self, x):
        return probabilistic_forward(x, self.raw_weights, self.temperature_value())

    def forward_eval(self, x):
        plan = _identity_plan(x.shape[1], x.device)
        return ops.prob_layer_eval(x, self.raw_weights.detach().unsqueeze(0), plan, self.temperature_value())

    def _builtin_regularization(self):
        return torch.tensor(0.0, device=self.raw_weights.device)

    def extra_repr(self):
        return f"input_dim={self.input_dim}, output_dim={self.output_dim}"
