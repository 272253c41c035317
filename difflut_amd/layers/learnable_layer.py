"""LearnableLayer: LUT layer whose input selection is learned.

Training: every node input is a softmax-weighted mix of all layer inputs,
m = x @ softmax(W / tau, -1).T; evaluation: the argmax input is selected.  Constructor,
`mapping.W` [output_size*n, input_size] (xavier-uniform), tau schedule and
`get_mapping_matrix` follow difflut/layers/learnable_layer.py:173-486.  The contraction, its
backward (softmax never materialised) and the hard selection run in libdifflut_hip.so.
"""
import warnings

import torch
import torch.nn as nn

from .. import _native, ops
from ..registry import register_layer
from ..utils.warnings import warn_default_value
from .base_layer import BaseLUTLayer

DEFAULT_LEARNABLE_LAYER_TAU = 0.001
DEFAULT_LEARNABLE_LAYER_TAU_START = 1.0
DEFAULT_LEARNABLE_LAYER_TAU_MIN = 0.0001
DEFAULT_LEARNABLE_LAYER_TAU_DECAY_ITERS = 1000.0
LEARNABLE_LAYER_CONNECTION_WARNING_THRESHOLD = 10
DEFAULT_LEARNABLE_LAYER_USE_CUDA_SOFT = False
_LEARNABLE_MAPPING_CUDA_AVAILABLE = _native.is_built()


class LearnableMappingModule(nn.Module):
    """W [output_size, input_size]; soft selection in training, cached argmax selection in eval.
    `output_size` is the layer's node count times inputs per node."""

    def __init__(self, input_size, output_size, tau=DEFAULT_LEARNABLE_LAYER_TAU,
                 use_cuda_soft=DEFAULT_LEARNABLE_LAYER_USE_CUDA_SOFT):
        super().__init__()
        self.input_size, self.output_size = input_size, output_size
        self.tau = tau
        self.use_cuda_soft = use_cuda_soft
        self.precision = 0  # 0: fp32 matrix cores; 1: bf16 operands with fp32 accumulation
        self.W = nn.Parameter(torch.randn(output_size, input_size))
        nn.init.xavier_uniform_(self.W)
        self.register_buffer("_cached_hard_indices", None)
        self.register_buffer("_cached_hard_mask", None)
        self._cache_valid = False
        self._hard_plan = None

    def train(self, mode=True):
        was_training = self.training
        super().train(mode)
        if mode and not was_training:
            self._cache_valid = False
        return self

    def _compute_hard_selection(self):
        with torch.no_grad():
            self._cached_hard_indices = ops.row_argmax(self.W.detach())
            self._hard_plan = ops.MappingPlan(self._cached_hard_indices.view(-1, 1), self.input_size)

    def forward(self, x):
        if self.training:
            return ops.soft_map(x, self.W, self.tau, self.precision)
        if (not self._cache_valid or self._cached_hard_indices is None or self._hard_plan is None
                or self._hard_plan.device != x.device):
            self._compute_hard_selection()
            self._cache_valid = True
        return ops.hard_select(x, self._cached_hard_indices, self._hard_plan)


@register_layer("learnable")
class LearnableLayer(BaseLUTLayer):
    def __init__(self, input_size, output_size, node_type, node_kwargs, tau=None, tau_start=None, tau_min=None,
                 tau_decay_iters=None, layer_config=None, flip_probability=None, grad_stabilization=None,
                 grad_target_std=None, grad_subtract_mean=None, grad_epsilon=None, use_cuda_soft=None):
        defaults = {"tau": DEFAULT_LEARNABLE_LAYER_TAU, "tau_start": DEFAULT_LEARNABLE_LAYER_TAU_START,
                    "tau_min": DEFAULT_LEARNABLE_LAYER_TAU_MIN, "tau_decay_iters": DEFAULT_LEARNABLE_LAYER_TAU_DECAY_ITERS,
                    "use_cuda_soft": DEFAULT_LEARNABLE_LAYER_USE_CUDA_SOFT}
        given = {"tau": tau, "tau_start": tau_start, "tau_min": tau_min, "tau_decay_iters": tau_decay_iters,
                 "use_cuda_soft": use_cuda_soft}
        for name, value in given.items():
            if value is None:
                given[name] = defaults[name]
                warn_default_value(name, defaults[name], stacklevel=2)
        if given["tau_start"] < given["tau_min"]:
            warnings.warn(f"LearnableLayer: tau_start ({given['tau_start']}) is less than tau_min "
                          f"({given['tau_min']}); tau will be clamped immediately.", UserWarning, stacklevel=2)
        super().__init__(input_size, output_size, node_type, node_kwargs, layer_config, flip_probability,
                         grad_stabilization, grad_target_std, grad_subtract_mean, grad_epsilon)
        connections = output_size * self.n
        if connections > input_size * LEARNABLE_LAYER_CONNECTION_WARNING_THRESHOLD:
            warnings.warn(f"LearnableLayer: Creating {connections} learnable connections from {input_size} inputs. "
                          "This may lead to overfitting.", UserWarning, stacklevel=2)
        self.tau_start, self.tau_min, self.tau_decay_iters = given["tau_start"], given["tau_min"], given["tau_decay_iters"]
        self.tau = self.tau_start  # training starts at tau_start, `tau` itself is only a placeholder
        self.use_cuda_soft = given["use_cuda_soft"]
        self.mapping = LearnableMappingModule(input_size, connections, self.tau, self.use_cuda_soft)
        self._node_plan = None

    def _identity_node_plan(self, device):
        """Nodes read the mapped tensor [batch, N*n] in order: node i takes columns i*n .. i*n+n-1."""
        if self._node_plan is None or self._node_plan.device != device:
            table = torch.arange(self.output_size * self.n, dtype=torch.int32, device=device)
            self._node_plan = ops.MappingPlan(table.view(self.output_size, self.n), self.output_size * self.n)
        return self._node_plan

    def get_mapping(self, x):
        return self.mapping(x).view(x.shape[0], self.output_size, self.n)

    def forward(self, x):
        self._validate_input_dims(x)
        mapped = self.mapping(x)  # [batch, N*n]
        out = self._run_nodes(mapped, self._identity_node_plan(mapped.device))
        if out is None:
            out = self._loop_nodes(mapped.view(x.shape[0], self.output_size, self.n))
        return out

    def get_mapping_matrix(self):
        with torch.no_grad():
            return ops.row_argmax(self.mapping.W.detach()).long().view(self.output_size, self.n)

    def update_tau(self, iteration):
        """tau = max(tau_start * 10^(-iteration / tau_decay_iters), tau_min)"""
        self.tau = max(self.tau_start * 10.0 ** (-iteration / self.tau_decay_iters), self.tau_min)
        self.mapping.tau = self.tau
        self.mapping._cache_valid = False

    def extra_repr(self):
        flip = f", flip_prob={self.flip_probability}" if self.flip_probability > 0 else ""
        stab = f", grad_stab={self.grad_stabilization}" if self.grad_stabilization != "none" else ""
        return (f"input_size={self.input_size}, output_size={self.output_size}, n={self.n}, tau={self.tau}, "
                f"mapping=learnable{flip}{stab}")
