"""Hybrid node: thresholded lookup forward (as DWN), probabilistic backward on the real-valued inputs.

API of difflut/nodes/hybrid_node.py:252-375 (constructor, `raw_luts` parameter [output_dim, 2^k],
`binary_combinations` buffer, `_get_luts`, train/eval forwards).  The arithmetic runs in
libdifflut_hip.so; a node called on its own goes through the whole-layer kernels with N = 1 and the
identity mapping.
"""
import torch
import torch.nn as nn

from .. import _native, ops
from ..registry import register_node
from .base_node import BaseNode
from .cuda import is_cuda_available
from .dwn_node import _identity_plan

DEFAULT_HYBRID_USE_CUDA = True

_HYBRID_CUDA_EXT_AVAILABLE = _native.is_built()


def hybrid_forward(input, luts, binary_combinations=None):
    """(batch, k) inputs and (output_dim, 2^k) table in [0, 1] -> (batch, output_dim); autograd-aware
    (hybrid_node.py:229-249).  `binary_combinations` is accepted for signature compatibility: the
    kernels enumerate the corners themselves (input 0 = least significant bit)."""
    plan = _identity_plan(input.shape[1], input.device)
    return ops.hybrid_layer(input, luts.unsqueeze(0), plan)


@register_node("hybrid")
class HybridNode(BaseNode):
    fused_kind = "hybrid"

    def __init__(self, input_dim=None, output_dim=None, use_cuda=DEFAULT_HYBRID_USE_CUDA, regularizers=None,
                 init_fn=None, init_kwargs=None):
        super().__init__(input_dim=input_dim, output_dim=output_dim, regularizers=regularizers, init_fn=init_fn,
                         init_kwargs=init_kwargs)
        self.use_cuda = use_cuda and is_cuda_available()
        # one normal draw per node, then the initialiser (hybrid_node.py:290-291)
        self.raw_luts = nn.Parameter(torch.randn(self.num_outputs, 2 ** self.num_inputs) * 0.1)
        self._apply_init_fn(self.raw_luts, name="raw_luts")
        addresses = torch.arange(2 ** self.num_inputs).unsqueeze(1)
        bits = (addresses >> torch.arange(self.num_inputs).unsqueeze(0)) & 1  # input 0 is the LSB
        self.register_buffer("binary_combinations", bits.to(torch.float32))

    def _get_luts(self):
        return ops.table_sigmoid(self.raw_luts)

    def forward_train(self, x):
        return hybrid_forward(x, self._get_luts(), self.binary_combinations)

    def forward_eval(self, x):
        plan = _identity_plan(x.shape[1], x.device)
        with torch.no_grad():
            return ops.dwn_layer_eval(x, self._get_luts().unsqueeze(0), plan)

    def _builtin_regularization(self):
        return torch.tensor(0.0, device=self.raw_luts.device, requires_grad=False)


__all__ = ["HybridNode"]
