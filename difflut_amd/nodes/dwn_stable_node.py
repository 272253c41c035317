"""Gradient-stabilised DWN node: thresholded lookup in a sigmoid table, EFD-style backward with the
weight 1/(h+1) and a gradient scale.

API of difflut/nodes/dwn_stable_node.py:232-371 (constructor, `raw_luts` parameter [output_dim, 2^k],
`gradient_scale` parameter, `_get_luts`, train/eval forwards).  The arithmetic runs in
libdifflut_hip.so; a node called on its own goes through the whole-layer kernels with N = 1 and the
identity mapping.  The scale is handed to the kernels as a device value, never read back by the host.
"""
import torch
import torch.nn as nn

from .. import _native, ops
from ..registry import register_node
from .base_node import BaseNode
from .cuda import is_cuda_available
from .dwn_node import _identity_plan

DEFAULT_DWN_STABLE_GRADIENT_SCALE = 1.0
DEFAULT_DWN_STABLE_USE_CUDA = True

_CUDA_EXT_AVAILABLE = _native.is_built()


def dwn_stable_forward(input, luts, gradient_scale):
    """(batch, k) inputs, (output_dim, 2^k) table already in [0, 1], scalar scale (number or tensor)
    -> (batch, output_dim); autograd-aware (dwn_stable_node.py:212-229)."""
    if not torch.is_tensor(gradient_scale):
        gradient_scale = torch.full((1,), float(gradient_scale), device=input.device)
    plan = _identity_plan(input.shape[1], input.device)
    return ops.dwn_stable_layer(input, luts.unsqueeze(0), gradient_scale.reshape(1), plan)


@register_node("dwn_stable")
class DWNStableNode(BaseNode):
    fused_kind = "dwn_stable"

    def __init__(self, input_dim=None, output_dim=None, use_cuda=DEFAULT_DWN_STABLE_USE_CUDA, regularizers=None,
                 gradient_scale=1.25, init_fn=None, init_kwargs=None):
        super().__init__(input_dim=input_dim, output_dim=output_dim, regularizers=regularizers, init_fn=init_fn,
                         init_kwargs=init_kwargs)
        self.use_cuda = use_cuda and is_cuda_available()
        self.gradient_scale = nn.Parameter(torch.tensor(float(gradient_scale)))
        # one normal draw per node, then the initialiser (dwn_stable_node.py:284-287)
        self.raw_luts = nn.Parameter(torch.randn(self.num_outputs, 2 ** self.num_inputs) * 0.1)
        self._apply_init_fn(self.raw_luts, name="raw_luts")

    def _get_luts(self):
        return ops.table_sigmoid(self.raw_luts)

    def forward_train(self, x):
        return dwn_stable_forward(x, self._get_luts(), self.gradient_scale.detach())

    def forward_eval(self, x):
        plan = _identity_plan(x.shape[1], x.device)
        with torch.no_grad():
            return ops.dwn_layer_eval(x, self._get_luts().unsqueeze(0), plan)

    def _builtin_regularization(self):
        return torch.tensor(0.0, device=self.raw_luts.device, requires_grad=False)
