"""DWN node: k-input lookup table with the extended-finite-difference (EFD) backward.

API of difflut/nodes/dwn_node.py:341-544 (constructor, `luts` parameter [output_dim, 2^k],
`alpha`/`beta` buffers, train/eval forwards).  The arithmetic runs in libdifflut_hip.so:
a node called on its own goes through the same whole-layer kernels as a RandomLayer of
N = 1 with the identity mapping; inside a layer the layer issues one fused call for all
nodes and this module only holds the parameters.
"""
import torch
import torch.nn as nn

from .. import _native, ops
from ..registry import register_node
from ..utils.warnings import warn_default_value
from .base_node import BaseNode
from .cuda import is_cuda_available

DWN_ALPHA_BASE = 0.5
DWN_ALPHA_DECAY = 0.75
DWN_BETA_NUMERATOR = 0.25
DWN_BETA_DENOMINATOR = 0.75
DWN_BINARY_THRESHOLD = 0.5
DEFAULT_DWN_USE_CUDA = True
DEFAULT_DWN_CLAMP_LUTS = True

# the reference's flags for its two extensions; here one library serves both roles
_CUDA_EXT_AVAILABLE = _native.is_built()
_FUSED_CUDA_EXT_AVAILABLE = _native.is_built()

_identity_plans = {}


def _identity_plan(k, device):
    key = (k, str(device))
    if key not in _identity_plans:
        _identity_plans[key] = ops.MappingPlan.identity(k, device)
    return _identity_plans[key]


def efd_forward(input, luts, alpha, beta):
    """(batch, k) inputs and (output_dim, 2^k) table -> (batch, output_dim); autograd-aware
    (dwn_node.py:319-338)."""
    plan = _identity_plan(input.shape[1], input.device)
    return ops.dwn_layer(input, luts.unsqueeze(0), plan, alpha, beta)


@register_node("dwn")
class DWNNode(BaseNode):
    fused_kind = "dwn"

    def __init__(self, input_dim=None, output_dim=None, use_cuda=DEFAULT_DWN_USE_CUDA, regularizers=None, alpha=None,
                 beta=None, clamp_luts=DEFAULT_DWN_CLAMP_LUTS, init_fn=None, init_kwargs=None):
        init_kwargs = dict(init_kwargs) if init_kwargs else {}
        if "input_dim" not in init_kwargs and input_dim is not None:
            init_kwargs["input_dim"] = input_dim  # residual_init needs the table width
        super().__init__(input_dim=input_dim, output_dim=output_dim, regularizers=regularizers, init_fn=init_fn,
                         init_kwargs=init_kwargs)
        self.use_cuda = use_cuda and is_cuda_available()
        self.clamp_luts = clamp_luts
        if alpha is None:
            alpha = DWN_ALPHA_BASE * DWN_ALPHA_DECAY ** (self.num_inputs - 1)
            warn_default_value("alpha", alpha, stacklevel=2)
        if beta is None:
            beta = DWN_BETA_NUMERATOR / DWN_BETA_DENOMINATOR
            warn_default_value("beta", beta, stacklevel=2)
        self.register_buffer("alpha", torch.tensor(alpha, dtype=torch.float32))
        self.register_buffer("beta", torch.tensor(beta, dtype=torch.float32))
        # one draw from the global generator per node, then the initialiser (dwn_node.py:423-424)
        self.luts = nn.Parameter(torch.rand(self.num_outputs, 2 ** self.num_inputs))
        self._apply_init_fn(self.luts, name="luts")

    def efd_scalars(self):
        """(alpha, beta) as Python floats; the buffers are fp32, read back once and cached."""
        key = (self.alpha._version, self.beta._version, self.alpha.data_ptr(), self.beta.data_ptr())
        if getattr(self, "_ab_key", None) != key:
            self._ab = (float(self.alpha), float(self.beta))
            self._ab_key = key
        return self._ab

    def forward_train(self, x):
        alpha, beta = self.efd_scalars()
        return efd_forward(x, self.luts, alpha, beta)

    def forward_eval(self, x):
        plan = _identity_plan(x.shape[1], x.device)
        return ops.dwn_layer_eval(x, self.luts.detach().unsqueeze(0), plan)

    def forward_with_mapping(self, x, mapping_indices):
        """Fused mapping + lookup with this node's table shared by every mapped position
        (dwn_node.py:485-540): returns (batch, layer_size, output_dim)."""
        layer_size, k = mapping_indices.shape
        if k != self.num_inputs:
            raise ValueError(f"Mapping indices input_dim ({k}) doesn't match node's input_dim ({self.num_inputs})")
        plan = ops.MappingPlan(mapping_indices, x.shape[1])
        luts = self.luts.unsqueeze(0).expand(layer_size, -1, -1)
        if self.training:
            alpha, beta = self.efd_scalars()
            out = ops.dwn_layer(x, luts, plan, alpha, beta)
        else:
            out = ops.dwn_layer_eval(x, luts.detach(), plan)
        return out.view(x.shape[0], layer_size, self.num_outputs)

    def _builtin_regularization(self):
        return torch.tensor(0.0, device=self.luts.device, requires_grad=False)
