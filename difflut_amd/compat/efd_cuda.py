"""efd_cuda.forward/backward (difflut/nodes/cuda/efd_cuda.cpp:22-45): one node, input [B,k],
luts [O,L].  A node is a layer of one node with the identity mapping."""
import efd_fused_cuda
from _common import torch

_identity = {}


def _ident(k, device):
    key = (k, str(device))
    if key not in _identity:
        _identity[key] = torch.arange(k, dtype=torch.int64, device=device).view(1, k)
    return _identity[key]


def forward(input, luts):
    return efd_fused_cuda.forward(input, _ident(input.shape[1], input.device), luts.unsqueeze(0).contiguous())[:, 0, :]


def backward(input, luts, grad_output, alpha, beta):
    gx, gl = efd_fused_cuda.backward(input, _ident(input.shape[1], input.device), luts.unsqueeze(0).contiguous(),
                                     grad_output.unsqueeze(1).contiguous(), alpha, beta)
    return [gx, gl[0]]
