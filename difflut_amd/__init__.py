"""difflut_amd: the DiffLUT LUT-node / mapping-layer hot path on AMD MI355X (gfx950).

Same registry names, constructors and autograd behaviour as the `difflut` package for
RandomLayer, LearnableLayer, DWNNode, ProbabilisticNode, ThermometerEncoder and GroupSum;
the arithmetic runs in hand-written HIP kernels (difflut_amd/lib/libdifflut_hip.so, C ABI
in include/difflut_hip.h) for tensors on a ROCm device.  Tensors on the CPU take plain-torch
operators of the same arithmetic (difflut_amd/cpu_ops.py), as the reference's operators do
when `x.is_cuda` is false.
"""
from .encoder.base_encoder import BaseEncoder
from .layers.base_layer import BaseLUTLayer
from .nodes.base_node import BaseNode
from .registry import (REGISTRY, register_convolutional_layer, register_encoder, register_initializer, register_layer,
                       register_node, register_regularizer)
from . import encoder, layers, nodes, utils  # noqa: E402,F401  (imports register the components)

__version__ = "0.1.0"

__all__ = ["REGISTRY", "register_node", "register_layer", "register_convolutional_layer", "register_encoder",
           "register_initializer", "register_regularizer", "BaseNode", "BaseLUTLayer", "BaseEncoder"]
