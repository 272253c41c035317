"""Consecutive RandomLayer + DWN layers run as one chained operator.

The reference runs a stack layer by layer (`difflut/layers/random_layer.py:306-340`), each layer
writing its `[batch, nodes]` fp32 output for the next one to threshold.  The tables, mappings and
state-dict keys of the wrapped layers are untouched; only the execution of the training forward
and backward changes (bit-planes between layers, tile-major gradients between layers)."""
import torch.nn as nn

from .. import ops
from .random_layer import RandomLayer


class DWNStack(nn.Module):
    """`DWNStack([layer1, layer2, ...])(x)` equals `layerN(... layer2(layer1(x)))`.

    Training-mode calls take the chained kernels when every member is a RandomLayer of DWN nodes
    with at most 6 inputs and matching widths; anything else (and eval mode) runs the members
    one after the other."""

    def __init__(self, layers):
        super().__init__()
        self.layers = nn.ModuleList(layers)

    def _chainable(self):
        width = None
        for layer in self.layers:
            if not isinstance(layer, RandomLayer) or layer._fused != "dwn" or layer.n > ops.FAST_K:
                return False
            if width is not None and layer.input_size != width:
                return False
            width = layer.output_size * layer.output_dim_per_node
        return len(self.layers) > 0

    def forward(self, x):
        if not (self.training and self._chainable()):
            for layer in self.layers:
                x = layer(x)
            return x
        self.layers[0]._validate_input_dims(x)
        plans = [layer.mapping_plan() for layer in self.layers]
        scalars = [layer.nodes[0].efd_scalars() for layer in self.layers]
        luts = [layer._banks["luts"].tensor() for layer in self.layers]
        return ops.DWNStackFunction.apply(x, plans, scalars, *luts)
