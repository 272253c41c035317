"""Consecutive RandomLayer + DWN layers run as one chained operator.

The reference runs a stack layer by layer (`difflut/layers/random_layer.py:306-340`), each layer
writing its `[batch, nodes]` fp32 output for the next one to threshold.  The tables, mappings and
state-dict keys of the wrapped layers are untouched; only the execution of the training forward
and backward changes (bit-planes between layers, tile-major gradients between layers)."""
import torch
import torch.nn as nn

from .. import ops
from .random_layer import RandomLayer


class DWNStack(nn.Module):
    """`DWNStack([layer1, layer2, ...])(x)` equals `layerN(... layer2(layer1(x)))`.

    Training-mode calls take the chained kernels when every member is a RandomLayer of DWN nodes
    with at most 6 inputs and matching widths; so do eval-mode calls whose first input is known to
    be binary (a fused thermometer encoder, or `binary_input=True`).  Anything else runs the members
    one after the other."""

    def __init__(self, layers, encoder=None, head=None, binary_input=False):
        """`encoder`: a fitted, flattening ThermometerEncoder whose code feeds the first layer; the stack
        then takes the raw features and equals `layerN(... layer1(encoder.encode(x)))`.  On the chained
        path the code is never written as a [batch, features * bits] fp32 tensor.
        `head`: a GroupSum applied to the last layer's output (`head(layerN(...))`); on the chained path the
        last layer sums its columns per group itself and its [batch, nodes] output is never written."""
        super().__init__()
        self.layers = nn.ModuleList(layers)
        self.encoder = encoder
        self.head = head
        # the caller's promise that x holds exact 0/1 values (an encoder's code does anyway): eval mode can then
        # run chained as well, since the eval address floor(sum x_j 2^j) is the thresholded one
        self.binary_input = binary_input

    def _fusable_head(self):
        from ..utils.modules import GroupSum

        head = self.head
        if not isinstance(head, GroupSum) or head.use_randperm:
            return False
        last = self.layers[-1]
        features = last.output_size * last.output_dim_per_node
        # groups at least 64 columns wide and no zero-padding warning to reproduce
        return features % head.k == 0 and features // head.k >= 64

    def _chainable(self):
        width = None
        for layer in self.layers:
            if not isinstance(layer, RandomLayer) or layer._fused != "dwn" or layer.n > ops.FAST_K:
                return False
            if width is not None and layer.input_size != width:
                return False
            width = layer.output_size * layer.output_dim_per_node
        return len(self.layers) > 0

    def _fusable_encoder(self, x):
        from ..encoder.thermometer import ThermometerEncoder

        enc = self.encoder
        return (isinstance(enc, ThermometerEncoder) and enc.flatten and enc.thresholds is not None and x.dim() == 2
                and torch.is_tensor(x) and x.shape[1] * enc.num_bits == self.layers[0].input_size)

    def forward(self, x):
        if not self.training and self._chainable() and x.is_cuda and x.dim() == 2 and x.shape[0] > 0:
            fused_encoder = self.encoder is not None and self._fusable_encoder(x)
            if fused_encoder or (self.encoder is None and self.binary_input and x.shape[1] == self.layers[0].input_size):
                thresholds = self.encoder.thresholds.to(x.device) if fused_encoder else None
                plans = [layer.mapping_plan() for layer in self.layers]
                luts = [layer._banks["luts"].tensor().detach() for layer in self.layers]
                fused_head = self.head is not None and self._fusable_head()
                with torch.no_grad():
                    y = ops.dwn_stack_eval(x, thresholds, plans, luts, (self.head.k, self.head.tau) if fused_head else None)
                    return y if self.head is None or fused_head else self.head(y)
        if not (self.training and self._chainable() and torch.is_tensor(x) and x.is_cuda):
            if self.encoder is not None:
                x = self.encoder.encode(x)
            for layer in self.layers:
                x = layer(x)
            return x if self.head is None else self.head(x)
        thresholds = None
        if self.encoder is not None:
            if self._fusable_encoder(x):
                thresholds = self.encoder.thresholds.to(x.device)
                if x.shape[0] == 0:
                    raise ValueError(f"BaseLUTLayer requires non-empty batch, got batch_size={x.shape[0]}")
            else:
                x = self.encoder.encode(x)
        if thresholds is None:
            self.layers[0]._validate_input_dims(x)
        plans = [layer.mapping_plan() for layer in self.layers]
        scalars = [layer.efd_scalars() for layer in self.layers]  # every node's own alpha and beta
        luts = [layer._banks["luts"].tensor() for layer in self.layers]
        if self.head is not None and self._fusable_head():
            return ops.DWNStackFunction.apply(x, thresholds, plans, scalars, (self.head.k, self.head.tau), *luts)
        y = ops.DWNStackFunction.apply(x, thresholds, plans, scalars, None, *luts)
        return y if self.head is None else self.head(y)
