"""Base class of the LUT layers.

Public surface of difflut/layers/base_layer.py:35-576: constructor arguments and validation,
`nodes` (an nn.ModuleList of output_size node modules), `n`, `output_dim_per_node`,
`get_mapping`, `regularization`, the bit-flip augmentation and the gradient-stabilisation hook.

What is different underneath: when every node is of a type the device library covers
(DWNNode, DWNStableNode, HybridNode, ProbabilisticNode) the layer runs all nodes in ONE call on one contiguous
[N, ...] parameter tensor instead of looping over N modules.  The per-node Parameters that
users, optimisers and state_dict see (`nodes.{i}.luts`, ...) are views into that tensor:
  * `ParameterBank.flat` is the [N, ...] leaf the fused autograd Function differentiates;
  * each node's Parameter is a `BankedParameter` whose storage is row i of `flat` and whose
    `.grad` reads row i of `flat.grad`, so optimisers update the shared storage in place
    and no per-node gradient copies are made;
  * `Module._apply` (.to/.cuda/.float) re-allocates parameters one by one, so the layer
    re-ties them after every `_apply`; `copy.deepcopy` and unpickling re-tie in `__setstate__`, so the
    objects `parameters()` yields are final before the first forward (an optimizer built right after
    a copy or a load keeps working).
The per-node scalar buffers the fused kernels need (`alpha`, `beta`, `temperature`) are banked the same way
(`ScalarBank`: one [N] tensor, each node's 0-dim buffer a view of it), so a state dict or an in-place edit that
gives nodes different values lands in the array the kernels are handed on every call: every fused path (single
layers, chained stacks, convolutional levels) uses each node's own values, as the reference's node loop does.
"""
import warnings
from abc import ABC, abstractmethod

import torch
import torch.nn as nn

from ..nodes.node_config import NodeConfig
from ..utils.warnings import warn_default_value
from .layer_config import LayerConfig, validate_layer_options

DEFAULT_LAYER_FLIP_PROBABILITY = 0.0
DEFAULT_LAYER_GRAD_STABILIZATION = "none"
DEFAULT_LAYER_GRAD_TARGET_STD = 1.0
DEFAULT_LAYER_GRAD_SUBTRACT_MEAN = False
DEFAULT_LAYER_GRAD_EPSILON = 1e-8
LAYER_REUSE_WARNING_THRESHOLD = 10
LAYER_UNDERUSE_WARNING_DIVISOR = 10
LAYER_MAX_NODE_INPUT_DIM = 15


class BankedParameter(nn.Parameter):
    """Row `row` of a ParameterBank, presented as an ordinary per-node Parameter."""

    def __new__(cls, data, bank=None, row=0):
        p = torch.Tensor._make_subclass(cls, data, True)
        p._bank, p._row = bank, row
        return p

    @property
    def grad(self):
        g = self._bank.flat.grad
        return None if g is None else g[self._row]

    @grad.setter
    def grad(self, value):
        flat = self._bank.flat
        if value is None:
            flat.grad = None  # gradients live in one tensor: clearing one row clears the bank
        else:
            if flat.grad is None:
                flat.grad = torch.zeros_like(flat)
            flat.grad[self._row].copy_(value)

    def __deepcopy__(self, memo):
        return nn.Parameter(self.data.clone(memory_format=torch.preserve_format), self.requires_grad)

    def __reduce_ex__(self, proto):
        return (nn.Parameter, (self.data.clone(), self.requires_grad))


class ParameterBank:
    """The parameter `name` of N nodes as one leaf tensor [N, *shape]."""

    def __init__(self, nodes, name):
        self.nodes, self.name = nodes, name
        self.flat = None
        self._stale = False  # set when another bank takes over one of my nodes, or a node's parameter is reassigned
        self.tie()

    def tie(self, keep_grad=None):
        params = [node._parameters[self.name] for node in self.nodes]
        for p in params:  # a bank that held one of these nodes (a sub-layer's own, a level's) no longer does
            other = getattr(p, "_bank", None)
            if other is not None and other is not self:
                other._stale = True
        flat = torch.stack([p.data for p in params]).contiguous()
        flat.requires_grad_(True)
        if keep_grad is not None:
            flat.grad = keep_grad.to(flat.device)
        self.flat = flat
        view = flat.detach()
        for row, node in enumerate(self.nodes):
            node._parameters[self.name] = BankedParameter(view[row], self, row)
        self._stale = False

    def tied(self):
        if self._stale:
            return False
        first = self.nodes[0]._parameters[self.name]
        last = self.nodes[-1]._parameters[self.name]
        step = self.flat[0].numel() * self.flat.element_size()
        base = self.flat.data_ptr()
        return (isinstance(first, BankedParameter) and first._bank is self and first.device == self.flat.device
                and first.data_ptr() == base and last.data_ptr() == base + step * (len(self.nodes) - 1))

    def tensor(self):
        if not self.tied():
            self.tie()
        return self.flat


class ScalarBank:
    """The 0-dim buffer `name` of N nodes as one tensor [N]; each node's buffer is a view of its entry, so
    `load_state_dict` and in-place edits land in the bank and the kernels, which are handed the whole array on
    every call, always see every node's current value.  The views keep the buffers' own dtype (`layer.double()`
    leaves double buffers); `tensor()` is the float32 array the kernels read.  The only host-side knowledge is
    `abs_max()` (the largest magnitude, which selects the form of the EFD coefficient table): read back when the
    bank's version counter changes or after `invalidate()`."""

    _PROBES = 16  # nodes checked per call beyond the first and the last when the layer is large

    def __init__(self, nodes, name):
        self.nodes, self.name = nodes, name
        self.flat, self._stale, self._key, self._abs_max, self._views, self._probe = None, False, None, None, [], 0
        self.tie()

    def tie(self):
        bufs = [node._buffers[self.name] for node in self.nodes]
        for b in bufs:
            other = getattr(b, "_scalar_bank", None)
            if other is not None and other is not self:
                other._stale = True
        self.flat = torch.stack([b.detach().reshape(()) for b in bufs]).contiguous()
        self._views = []
        for row, node in enumerate(self.nodes):
            view = self.flat[row]
            view._scalar_bank = self
            node._buffers[self.name] = view
            self._views.append(view)
        self._stale, self._key = False, None

    def _is_view(self, row):
        return self.nodes[row]._buffers[self.name] is self._views[row]

    def tied(self):
        """Every node's buffer is still the view handed out by tie().  All nodes are checked on small layers; on large
        ones the first, the last and a window of nodes that moves on with every call (assignments through
        `node.<name> = ...` set the stale flag themselves)."""
        if self._stale or not self._views or self._views[0].device != self.flat.device:
            return False
        n = len(self.nodes)
        if n <= 4 * self._PROBES:
            return all(self._is_view(row) for row in range(n))
        rows = [0, n - 1] + [(self._probe + i) % n for i in range(self._PROBES)]
        self._probe = (self._probe + self._PROBES) % n
        return all(self._is_view(row) for row in rows)

    def tensor(self):
        """The float32 device array [N] for the kernels (the bank itself when it is float32)."""
        if not self.tied():
            self.tie()
        return self.flat if self.flat.dtype == torch.float32 else self.flat.float()

    def invalidate(self):
        """Forget the host-side summary: needed after a write that bypasses the version counter (`buffer.data.fill_`,
        an external kernel)."""
        self._key = None

    def abs_max(self):
        flat = self.tensor()
        key = (self.flat._version, self.flat.data_ptr())
        if key != self._key:
            self._abs_max = float(flat.detach().abs().max())
            self._key = key
        return self._abs_max


class LUTLayerMixin(nn.Module):
    """Bit-flip augmentation and gradient rescaling shared by the layers (base_layer.py:35-339)."""

    def _init_lut_layer_mixin(self, layer_config=None, flip_probability=None, grad_stabilization=None,
                              grad_target_std=None, grad_subtract_mean=None, grad_epsilon=None):
        if layer_config is not None:
            if not isinstance(layer_config, LayerConfig):
                raise TypeError(f"layer_config must be a LayerConfig instance, got {type(layer_config)}.")
            values = (layer_config.flip_probability, layer_config.grad_stabilization, layer_config.grad_target_std,
                      layer_config.grad_subtract_mean, layer_config.grad_epsilon)
        else:
            given = (flip_probability, grad_stabilization, grad_target_std, grad_subtract_mean, grad_epsilon)
            defaults = (DEFAULT_LAYER_FLIP_PROBABILITY, DEFAULT_LAYER_GRAD_STABILIZATION,
                        DEFAULT_LAYER_GRAD_TARGET_STD, DEFAULT_LAYER_GRAD_SUBTRACT_MEAN, DEFAULT_LAYER_GRAD_EPSILON)
            names = ("flip_probability", "grad_stabilization", "grad_target_std", "grad_subtract_mean",
                     "grad_epsilon")
            values = []
            for name, value, default in zip(names, given, defaults):
                if value is None:
                    value = default
                    warn_default_value(name, value, stacklevel=3)
                values.append(value)
            validate_layer_options(values[0], values[1], values[2], values[4])
        (self.flip_probability, self.grad_stabilization, self.grad_target_std, self.grad_subtract_mean,
         self.grad_epsilon) = values
        self._flip_mask_buffer = None

    def _flip_mask(self, shape, device):
        """The positions the bit-flip augmentation inverts this call (training only; None = none): below 5 % an exact
        count of positions drawn without replacement, otherwise one Bernoulli draw per entry - the two branches and
        their generator calls of base_layer.py:149-264."""
        if self.flip_probability <= 0.0 or not self.training:
            return None
        numel = 1
        for d in shape:
            numel *= d
        if self.flip_probability < 0.05:
            count = int(numel * self.flip_probability)
            if count == 0:
                return None
            mask = torch.zeros(numel, dtype=torch.bool, device=device)
            mask[torch.randperm(numel, device=device)[:count]] = True
            return mask.view(shape)
        return torch.bernoulli(torch.full(tuple(shape), self.flip_probability, device=device, dtype=torch.float32)).bool()

    def _apply_bit_flip(self, x):
        """Training only: x -> 1 - x on a random subset; the flip is detached so gradients flow as if
        no bit had been flipped."""
        mask = self._flip_mask(x.shape, x.device)
        if mask is None:
            return x
        delta = torch.where(mask, 1.0 - 2.0 * x.detach(), torch.zeros_like(x))
        return x + delta

    def _apply_gradient_stabilization(self, grad):
        """grad <- (grad - mean) * sqrt(target / (mean(grad^2) + eps)), over the whole layer or per sample."""
        if self.grad_stabilization == "none" or not self.training or grad is None:
            return grad
        dims = None if self.grad_stabilization == "layerwise" else 1
        if grad.is_cuda and grad.dim() == 2 and grad.dtype == torch.float32:
            from .. import ops  # one or two library launches instead of seven torch kernels

            return ops.grad_stabilize(grad, dims == 1, self.grad_target_std, self.grad_subtract_mean, self.grad_epsilon)
        g = grad.clone()
        if self.grad_subtract_mean:
            g -= g.mean() if dims is None else g.mean(dim=1, keepdim=True)
        var = g.pow(2).mean() if dims is None else g.pow(2).mean(dim=1, keepdim=True)
        return g * torch.sqrt(self.grad_target_std / (var + self.grad_epsilon))


class BaseLUTLayer(ABC, LUTLayerMixin, nn.Module):
    """input (batch, input_size) -> output (batch, output_size * output_dim_per_node)."""

    def __init__(self, input_size, output_size, node_type, node_kwargs, layer_config=None, flip_probability=None,
                 grad_stabilization=None, grad_target_std=None, grad_subtract_mean=None, grad_epsilon=None):
        super().__init__()
        if not isinstance(input_size, int) or input_size <= 0:
            raise ValueError(f"input_size must be a positive integer, got {input_size}.")
        if not isinstance(output_size, int) or output_size <= 0:
            raise ValueError(f"output_size must be a positive integer, got {output_size}.")
        self._init_lut_layer_mixin(layer_config, flip_probability, grad_stabilization, grad_target_std,
                                   grad_subtract_mean, grad_epsilon)
        self.input_size, self.output_size = input_size, output_size
        kwargs = node_kwargs.to_dict() if isinstance(node_kwargs, NodeConfig) else dict(node_kwargs or {})
        # node by node, so the global generator is consumed in node order like the reference's list
        # comprehension (base_layer.py:397)
        self.nodes = nn.ModuleList([node_type(**kwargs) for _ in range(output_size)])
        self.n = self.nodes[0].num_inputs
        self.output_dim_per_node = self.nodes[0].num_outputs
        self._banks, self._scalars = {}, {}
        self._fused = self._detect_fused_kind()
        if self._fused == "dwn":
            self._banks["luts"] = ParameterBank(self.nodes, "luts")
            self._scalars["alpha"] = ScalarBank(self.nodes, "alpha")
            self._scalars["beta"] = ScalarBank(self.nodes, "beta")
        elif self._fused == "probabilistic":
            self._banks["raw_weights"] = ParameterBank(self.nodes, "raw_weights")
            self._scalars["temperature"] = ScalarBank(self.nodes, "temperature")
        elif self._fused == "dwn_stable":
            self._banks["raw_luts"] = ParameterBank(self.nodes, "raw_luts")
            self._banks["gradient_scale"] = ParameterBank(self.nodes, "gradient_scale")
        elif self._fused == "hybrid":
            self._banks["raw_luts"] = ParameterBank(self.nodes, "raw_luts")
        self._validate_layer_config()

    # ------------------------------------------------------------------ fused execution
    def _detect_fused_kind(self):
        from ..nodes.dwn_node import DWNNode
        from ..nodes.dwn_stable_node import DWNStableNode
        from ..nodes.hybrid_node import HybridNode
        from ..nodes.probabilistic_node import ProbabilisticNode

        kinds = {type(node) for node in self.nodes}
        for cls in (DWNNode, ProbabilisticNode, DWNStableNode, HybridNode):
            if kinds == {cls}:
                return cls.fused_kind
        return None  # other node types: per-node loop over the gathered inputs

    def _apply(self, fn, *args, **kwargs):
        grads = {name: bank.flat.grad for name, bank in self._banks.items()}
        for bank in self._banks.values():
            bank.flat.grad = None
        super()._apply(fn, *args, **kwargs)
        for name, bank in self._banks.items():
            bank.tie(keep_grad=None if grads[name] is None else fn(grads[name]))
        for bank in self._scalars.values():
            bank.tie()
        return self

    def __setstate__(self, state):
        # copy.deepcopy and unpickling hand back plain per-node Parameters: tie them to their banks now, so that
        # what parameters() yields is not replaced by the first forward
        super().__setstate__(state)
        self.__dict__.setdefault("_scalars", {})
        for bank in self._banks.values():
            bank.nodes = self.nodes
            bank.tie()
        for bank in self._scalars.values():
            bank.nodes = self.nodes
            bank.tie()

    def efd_scalars(self):
        """(alpha [N], beta [N], max |beta|) of a DWN layer for the kernels: the nodes' own values as float32 device
        arrays (every call reads the nodes' current values, dwn_node.py:450) and the host value that selects the form
        of the coefficient table."""
        return self._scalars["alpha"].tensor(), self._scalars["beta"].tensor(), self._scalars["beta"].abs_max()

    def temperatures(self):
        """The nodes' temperatures [N] as a float32 device array (probabilistic_node.py:277-282 reads each node's)."""
        return self._scalars["temperature"].tensor()

    def invalidate_scalars(self):
        """Call after writing a node's `alpha` / `beta` / `temperature` in a way autograd's version counter does not
        see (`node.beta.data.fill_(...)`, an external kernel).  The kernels read the values themselves on every call;
        what this refreshes is the host's max |beta|, which decides between the two forms of the EFD coefficient
        table (the compact one divides by 1 - beta and is only used while every |beta| <= 1/2)."""
        for bank in self._scalars.values():
            bank.invalidate()

    def bank_parameters(self):
        """The layer's trainable tensors with every node parameter as ONE leaf [N, ...] (the storage the
        per-node parameters are views of) followed by the layer's own parameters.  Handing these to an
        optimizer instead of `parameters()` (N small tensors) makes its step one kernel per tensor;
        both see the same memory.  Call after the layer is on its device: `.to()` re-creates the leaves."""
        banks = [bank.tensor() for bank in self._banks.values()]
        # the layer's own parameters: everything outside `nodes` (not a walk over the N node modules)
        own = [p for p in self._parameters.values() if p is not None]
        for name, child in self.named_children():
            if name != "nodes":
                own.extend(child.parameters())
        return banks + own

    def _run_nodes(self, x, plan):
        """All nodes on x [batch, width] through `plan` (index table over width) -> [batch, N*O]."""
        if self._fused == "dwn":
            from .. import ops

            luts = self._banks["luts"].tensor()
            if self.training:
                return ops.dwn_layer(x, luts, plan, *self.efd_scalars())
            return ops.dwn_layer_eval(x, luts.detach(), plan)
        if self._fused == "probabilistic":
            from .. import ops

            raw = self._banks["raw_weights"].tensor()
            if self.training:
                return ops.prob_layer(x, raw, plan, self.temperatures())
            return ops.prob_layer_eval(x, raw.detach(), plan, self.temperatures())
        if self._fused in ("dwn_stable", "hybrid"):
            from .. import ops

            raw = self._banks["raw_luts"].tensor()
            if not self.training:
                with torch.no_grad():
                    return ops.dwn_layer_eval(x, ops.table_sigmoid(raw), plan)
            luts = ops.table_sigmoid(raw)
            if self._fused == "hybrid":
                return ops.hybrid_layer(x, luts, plan)
            return ops.dwn_stable_layer(x, luts, self._banks["gradient_scale"].tensor().detach(), plan)
        return None

    def _loop_nodes(self, mapped):
        """Fallback for node types without a fused kernel: mapped [batch, N, n] -> [batch, N*O]."""
        outs = [node(mapped[:, i, :]) for i, node in enumerate(self.nodes)]
        return torch.stack(outs, dim=1).reshape(mapped.shape[0], -1)

    # ------------------------------------------------------------------ validation
    def _validate_layer_config(self):
        total = self.output_size * self.n
        if total > self.input_size * LAYER_REUSE_WARNING_THRESHOLD:
            warnings.warn(f"BaseLUTLayer: Creating {total} node input connections from only {self.input_size} input "
                          f"features (about {total // self.input_size}x reuse).", UserWarning, stacklevel=2)
        if total < self.input_size // LAYER_UNDERUSE_WARNING_DIVISOR:
            warnings.warn(f"BaseLUTLayer: Creating only {total} node inputs from {self.input_size} input features. "
                          "Most input features will be unused.", UserWarning, stacklevel=2)
        if self.n > LAYER_MAX_NODE_INPUT_DIM:
            warnings.warn(f"BaseLUTLayer: Node input dimension (n={self.n}) is quite large (2^{self.n} entries).",
                          UserWarning, stacklevel=2)

    def _validate_input_dims(self, x):
        if x.dim() != 2:
            raise ValueError(f"BaseLUTLayer expects 2D input (batch_size, input_size), but got shape {x.shape} "
                             f"with {x.dim()} dimensions.")
        if x.shape[1] != self.input_size:
            raise ValueError(f"BaseLUTLayer expected input with {self.input_size} features, but got {x.shape[1]} "
                             f"features. Shape: {x.shape}.")
        if x.shape[0] == 0:
            raise ValueError(f"BaseLUTLayer requires non-empty batch, got batch_size={x.shape[0]}")

    # ------------------------------------------------------------------ interface
    @abstractmethod
    def get_mapping(self, x):
        """Mapped inputs (batch, output_size, n)."""

    def get_mapping_indices(self):
        return None

    def forward(self, x):
        self._validate_input_dims(x)
        if self.training and self.flip_probability > 0.0:
            x = self._apply_bit_flip(x)
        out = self._loop_nodes(self.get_mapping(x))
        if self.grad_stabilization != "none" and self.training and out.requires_grad:
            out.register_hook(self._apply_gradient_stabilization)
        return out

    def regularization(self):
        params = list(self.parameters())
        total = torch.tensor(0.0, device=params[0].device if params else "cpu")
        for node in self.nodes:
            if callable(getattr(node, "regularization", None)):
                total = total + node.regularization()
        return total
