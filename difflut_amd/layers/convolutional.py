"""Convolutional LUT layer: every output channel is a small tree of LUT layers applied to each patch.

Constructor, configuration object, sub-module layout (`first_layer_chunks`, `trees`, hence the
state-dict keys) and forward semantics follow difflut/layers/convolutional.py:13-267.  What differs
is the execution.  The reference loops over chunks of first layers and then over every tree and
every tree layer, out_channels * tree_depth tiny layer calls per forward.  Here all trees' layers of
one depth level run as ONE block-diagonal layer call: level l has out_channels * n^(depth-l) nodes,
tree t's nodes read the columns of tree t only (its index table shifted by t times the level's
width), and for DWN nodes the levels are chained (bit-planes between levels, tile-major gradients
back) and the patch matrix is only ever written as bit-planes.  Patch extraction and its adjoint are
the library's own kernels instead of `nn.Unfold` (kept as the `unfold` attribute for inspection).  The node parameters of a level live in one [nodes, ...] tensor; the per-node Parameters of
the sub-layers are views of it.
"""
import torch
import torch.nn as nn

from .. import _native, ops
from ..nodes.node_config import NodeConfig
from ..registry import register_convolutional_layer
from .base_layer import LUTLayerMixin, ParameterBank, ScalarBank
from .layer_config import GroupedInputConfig
from .random_layer import RandomLayer

_BANKED = {"dwn": ("luts",), "probabilistic": ("raw_weights",), "dwn_stable": ("raw_luts", "gradient_scale"),
           "hybrid": ("raw_luts",)}
# the per-node scalar buffers the kernels read, banked per depth level like the parameters
_BANKED_SCALARS = {"dwn": ("alpha", "beta"), "probabilistic": ("temperature",), "dwn_stable": (), "hybrid": ()}


class ConvolutionConfig:
    def __init__(self, tree_depth=2, in_channels=None, out_channels=None, receptive_field=5, stride=1, padding=0,
                 chunk_size=32, seed=42):
        assert in_channels is not None, "in_channels must be specified"
        assert out_channels is not None, "out_channels must be specified"
        self.tree_depth = tree_depth
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.receptive_field = receptive_field
        self.stride = stride
        self.padding = padding
        self.chunk_size = chunk_size
        self.seed = seed


def _pair(v):
    return (v, v) if isinstance(v, int) else v


@register_convolutional_layer("convolutional")
class ConvolutionalLayer(LUTLayerMixin, nn.Module):
    def __init__(self, convolution_config, node_type, node_kwargs, layer_type, n_inputs_per_node=6, layer_config=None,
                 flip_probability=None, grad_stabilization=None, grad_target_std=None, grad_subtract_mean=None,
                 grad_epsilon=None, grouped_connections=False, ensure_full_coverage=False):
        super().__init__()
        self._init_lut_layer_mixin(layer_config, flip_probability, grad_stabilization, grad_target_std,
                                   grad_subtract_mean, grad_epsilon)
        cfg = convolution_config
        self.tree_depth = cfg.tree_depth
        self.in_channels, self.out_channels = cfg.in_channels, cfg.out_channels
        self.receptive_field = _pair(cfg.receptive_field)
        self.input_size = self.in_channels * self.receptive_field[0] * self.receptive_field[1]
        self.stride, self.padding = _pair(cfg.stride), _pair(cfg.padding)
        self.node_type, self.layer_type = node_type, layer_type
        self.n_inputs_per_node = n_inputs_per_node
        self.seed = cfg.seed
        self.chunk_size = min(cfg.chunk_size, self.out_channels)
        # nodes per tree at each level: n^depth, ..., n, 1
        self.hidden_layers = [n_inputs_per_node ** (self.tree_depth - i) for i in range(self.tree_depth + 1)]
        grouped = None
        if grouped_connections:
            assert self.input_size % self.in_channels == 0, "Input size must be divisible by number of groups."
            grouped = GroupedInputConfig(n_groups=self.in_channels, input_size=self.input_size,
                                         output_trees=self.out_channels, luts_per_tree=self.hidden_layers[0],
                                         bits_per_node=n_inputs_per_node, seed=self.seed,
                                         ensure_full_coverage=ensure_full_coverage)
        # sub-modules in the reference's construction order (node parameters draw from the global generator)
        self.first_layer_chunks = nn.ModuleList()
        for start in range(0, self.out_channels, self.chunk_size):
            end = min(start + self.chunk_size, self.out_channels)
            self.first_layer_chunks.append(layer_type(
                input_size=self.input_size, output_size=self.hidden_layers[0] * (end - start), node_type=node_type,
                node_kwargs=node_kwargs, mapping_indices=grouped.get_mapping_indices(start, end) if grouped else None))
        self.trees = nn.ModuleList()
        for _ in range(self.out_channels):
            tree, width = nn.ModuleList(), self.hidden_layers[0]
            for size in self.hidden_layers[1:]:
                tree.append(layer_type(input_size=width, output_size=size, node_type=node_type, node_kwargs=node_kwargs))
                width = size
            self.trees.append(tree)
        self.unfold = nn.Unfold(kernel_size=self.receptive_field, padding=self.padding, stride=self.stride)
        self._kind = self._detect_kind()
        self._level_banks, self._level_scalar_banks, self._plans, self._plan_key = [], [], None, None
        if self._kind is not None:
            self._tie_levels()

    # ------------------------------------------------------------------ block-diagonal levels
    def _sublayers(self):
        yield from self.first_layer_chunks
        for tree in self.trees:
            yield from tree

    def _detect_kind(self):
        """The fused kind shared by every sub-layer, or None (then the reference's loop runs)."""
        kinds = set()
        for layer in self._sublayers():
            if not isinstance(layer, RandomLayer) or layer.output_dim_per_node != 1:
                return None
            kinds.add(layer._fused)
        kind = kinds.pop() if len(kinds) == 1 else None
        return kind if kind in _BANKED else None

    def _level_layers(self, level):
        """Sub-layers of a depth level in column order: level 0 the chunks, level l tree by tree."""
        return list(self.first_layer_chunks) if level == 0 else [tree[level - 1] for tree in self.trees]

    def _tie_levels(self):
        self._level_banks, self._level_scalar_banks = [], []
        for level in range(self.tree_depth + 1):
            nodes = [node for layer in self._level_layers(level) for node in layer.nodes]
            self._level_banks.append({name: ParameterBank(nodes, name) for name in _BANKED[self._kind]})
            self._level_scalar_banks.append({name: ScalarBank(nodes, name) for name in _BANKED_SCALARS[self._kind]})

    def _apply(self, fn, *args, **kwargs):
        grads = [{name: bank.flat.grad for name, bank in banks.items()} for banks in self._level_banks]
        for banks in self._level_banks:
            for bank in banks.values():
                bank.flat.grad = None
        super()._apply(fn, *args, **kwargs)
        for banks, kept in zip(self._level_banks, grads):
            for name, bank in banks.items():
                bank.tie(keep_grad=None if kept[name] is None else fn(kept[name]))
        for banks in self._level_scalar_banks:
            for bank in banks.values():
                bank.tie()
        self._plans = None
        return self

    def __setstate__(self, state):
        # after copy.deepcopy / unpickling the per-node Parameters are plain again: tie them to the level banks now
        super().__setstate__(state)
        self.__dict__.setdefault("_level_scalar_banks", [])
        if self._kind is not None:
            self._tie_levels()
        self._plans = None

    def _level_scalars(self, level):
        """What the kernels take for a depth level, every node's own values (a level runs as one fused layer call over
        the nodes of all its sub-layers): DWN (alpha [nodes], beta [nodes], max |beta|), probabilistic temperature [nodes]."""
        banks = self._level_scalar_banks[level]
        if self._kind == "dwn":
            return banks["alpha"].tensor(), banks["beta"].tensor(), banks["beta"].abs_max()
        return banks["temperature"].tensor()

    def invalidate_scalars(self):
        """After a write to a node's alpha / beta / temperature that bypasses the version counter (`.data` edits)."""
        for banks in self._level_scalar_banks:
            for bank in banks.values():
                bank.invalidate()

    def bank_parameters(self):
        """One leaf [nodes of the level, ...] per depth level and node parameter (what the fused calls
        differentiate); hand these to an optimizer instead of the per-node `parameters()`."""
        return [bank.tensor() for banks in self._level_banks for bank in banks.values()]

    def _level_plans(self, device):
        tables = [layer._mapping_indices for layer in self._sublayers()]
        key = (str(device),) + tuple((t.data_ptr(), t._version) for t in tables)
        if self._plans is None or self._plan_key != key:
            plans = []
            for level in range(self.tree_depth + 1):
                layers = self._level_layers(level)
                if level == 0:
                    idx = torch.cat([layer._mapping_indices.to(torch.int32) for layer in layers])
                    width = self.input_size
                else:
                    per_tree = self.hidden_layers[level - 1]
                    idx = torch.cat([layer._mapping_indices.to(torch.int32) + t * per_tree for t, layer in enumerate(layers)])
                    width = per_tree * self.out_channels
                plans.append(ops.MappingPlan(idx.to(device), width))
            self._plans, self._plan_key = plans, key
        return self._plans

    def _geometry(self):
        return (*self.receptive_field, *self.stride, *self.padding)

    def _chained(self):
        """DWN trees in training mode run as one chained call that reads the image itself."""
        return self._kind == "dwn" and self.training and self.n_inputs_per_node <= ops.FAST_K

    def _run_levels(self, patches, image=None, flip=None):
        """patches [rows, input_size] (or, chained, the image batch and the flip mask of its patch matrix) ->
        [rows, out_channels] through the depth levels."""
        device = patches.device if patches is not None else image.device
        plans = self._level_plans(device)
        banks = [{name: bank.tensor() for name, bank in level.items()} for level in self._level_banks]
        levels = range(self.tree_depth + 1)
        kind, h = self._kind, patches
        if image is not None:
            scalars = [self._level_scalars(level) for level in levels]
            source = self._geometry() if flip is None else (*self._geometry(), flip)
            return ops.DWNStackFunction.apply(image, source, plans, scalars, None, *[b["luts"] for b in banks])
        if kind == "dwn" and self.training and self.n_inputs_per_node <= ops.FAST_K and h.is_cuda:
            scalars = [self._level_scalars(level) for level in levels]
            return ops.DWNStackFunction.apply(h, None, plans, scalars, None, *[b["luts"] for b in banks])
        for level, plan, bank in zip(levels, plans, banks):
            if kind == "dwn":
                if self.training:
                    h = ops.dwn_layer(h, bank["luts"], plan, *self._level_scalars(level))
                else:
                    h = ops.dwn_layer_eval(h, bank["luts"].detach(), plan)
            elif kind == "probabilistic":
                temperature = self._level_scalars(level)
                if self.training:
                    h = ops.prob_layer(h, bank["raw_weights"], plan, temperature)
                else:
                    h = ops.prob_layer_eval(h, bank["raw_weights"].detach(), plan, temperature)
            elif not self.training:
                with torch.no_grad():
                    h = ops.dwn_layer_eval(h, ops.table_sigmoid(bank["raw_luts"]), plan)
            elif kind == "hybrid":
                h = ops.hybrid_layer(h, ops.table_sigmoid(bank["raw_luts"]), plan)
            else:
                h = ops.dwn_stable_layer(h, ops.table_sigmoid(bank["raw_luts"]),
                                                     bank["gradient_scale"].detach(), plan)
        return h

    def _loop_trees(self, patches):
        """The reference's loop (convolutional.py:214-242), for sub-layers without a fused kernel."""
        out = torch.empty(patches.shape[0], self.out_channels, device=patches.device)
        tree_idx = 0
        for chunk_idx, chunk in enumerate(self.first_layer_chunks):
            start = chunk_idx * self.chunk_size
            count = min(start + self.chunk_size, self.out_channels) - start
            first = chunk(patches).view(patches.shape[0], count, self.hidden_layers[0])
            for local in range(count):
                h = first[:, local, :]
                for layer in self.trees[tree_idx]:
                    h = layer(h)
                out[:, tree_idx] = h.squeeze(-1)
                tree_idx += 1
        return out

    # ------------------------------------------------------------------ interface
    def forward(self, x):
        if x.dim() != 4 or x.shape[1] != self.in_channels:
            raise ValueError(f"ConvolutionalLayer expects (batch, {self.in_channels}, height, width), got {tuple(x.shape)}")
        batch = x.shape[0]
        out_h = (x.shape[2] + 2 * self.padding[0] - self.receptive_field[0]) // self.stride[0] + 1
        out_w = (x.shape[3] + 2 * self.padding[1] - self.receptive_field[1]) // self.stride[1] + 1
        positions = out_h * out_w
        # bit-flip augmentation of the patch matrix (convolutional.py:205-207): the mask is drawn here, the patch
        # extraction applies it on the way (also when the patches only ever exist as bit-planes)
        flip = self._flip_mask((batch * positions, self.input_size), x.device)
        if self._kind is not None and self._chained() and x.is_cuda:
            out = self._run_levels(None, image=x, flip=flip)
        else:
            patches = ops.unfold(x, self._geometry(), flip)  # (batch * positions, channels * kh * kw)
            out = self._run_levels(patches) if self._kind is not None else self._loop_trees(patches)
        out = out.view(batch, positions, self.out_channels).transpose(1, 2)
        out = out.reshape(batch, self.out_channels, out_h, out_w)
        if self.grad_stabilization != "none" and self.training and out.requires_grad:
            def hook(grad):
                return self._apply_gradient_stabilization(grad.reshape(grad.shape[0], -1)).view(grad.shape)
            out.register_hook(hook)
        return out

    def __repr__(self):
        return (f"ConvolutionalLUTLayer(\n  receptive_field={self.receptive_field}, stride={self.stride}, "
                f"padding={self.padding}\n  in_channels={self.in_channels}, out_channels={self.out_channels}\n"
                f"  tree_architecture={self.hidden_layers}\n  node_type={self.node_type}, layer_type={self.layer_type}\n"
                f"  n_inputs_per_node={self.n_inputs_per_node}, tree_depth={self.tree_depth}\n"
                f"  total_trees={len(self.trees)}, chunk_size={self.chunk_size}, "
                f"num_chunks={len(self.first_layer_chunks)}\n)")
