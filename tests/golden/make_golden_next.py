#!/usr/bin/env python3
"""Golden vectors for the node types and layers added after the first set (gradient-stabilised DWN node,
hybrid node, grouped input mapping, convolutional layer), written by the reference's own CPU path.

Run in the build container only (the reference checkout does not travel):

    python tests/golden/make_golden_next.py [/root/reference]

The arithmetic of these pieces is pinned by mathematics in tests/test_oracle.py; what only the reference can
say is (a) which index tables GroupedInputConfig and a ConvolutionalLayer draw for a seed, and the values of
default-initialised `raw_luts` (both depend on how torch's CPU generator is consumed), and (b) that the chunk /
tree structure of a ConvolutionalLayer, loaded through its state dict, gives the same outputs and gradients
when every depth level is run as one block-diagonal layer.  Node vectors are stored as a cross-check.

Output: reference_vectors_next.npz (inputs and expected outputs only; no code).
"""
import os
import sys
import warnings

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
warnings.filterwarnings("ignore")

from difflut.layers.convolutional import ConvolutionalLayer, ConvolutionConfig  # noqa: E402
from difflut.layers.layer_config import GroupedInputConfig  # noqa: E402
from difflut.layers.random_layer import RandomLayer  # noqa: E402
from difflut.nodes.dwn_node import DWNNode  # noqa: E402
from difflut.nodes.dwn_stable_node import DWNStableNode  # noqa: E402
from difflut.nodes.hybrid_node import HybridNode  # noqa: E402
from difflut.nodes.node_config import NodeConfig  # noqa: E402
from difflut.nodes.probabilistic_node import ProbabilisticNode  # noqa: E402
from difflut.nodes.utils.initializers import uniform_init  # noqa: E402

out = {}


def put(name, t):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    out[name] = np.asarray(t)


# ------------------------------------------------ stabilised and hybrid nodes
torch.manual_seed(21)
for cls, kind in ((DWNStableNode, "stable"), (HybridNode, "hybrid")):
    for tag, B, k, O in (("k6o1", 12, 6, 1), ("k3o2", 9, 3, 2)):
        kw = {"gradient_scale": 1.6} if kind == "stable" else {}
        node = cls(input_dim=k, output_dim=O, use_cuda=False, **kw)
        put(f"{kind}_{tag}_default_raw", node.raw_luts)  # randn * 0.1 from the global generator
        node = cls(input_dim=k, output_dim=O, use_cuda=False, init_fn=uniform_init, init_kwargs={"a": -2.0, "b": 2.0}, **kw)
        node.train()
        x = (0.02 + 0.96 * torch.rand(B, k)).requires_grad_()
        gy = torch.randn(B, O)
        y = node(x)
        y.backward(gy)
        put(f"{kind}_{tag}_x", x); put(f"{kind}_{tag}_raw", node.raw_luts); put(f"{kind}_{tag}_gy", gy)
        put(f"{kind}_{tag}_y", y); put(f"{kind}_{tag}_gx", x.grad); put(f"{kind}_{tag}_graw", node.raw_luts.grad)
        node.eval()
        xb = torch.randint(0, 2, (B, k)).float()
        put(f"{kind}_{tag}_eval_x", xb); put(f"{kind}_{tag}_eval_y", node(xb))
put("next_rand_after_nodes", torch.rand(3))  # generator position: pins how the constructors consume it

# ------------------------------------------------ grouped input mapping
for tag, cover in (("cover", True), ("nocover", False)):
    torch.manual_seed(77)
    cfg = GroupedInputConfig(n_groups=4, input_size=36, output_trees=5, luts_per_tree=6, bits_per_node=6, seed=42,
                             ensure_full_coverage=cover)
    put(f"grouped_{tag}_table", cfg.mapping_indices)
    put(f"grouped_{tag}_chunk_1_3", cfg.get_mapping_indices(1, 3))
    put(f"grouped_{tag}_next_rand", torch.rand(2))  # the caller's generator state is restored

# ------------------------------------------------ convolutional layer, DWN trees of depth 2
torch.manual_seed(31)
conv_cfg = ConvolutionConfig(tree_depth=2, in_channels=2, out_channels=3, receptive_field=2, stride=1, padding=0,
                             chunk_size=2, seed=42)
layer = ConvolutionalLayer(conv_cfg, DWNNode,
                           NodeConfig(input_dim=2, output_dim=1, init_fn=uniform_init, init_kwargs={"a": -1.0, "b": 2.0}),
                           RandomLayer, n_inputs_per_node=2)
layer.train()
x = torch.rand(2, 2, 4, 4, requires_grad=True)
y = layer(x)
gy = torch.randn_like(y)
y.backward(gy)
put("conv_x", x); put("conv_y", y); put("conv_gy", gy); put("conv_gx", x.grad)
for name, value in layer.state_dict().items():
    put(f"conv_state.{name}", value)
for name, param in layer.named_parameters():
    put(f"conv_grad.{name}", param.grad)
layer.eval()
xb = torch.randint(0, 2, (2, 2, 4, 4)).float()
put("conv_eval_x", xb); put("conv_eval_y", layer(xb))

# grouped connections, probabilistic nodes, one level: only the drawn tables matter here
torch.manual_seed(32)
gcfg = ConvolutionConfig(tree_depth=1, in_channels=4, out_channels=5, receptive_field=3, stride=1, padding=0,
                         chunk_size=2, seed=43)
glayer = ConvolutionalLayer(gcfg, ProbabilisticNode, NodeConfig(input_dim=6, output_dim=1), RandomLayer,
                            n_inputs_per_node=6, grouped_connections=True, ensure_full_coverage=True)
for c, chunk in enumerate(glayer.first_layer_chunks):
    put(f"gconv_chunk{c}_idx", chunk._mapping_indices)
put("gconv_tree0_idx", glayer.trees[0][0]._mapping_indices)
put("gconv_tree4_idx", glayer.trees[4][0]._mapping_indices)
put("gconv_first_raw", glayer.first_layer_chunks[0].nodes[0].raw_weights)
put("gconv_last_raw", glayer.trees[4][0].nodes[0].raw_weights)

here = os.path.dirname(os.path.abspath(__file__))
np.savez_compressed(os.path.join(here, "reference_vectors_next.npz"), **out)
print(f"wrote {len(out)} arrays, torch {torch.__version__}")
