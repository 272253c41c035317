#!/usr/bin/env python3
"""Write the golden vectors in this folder by running the reference's own CPU path.

Run in the build container only (the reference checkout does not travel):

    python tests/golden/make_golden.py [/root/reference]

What is snapshotted, and why an import is the only way to pin it:
  * the exact index table RandomLayer draws for a seed (reference
    difflut/layers/random_layer.py:195-256) - depends on how many numbers each
    torch CPU-generator call consumes, which no closed form states;
  * the default-initialised tables of a seeded layer (dwn_node.py:423,
    probabilistic_node.py:224) - same reason;
  * one end-to-end pass of the smallest training configuration (thermometer ->
    RandomLayer+DWN -> GroupSum -> cross-entropy) with every gradient, as a
    single cross-check of the restated pieces working together.
For completeness the per-function vectors (DWN fwd/EFD bwd, probabilistic
fwd/bwd, soft/hard learnable mapping, thermometer, GroupSum) are stored too, so
the oracle is compared with the reference's numbers and not only with maths.

Outputs: reference_vectors.npz (inputs and expected outputs only; no code).
"""
import os
import sys
import warnings

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
warnings.filterwarnings("ignore")

from difflut.encoder.thermometer import ThermometerEncoder  # noqa: E402
from difflut.layers.learnable_layer import LearnableLayer  # noqa: E402
from difflut.layers.random_layer import RandomLayer  # noqa: E402
from difflut.nodes.dwn_node import DWNNode  # noqa: E402
from difflut.nodes.node_config import NodeConfig  # noqa: E402
from difflut.nodes.probabilistic_node import ProbabilisticNode  # noqa: E402
from difflut.nodes.utils.initializers import residual_init, uniform_init  # noqa: E402
from difflut.utils.modules import GroupSum  # noqa: E402

out = {}


def put(name, t):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    out[name] = np.asarray(t)


# ---------------------------------------------------------------- a1 mapping
MAPPING_CASES = [  # (tag, I, N, k, seed, full_coverage)
    ("fused_a", 25, 36, 6, 42, True),
    ("fused_b", 16, 25, 4, 42, True),
    ("layer_fn", 256, 128, 4, 42, True),
    ("exact3", 48, 24, 6, 7, True),  # N*k = 3*I exactly, no multinomial tail
    ("cfg1", 3136, 2000, 6, 42, True),
    ("nocover", 64, 20, 6, 7, False),
]
for tag, I, N, k, seed, cover in MAPPING_CASES:
    torch.manual_seed(1234)
    before = torch.get_rng_state()
    layer = RandomLayer(
        I, N, DWNNode, NodeConfig(input_dim=k, output_dim=1), seed=seed,
        ensure_full_input_coverage=cover,
    )
    put(f"map_{tag}_idx", layer._mapping_indices)
    put(f"map_{tag}_meta", np.array([I, N, k, seed, int(cover)], dtype=np.int64))
    # tables of the first and last node: pins that node construction consumes the
    # global generator in node order, before the (state-restoring) mapping draw
    put(f"map_{tag}_lut_first", layer.nodes[0].luts)
    put(f"map_{tag}_lut_last", layer.nodes[N - 1].luts)
    put(f"map_{tag}_next_rand", torch.rand(4))  # generator position after construction

# ------------------------------------------------------ a6/a8/a9 DWN node
torch.manual_seed(0)
for tag, B, k, O in [("k6o2", 16, 6, 2), ("k4o1", 12, 4, 1), ("k2o3", 9, 2, 3)]:
    node = DWNNode(input_dim=k, output_dim=O, init_fn=uniform_init, init_kwargs={"a": -1.0, "b": 1.0})
    node.train()
    x = torch.rand(B, k, requires_grad=True)
    gy = torch.randn(B, O)
    y = node(x)
    y.backward(gy)
    put(f"dwn_{tag}_x", x)
    put(f"dwn_{tag}_luts", node.luts)
    put(f"dwn_{tag}_gy", gy)
    put(f"dwn_{tag}_y", y)
    put(f"dwn_{tag}_gx", x.grad)
    put(f"dwn_{tag}_gl", node.luts.grad)
    put(f"dwn_{tag}_ab", np.array([node.alpha.item(), node.beta.item()], dtype=np.float64))
    node.eval()
    xb = torch.randint(0, 2, (B, k)).float()
    put(f"dwn_{tag}_eval_x", xb)
    put(f"dwn_{tag}_eval_y", node(xb))

# non-default alpha / beta
node = DWNNode(input_dim=3, output_dim=1, alpha=0.7, beta=0.9, init_fn=uniform_init,
               init_kwargs={"a": -1.0, "b": 1.0})
x = torch.rand(10, 3, requires_grad=True)
gy = torch.randn(10, 1)
node(x).backward(gy)
put("dwn_ab_x", x); put("dwn_ab_luts", node.luts); put("dwn_ab_gy", gy)
put("dwn_ab_gx", x.grad); put("dwn_ab_gl", node.luts.grad)

# residual-init known answer (reference tests/test_nodes/test_residual_initialization.py:56-105)
node = DWNNode(input_dim=6, output_dim=1, init_fn=residual_init,
               init_kwargs={"node_type": "dwn", "noise_factor": 0.0, "logit_clarity": 5.0, "input_dim": 6})
put("dwn_residual_luts", node.luts)

# --------------------------------------------- a11/a12/a13 probabilistic node
for tag, B, k, O, T in [("k4o2", 32, 4, 2, 1.0), ("k6o1", 20, 6, 1, 0.5)]:
    node = ProbabilisticNode(input_dim=k, output_dim=O, init_fn=uniform_init,
                             init_kwargs={"a": 0.0, "b": 1.0}, temperature=T, use_cuda=False)
    node.train()
    x = torch.sigmoid(torch.randn(B, k)).requires_grad_()
    gy = torch.randn(B, O)
    y = node(x)
    y.backward(gy)
    put(f"prob_{tag}_x", x); put(f"prob_{tag}_w", node.raw_weights); put(f"prob_{tag}_gy", gy)
    put(f"prob_{tag}_y", y); put(f"prob_{tag}_gx", x.grad); put(f"prob_{tag}_gw", node.raw_weights.grad)
    put(f"prob_{tag}_T", np.array([T], dtype=np.float64))
    node.eval()
    xb = torch.randint(0, 2, (B, k)).float()
    put(f"prob_{tag}_eval_x", xb); put(f"prob_{tag}_eval_y", node(xb))

# ------------------------------------------------ a14 learnable mapping
torch.manual_seed(3)
lay = LearnableLayer(20, 7, DWNNode, NodeConfig(input_dim=3, output_dim=1), tau=1.0, tau_start=1.0,
                     tau_min=1e-4, tau_decay_iters=1000.0, use_cuda_soft=False)
lay.train()
x = torch.rand(5, 20, requires_grad=True)
m = lay.get_mapping(x)
gm = torch.randn_like(m)
m.backward(gm)
put("soft_x", x); put("soft_W", lay.mapping.W); put("soft_gm", gm); put("soft_m", m)
put("soft_gx", x.grad); put("soft_gW", lay.mapping.W.grad); put("soft_tau", np.array([lay.tau]))
lay.eval()
put("hard_m", lay.get_mapping(x.detach()))
put("hard_idx", lay.get_mapping_matrix())
lay.update_tau(500)
put("soft_tau_500", np.array([lay.tau]))
lay.train()
lay.mapping.W.grad = None
x2 = x.detach().clone().requires_grad_()
m2 = lay.get_mapping(x2)
m2.backward(gm)
put("soft500_m", m2); put("soft500_gx", x2.grad); put("soft500_gW", lay.mapping.W.grad)

# ------------------------------------------------ a16 thermometer, a17 GroupSum
torch.manual_seed(4)
xt = torch.rand(9, 5) * 3.0 - 1.0
enc = ThermometerEncoder(num_bits=4).fit(xt)
put("thermo_x", xt); put("thermo_thr", enc.thresholds); put("thermo_bits", enc.encode(xt))
gs = GroupSum(k=5, tau=2.0, use_randperm=False)
xg = torch.randn(6, 20)
put("groupsum_x", xg); put("groupsum_y", gs(xg))

# ---------------------------------------- smallest training configuration, reduced
torch.manual_seed(5)
B, F, N, k = 8, 20, 30, 6
xr = torch.rand(B, F)
enc = ThermometerEncoder(num_bits=4).fit(xr)
bits = enc.encode(xr).requires_grad_()
layer = RandomLayer(F * 4, N, DWNNode,
                    NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init,
                               init_kwargs={"a": -1.0, "b": 1.0}), seed=42)
layer.train()
head = GroupSum(k=10, tau=1.0, use_randperm=False)
labels = torch.randint(0, 10, (B,))
logits = head(layer(bits))
loss = torch.nn.functional.cross_entropy(logits, labels)
loss.backward()
put("e2e_x", xr); put("e2e_bits", bits); put("e2e_idx", layer._mapping_indices)
put("e2e_luts", torch.stack([n.luts for n in layer.nodes]))
put("e2e_labels", labels); put("e2e_logits", logits); put("e2e_loss", loss)
put("e2e_gbits", bits.grad)
put("e2e_gluts", torch.stack([n.luts.grad for n in layer.nodes]))

here = os.path.dirname(os.path.abspath(__file__))
np.savez_compressed(os.path.join(here, "reference_vectors.npz"), **out)
print(f"wrote {len(out)} arrays, torch {torch.__version__}")
