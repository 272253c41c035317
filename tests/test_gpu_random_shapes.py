"""Seeded sweep over random layer shapes: chained execution (with and without a GroupSum head) against the
layers one by one, the first layer's forward against the oracle bit for bit, and chained inference on binary
input against the layers' own eval forward.  The shapes are drawn so that tables made of whole permutations
(every input used exactly three times), long per-input lists, one input per node (k = 1), several outputs per
node and ragged batch sizes all occur."""
import warnings

import numpy as np
import pytest
import torch

from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu


def _draw(rng):
    B = int(rng.integers(1, 400))
    I = int(rng.integers(8, 260))
    k = int(rng.integers(1, 7))
    O = int(rng.choice([1, 1, 2]))
    depth = int(rng.integers(1, 4))
    widths = [int(rng.integers(max(2, k), 400)) for _ in range(depth)]
    if rng.random() < 0.4 and depth >= 2 and (widths[0] * O * 3) % k == 0:
        widths[1] = max(k, (widths[0] * O * 3) // k)      # three whole permutations of the first layer's outputs
    if rng.random() < 0.3:
        widths[0] = int(I * rng.integers(2, 12))          # long lists per input
    groups = int(rng.choice([0, 2, 3, 5]))
    tau = float(rng.choice([1.0, 0.5, 3.0]))
    return B, I, k, O, widths, groups, tau


@pytest.mark.parametrize("seed", [1, 2])
def test_random_shapes_chained_head_and_eval(seed):
    from difflut_amd import REGISTRY
    from difflut_amd.layers import DWNStack
    from difflut_amd.nodes.node_config import NodeConfig
    from difflut_amd.nodes.utils import uniform_init
    from difflut_amd.utils import GroupSum
    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for case in range(30):
            B, I, k, O, widths, groups, tau = _draw(rng)
            what = f"seed {seed} case {case}: B={B} I={I} k={k} O={O} widths={widths} groups={groups} tau={tau}"
            layers, width = [], I
            for li, n in enumerate(widths):
                layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                           NodeConfig(input_dim=k, output_dim=O, init_fn=uniform_init,
                                                                      init_kwargs={"a": -1.0, "b": 2.0}),
                                                           seed=case * 7 + li).cuda())
                width = n * O
            head = GroupSum(k=groups, tau=tau, use_randperm=False) if groups else None
            x = torch.rand(B, I, device="cuda")
            xa = x.clone().requires_grad_()
            h = xa
            for layer in layers:
                h = layer(h)
            out = head(h) if head else h
            gy = torch.randn_like(out)
            out.backward(gy)
            want_gl = [layer._banks["luts"].flat.grad.clone() for layer in layers]
            want_gx = xa.grad.clone()
            for layer in layers:
                layer._banks["luts"].flat.grad = None
            stack = DWNStack(layers, head=head).train()
            xb = x.clone().requires_grad_()
            got = stack(xb)
            got.backward(gy)
            torch.testing.assert_close(got, out, rtol=1e-5, atol=1e-5, msg=lambda m: f"{what}: output\n{m}")
            for li, (layer, want) in enumerate(zip(layers, want_gl)):
                torch.testing.assert_close(layer._banks["luts"].flat.grad, want, rtol=1e-4,
                                           atol=1e-5 * max(1.0, float(want.abs().max())),
                                           msg=lambda m: f"{what}: table gradient of layer {li}\n{m}")
                layer._banks["luts"].flat.grad = None
            torch.testing.assert_close(xb.grad, want_gx, rtol=1e-4, atol=1e-5 * max(1.0, float(want_gx.abs().max())),
                                       msg=lambda m: f"{what}: input gradient\n{m}")
            # first layer: forward and both gradients against the oracle
            idx = layers[0]._mapping_indices.cpu().numpy().astype(np.int64)
            luts = layers[0]._banks["luts"].tensor().detach().cpu().numpy()
            xc = x.clone().requires_grad_()
            y0 = layers[0](xc)
            assert np.array_equal(y0.detach().cpu().numpy().reshape(B, widths[0], O),
                                  orc.dwn_layer_forward(x.cpu().numpy(), idx, luts)), what
            g0 = torch.randn_like(y0)
            y0.backward(g0)
            alpha, beta = layers[0].nodes[0].efd_scalars()
            ogx, ogl = orc.dwn_layer_backward(x.cpu().numpy(), idx, luts, g0.cpu().numpy().reshape(B, widths[0], O),
                                              np.float32(alpha), np.float32(beta))
            np.testing.assert_allclose(xc.grad.cpu().numpy(), ogx, rtol=1e-4, atol=1e-5 * max(1.0, float(np.abs(ogx).max())),
                                       err_msg=what)
            np.testing.assert_allclose(layers[0]._banks["luts"].flat.grad.cpu().numpy().reshape(ogl.shape), ogl, rtol=1e-4,
                                       atol=1e-5 * max(1.0, float(np.abs(ogl).max())), err_msg=what)
            # inference on binary input, chained against one by one
            xbin = torch.bernoulli(torch.full((B, I), 0.5, device="cuda"))
            chained = DWNStack(layers, head=head, binary_input=True).eval()(xbin)
            he = xbin
            for layer in layers:
                layer.eval()
                he = layer(he)
            assert torch.equal(chained, head(he) if head else he), what
