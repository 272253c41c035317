"""Per-node alpha / beta (dwn_node.py:417-418, 450: every node reads its own buffers): a state dict that gives the nodes
of one layer different values is honoured by RandomLayer.forward, node by node, against the oracle; the paths that take
one pair per layer refuse it."""
import numpy as np
import pytest
import torch

from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu


def _layer(I, N, k, O=1):
    from difflut_amd.layers import RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig
    from difflut_amd.nodes.utils import uniform_init
    return RandomLayer(I, N, DWNNode, NodeConfig(input_dim=k, output_dim=O, init_fn=uniform_init,
                                                 init_kwargs={"a": -1.0, "b": 1.0}), seed=9)


@pytest.mark.parametrize("case", [(130, 50, 40, 6, 1, (0.1, 0.3), (1 / 3, 0.25)),    # every |beta| <= 1/2: shared table form
                                  (70, 30, 33, 4, 2, (0.2, 0.05), (1 / 3, 0.8)),     # one beta above 1/2: per-slot form
                                  (9, 30, 11, 7, 1, (0.1, 0.4), (0.3, 0.6))])        # k > 6: generic kernels
def test_state_dict_with_two_alphas_and_betas_against_oracle_per_node(case):
    B, I, N, k, O, alphas, betas = case
    torch.manual_seed(B + N)
    layer = _layer(I, N, k, O)
    state = layer.state_dict()
    for n in range(N):
        state[f"nodes.{n}.alpha"] = torch.tensor(alphas[n % 2], dtype=torch.float32)
        state[f"nodes.{n}.beta"] = torch.tensor(betas[(n // 2) % 2], dtype=torch.float32)
    layer.load_state_dict(state)
    layer = layer.cuda().train()
    x = torch.rand(B, I, device="cuda", requires_grad=True)
    gy = torch.randn(B, N * O, device="cuda")
    y = layer(x)
    y.backward(gy)
    xs, idx = x.detach().cpu().numpy(), layer._mapping_indices.cpu().numpy().astype(np.int64)
    luts = layer._banks["luts"].flat.detach().cpu().numpy()
    assert np.array_equal(y.detach().cpu().numpy(), orc.dwn_layer_forward(xs, idx, luts).reshape(B, N * O))
    # the input gradient is linear in gy: one oracle run per (alpha, beta) pair on the gradient of the nodes that carry it
    g = gy.cpu().numpy().reshape(B, N, O)
    want_gx, want_gl = np.zeros((B, I), np.float64), None
    for ia, a in enumerate(alphas):
        for ib, b in enumerate(betas):
            mask = np.array([(n % 2 == ia) and ((n // 2) % 2 == ib) for n in range(N)])
            gxa, gl = orc.dwn_layer_backward(xs, idx, luts, g * mask[None, :, None], np.float32(a), np.float32(b))
            want_gx += gxa
            want_gl = gl if want_gl is None else want_gl + gl
    np.testing.assert_allclose(x.grad.cpu().numpy(), want_gx, rtol=1e-5, atol=4e-6)
    np.testing.assert_allclose(layer._banks["luts"].flat.grad.cpu().numpy(), want_gl, rtol=1e-5, atol=1e-5)
    # one node's values changed in place afterwards are seen on the next call
    with torch.no_grad():
        layer.nodes[3].alpha.fill_(0.0)
    x2 = x.detach().clone().requires_grad_()
    only3 = torch.zeros_like(gy)
    only3[:, 3 * O:(3 + 1) * O] = gy[:, 3 * O:(3 + 1) * O]
    layer(x2).backward(only3)
    assert float(x2.grad.abs().max()) == 0.0


def test_chained_layers_refuse_per_node_scalars():
    from difflut_amd.layers import DWNStack
    a, b = _layer(40, 64, 6).cuda(), _layer(64, 32, 6).cuda()
    with torch.no_grad():
        b.nodes[10].beta.fill_(0.5)
    stack = DWNStack([a, b]).train()
    with pytest.raises(RuntimeError, match="different alpha / beta"):
        stack(torch.rand(70, 40, device="cuda"))
    with torch.no_grad():
        for node in b.nodes:
            node.beta.fill_(0.5)   # one value for the whole layer again, just not the default
    y = stack(torch.rand(70, 40, device="cuda"))
    assert y.shape == (70, 32)
