"""Per-node alpha / beta (dwn_node.py:417-418, 450: every node reads its own buffers): a state dict that gives the nodes
of one layer different values is honoured node by node - by RandomLayer.forward against the oracle, by chained stacks
and convolutional levels against the layers called one by one; the same for the probabilistic node's temperature
(probabilistic_node.py:277-282)."""
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


def _spread_scalars(layer, alphas, betas):
    with torch.no_grad():
        for n, node in enumerate(layer.nodes):
            node.alpha.fill_(alphas[n % len(alphas)])
            node.beta.fill_(betas[(n // 2) % len(betas)])


@pytest.mark.parametrize("head", [False, True])
@pytest.mark.parametrize("betas", [(1 / 3, 0.25, 0.1), (1 / 3, 0.8)])  # shared table form / per-slot form
def test_chained_layers_take_every_nodes_own_scalars(betas, head):
    """A DWNStack whose layers carry per-node alpha / beta equals the same layers called one by one (each of which is
    checked against the oracle node by node above): outputs bit for bit, gradients to rounding."""
    import copy

    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum

    torch.manual_seed(21)
    layers = [_layer(40, 128, 6), _layer(128, 640, 6), _layer(640, 640, 5)]
    for li, layer in enumerate(layers):
        _spread_scalars(layer, (0.1, 0.3, 0.2 + 0.05 * li), betas)
    layers = [layer.cuda().train() for layer in layers]
    twins = copy.deepcopy(layers)
    group = GroupSum(k=10, tau=2.0, use_randperm=False) if head else None
    stack = DWNStack(layers, head=group).train()
    x = torch.rand(200, 40, device="cuda")
    x1, x2 = x.clone().requires_grad_(), x.clone().requires_grad_()
    y = stack(x1)
    h = x2
    for layer in twins:
        h = layer(h)
    if head:
        h = group(h)
    np.testing.assert_allclose(y.detach().cpu().numpy(), h.detach().cpu().numpy(), rtol=1e-6, atol=1e-6)
    gy = torch.randn_like(y)
    y.backward(gy)
    h.backward(gy)
    np.testing.assert_allclose(x1.grad.cpu().numpy(), x2.grad.cpu().numpy(), rtol=1e-5, atol=2e-6)
    for a, b in zip(layers, twins):
        np.testing.assert_allclose(a._banks["luts"].flat.grad.cpu().numpy(), b._banks["luts"].flat.grad.cpu().numpy(),
                                   rtol=1e-5, atol=1e-5)
    # and the gradients do depend on the nodes' values: node 5 of the last layer with alpha = 0 sends nothing back
    with torch.no_grad():
        layers[-1].nodes[5].alpha.fill_(0.0)
    if not head:
        only5 = torch.zeros_like(gy)
        only5[:, 5] = gy[:, 5]
        x3 = x.clone().requires_grad_()
        stack(x3).backward(only5)
        assert float(x3.grad.abs().max()) == 0.0


@pytest.mark.parametrize("k", [4, 7])  # the tiled kernels and the generic ones
def test_probabilistic_layer_with_per_node_temperatures_against_oracle(k):
    from difflut_amd.layers import RandomLayer
    from difflut_amd.nodes import NodeConfig, ProbabilisticNode
    from difflut_amd.nodes.utils import uniform_init

    torch.manual_seed(5 + k)
    B, I, N = 150, 48, 37
    layer = RandomLayer(I, N, ProbabilisticNode, NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init,
                                                             init_kwargs={"a": -2.0, "b": 2.0}), seed=3)
    temps = np.linspace(0.4, 2.5, N).astype(np.float32)
    state = layer.state_dict()
    for n in range(N):
        state[f"nodes.{n}.temperature"] = torch.tensor(temps[n])
    layer.load_state_dict(state)
    layer = layer.cuda().train()
    x = torch.sigmoid(torch.randn(B, I, device="cuda")).requires_grad_()
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    xs, idx = x.detach().cpu().numpy(), layer._mapping_indices.cpu().numpy().astype(np.int64)
    raw = layer._banks["raw_weights"].flat.detach().cpu().numpy()
    want_gx = np.zeros((B, I), np.float64)
    for n in range(N):
        xk = xs[:, idx[n]]
        np.testing.assert_allclose(y.detach().cpu().numpy()[:, n:n + 1], orc.prob_forward(xk, raw[n], float(temps[n])),
                                   rtol=1e-5, atol=1e-6)
        gxn, gwn = orc.prob_backward(xk, raw[n], gy.cpu().numpy()[:, n:n + 1], float(temps[n]))
        np.add.at(want_gx, (slice(None), idx[n]), gxn)
        np.testing.assert_allclose(layer._banks["raw_weights"].flat.grad[n].cpu().numpy(), gwn, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(x.grad.cpu().numpy(), want_gx, rtol=1e-5, atol=4e-6)
    layer.eval()
    xb = (torch.rand(B, I, device="cuda") > 0.5).float()
    with torch.no_grad():
        ye = layer(xb).cpu().numpy()
    for n in range(N):
        assert np.array_equal(ye[:, n:n + 1], orc.prob_eval_forward(xb.cpu().numpy()[:, idx[n]], raw[n], float(temps[n])))


def test_convolutional_levels_take_every_nodes_own_scalars():
    """A reference state dict whose nodes differ inside a depth level runs, and equals the CPU branch of the same
    layer (checked against the reference's vectors and the oracle in tests/test_cpu_dispatch.py)."""
    import copy

    from difflut_amd.layers import ConvolutionalLayer, ConvolutionConfig, RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig
    from difflut_amd.nodes.utils import uniform_init

    torch.manual_seed(77)
    cfg = ConvolutionConfig(tree_depth=2, in_channels=3, out_channels=5, receptive_field=3, stride=1, padding=1,
                            chunk_size=2, seed=11)
    layer = ConvolutionalLayer(cfg, DWNNode, NodeConfig(input_dim=3, output_dim=1, init_fn=uniform_init,
                                                        init_kwargs={"a": -1.0, "b": 1.0}), RandomLayer,
                               n_inputs_per_node=3)
    count = 0
    with torch.no_grad():
        for sub in layer._sublayers():
            for node in sub.nodes:
                node.alpha.fill_(0.05 + 0.01 * (count % 7))
                node.beta.fill_((0.1, 1 / 3, 0.7)[count % 3])
                count += 1
    cpu = copy.deepcopy(layer).train()
    dev = layer.cuda().train()
    x = torch.rand(6, 3, 9, 9)
    xc, xd = x.clone().requires_grad_(), x.cuda().requires_grad_()
    yc, yd = cpu(xc), dev(xd)
    assert np.array_equal(yd.detach().cpu().numpy(), yc.detach().numpy())
    gy = torch.randn_like(yc)
    yc.backward(gy)
    yd.backward(gy.cuda())
    np.testing.assert_allclose(xd.grad.cpu().numpy(), xc.grad.numpy(), rtol=1e-5, atol=4e-6)
    for (name, pc), (_, pd) in zip(cpu.named_parameters(), dev.named_parameters()):
        np.testing.assert_allclose(pd.grad.cpu().numpy(), pc.grad.numpy(), rtol=1e-5, atol=1e-5, err_msg=name)
