"""The CPU branch of the operators (`difflut_amd/cpu_ops.py`): a module that lives on the CPU takes plain-torch code,
as the reference's does (random_layer.py:272-304, dwn_node.py:319-338, probabilistic_node.py:277-300).  Checked here
against the oracle and the reference's vectors; none of these tests needs a device or the HIP library."""
import warnings

import numpy as np
import pytest
import torch

from oracle import difflut_oracle as orc

warnings.filterwarnings("ignore")


def _api():
    from difflut_amd import REGISTRY
    from difflut_amd.nodes import NodeConfig
    from difflut_amd.nodes.utils import uniform_init

    return REGISTRY, NodeConfig, uniform_init


def _random_layer(node, I, N, k, O=1, lo=-1.0, hi=1.0, seed=42):
    REGISTRY, NodeConfig, uniform_init = _api()
    return REGISTRY.get_layer("random")(I, N, REGISTRY.get_node(node),
                                        NodeConfig(input_dim=k, output_dim=O, init_fn=uniform_init,
                                                   init_kwargs={"a": lo, "b": hi}), seed=seed)


def _stacked(layer, name):
    return torch.stack([getattr(n, name).detach() for n in layer.nodes]).numpy()


def _stacked_grad(layer, name):
    return torch.stack([getattr(n, name).grad for n in layer.nodes]).numpy()


@pytest.mark.parametrize("k,O", [(2, 1), (4, 2), (6, 1), (7, 1)])
def test_random_dwn_layer_on_cpu_against_oracle(k, O):
    torch.manual_seed(k)
    B, I, N = 37, 45, 23
    layer = _random_layer("dwn", I, N, k, O)
    x = torch.rand(B, I, requires_grad=True)
    y = layer(x)
    assert y.device.type == "cpu" and y.shape == (B, N * O)
    gy = torch.randn_like(y)
    y.backward(gy)
    luts, idx = _stacked(layer, "luts"), layer._mapping_indices.numpy()
    assert np.array_equal(y.detach().numpy(), orc.dwn_layer_forward(x.detach().numpy(), idx, luts).reshape(B, -1))
    gx, gl = orc.dwn_layer_backward(x.detach().numpy(), idx, luts, gy.numpy().reshape(B, N, O),
                                    np.float32(0.5 * 0.75 ** (k - 1)), np.float32(1 / 3))
    np.testing.assert_allclose(x.grad.numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(_stacked_grad(layer, "luts"), gl, rtol=1e-5, atol=1e-5)
    layer.eval()
    xb = (torch.rand(B, I) > 0.5).float()
    want = np.stack([orc.dwn_eval_forward(xb.numpy()[:, idx[n]], luts[n]) for n in range(N)], axis=1).reshape(B, -1)
    with torch.no_grad():
        assert np.array_equal(layer(xb).numpy(), want)


def test_per_node_alpha_beta_on_cpu():
    """Every node's own alpha and beta are honoured (dwn_node.py:450 reads them per node)."""
    torch.manual_seed(3)
    B, I, N, k = 19, 30, 11, 4
    layer = _random_layer("dwn", I, N, k)
    alphas = torch.linspace(0.05, 0.4, N)
    betas = torch.linspace(0.0, 0.9, N)
    with torch.no_grad():
        for n, node in enumerate(layer.nodes):
            node.alpha.fill_(alphas[n])
            node.beta.fill_(betas[n])
    x = torch.rand(B, I, requires_grad=True)
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    luts, idx = _stacked(layer, "luts"), layer._mapping_indices.numpy()
    want = np.zeros((B, I), dtype=np.float64)
    for n in range(N):
        gxn, _ = orc.efd_backward(x.detach().numpy()[:, idx[n]], luts[n], gy.numpy()[:, n:n + 1],
                                  np.float32(alphas[n]), np.float32(betas[n]))
        np.add.at(want, (slice(None), idx[n].astype(np.int64)), gxn)
    np.testing.assert_allclose(x.grad.numpy(), want, rtol=1e-5, atol=2e-6)


def test_random_probabilistic_layer_on_cpu_against_oracle():
    torch.manual_seed(5)
    B, I, N, k = 33, 40, 17, 4
    layer = _random_layer("probabilistic", I, N, k, lo=0.0, hi=1.0)
    x = torch.sigmoid(torch.randn(B, I)).requires_grad_()
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    raw, idx = _stacked(layer, "raw_weights"), layer._mapping_indices.numpy()
    np.testing.assert_allclose(y.detach().numpy(), orc.prob_layer_forward(x.detach().numpy(), idx, raw)[:, :, 0],
                               rtol=1e-5, atol=1e-6)
    gx, gw = orc.prob_layer_backward(x.detach().numpy(), idx, raw, gy.numpy()[:, :, None])
    np.testing.assert_allclose(x.grad.numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(_stacked_grad(layer, "raw_weights"), gw, rtol=1e-5, atol=2e-6)
    layer.eval()
    xb = (torch.rand(B, I) > 0.5).float()
    want = np.stack([orc.prob_eval_forward(xb.numpy()[:, idx[n]], raw[n]) for n in range(N)], axis=1).reshape(B, -1)
    with torch.no_grad():
        assert np.array_equal(layer(xb).numpy(), want)


def test_per_node_temperature_on_cpu():
    torch.manual_seed(6)
    B, I, N, k = 12, 20, 7, 3
    layer = _random_layer("probabilistic", I, N, k, lo=-2.0, hi=2.0)
    temps = torch.linspace(0.5, 2.0, N)
    with torch.no_grad():
        for n, node in enumerate(layer.nodes):
            node.temperature.fill_(temps[n])
    x = torch.sigmoid(torch.randn(B, I))
    y = layer(x).detach().numpy()
    raw, idx = _stacked(layer, "raw_weights"), layer._mapping_indices.numpy()
    for n in range(N):
        want = orc.prob_forward(x.numpy()[:, idx[n]], raw[n], float(temps[n]))
        np.testing.assert_allclose(y[:, n:n + 1], want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("node", ["dwn_stable", "hybrid"])
def test_stable_and_hybrid_layers_on_cpu_against_oracle(node):
    torch.manual_seed(8)
    B, I, N, k = 21, 36, 13, 4
    layer = _random_layer(node, I, N, k, lo=-2.0, hi=2.0)
    x = torch.rand(B, I, requires_grad=True)
    y = layer(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    raw, idx = _stacked(layer, "raw_luts"), layer._mapping_indices.numpy()
    # the looked-up entries are torch.sigmoid(raw) as in the reference (dwn_stable_node.py:289-295); the oracle's
    # sigmoid may round the last bit the other way
    np.testing.assert_allclose(y.detach().numpy(),
                               orc.dwn_layer_forward(x.detach().numpy(), idx, orc.table_sigmoid(raw)).reshape(B, -1),
                               rtol=1e-6, atol=0)
    if node == "dwn_stable":
        scale = np.array([float(n.gradient_scale) for n in layer.nodes], dtype=np.float32)
        gx, graw = orc.stable_layer_backward(x.detach().numpy(), idx, raw, gy.numpy().reshape(B, N, 1), scale)
    else:
        gx, graw = orc.hybrid_layer_backward(x.detach().numpy(), idx, raw, gy.numpy().reshape(B, N, 1))
    np.testing.assert_allclose(x.grad.numpy(), gx, rtol=1e-4, atol=2e-6)
    np.testing.assert_allclose(_stacked_grad(layer, "raw_luts"), graw, rtol=1e-4, atol=2e-6)


def test_learnable_layer_on_cpu_against_oracle():
    REGISTRY, NodeConfig, uniform_init = _api()
    torch.manual_seed(9)
    B, I, N, k = 14, 24, 9, 3
    layer = REGISTRY.get_layer("learnable")(I, N, REGISTRY.get_node("dwn"),
                                            NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init,
                                                       init_kwargs={"a": -1.0, "b": 1.0}),
                                            tau=1.0, tau_start=1.0, tau_min=1e-4, tau_decay_iters=1000.0)
    x = torch.rand(B, I, requires_grad=True)
    mapped = layer.get_mapping(x)
    W = layer.mapping.W.detach().numpy()
    np.testing.assert_allclose(mapped.detach().numpy().reshape(B, -1), orc.soft_mapping_forward(x.detach().numpy(), W, 1.0),
                               rtol=1e-5, atol=1e-6)
    y = layer(x)
    y.backward(torch.randn_like(y))
    assert x.grad is not None and layer.mapping.W.grad is not None and float(layer.mapping.W.grad.abs().sum()) > 0
    layer.eval()
    with torch.no_grad():
        picked = layer.get_mapping(x).numpy().reshape(B, -1)
    np.testing.assert_array_equal(picked, orc.hard_mapping(x.detach().numpy(), W)[0])
    assert np.array_equal(layer.get_mapping_matrix().numpy().reshape(-1), W.argmax(-1))


def test_smallest_training_configuration_on_cpu(golden):
    """thermometer -> RandomLayer + DWN -> GroupSum -> cross-entropy on the CPU against the reference's numbers,
    module by module and through a DWNStack (which runs its members one by one there)."""
    REGISTRY, NodeConfig, uniform_init = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum, cross_entropy

    g = golden
    x = torch.tensor(g["e2e_x"])
    enc = REGISTRY.build_encoder("thermometer", num_bits=4).fit(x)
    bits = enc.encode(x).requires_grad_()
    assert np.array_equal(bits.detach().numpy(), g["e2e_bits"])
    layer = _random_layer("dwn", 80, 30, 6)
    assert np.array_equal(layer._mapping_indices.numpy(), g["e2e_idx"])
    with torch.no_grad():
        for n, node in enumerate(layer.nodes):
            node.luts.copy_(torch.tensor(g["e2e_luts"][n]))
    logits = GroupSum(k=10, tau=1.0, use_randperm=False)(layer(bits))
    np.testing.assert_allclose(logits.detach().numpy(), g["e2e_logits"], rtol=1e-6, atol=1e-6)
    loss = cross_entropy(logits, torch.tensor(g["e2e_labels"]))
    assert loss.item() == pytest.approx(float(g["e2e_loss"]), rel=1e-6)
    loss.backward()
    np.testing.assert_allclose(bits.grad.numpy(), g["e2e_gbits"], rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(_stacked_grad(layer, "luts"), g["e2e_gluts"], rtol=1e-5, atol=1e-7)
    stack = DWNStack([layer], encoder=enc, head=GroupSum(k=10, tau=1.0, use_randperm=False))
    np.testing.assert_allclose(stack(x).detach().numpy(), g["e2e_logits"], rtol=1e-6, atol=1e-6)


def test_convolutional_layer_on_cpu_against_reference_vectors(golden_next):
    from difflut_amd.layers import ConvolutionalLayer, ConvolutionConfig, RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig

    g = golden_next
    cfg = ConvolutionConfig(tree_depth=2, in_channels=2, out_channels=3, receptive_field=2, stride=1, padding=0,
                            chunk_size=2, seed=42)
    layer = ConvolutionalLayer(cfg, DWNNode, NodeConfig(input_dim=2, output_dim=1), RandomLayer, n_inputs_per_node=2)
    layer.load_state_dict({k[len("conv_state."):]: torch.tensor(v) for k, v in g.items() if k.startswith("conv_state.")})
    layer.train()
    x = torch.tensor(g["conv_x"], requires_grad=True)
    y = layer(x)
    assert np.array_equal(y.detach().numpy(), g["conv_y"])
    y.backward(torch.tensor(g["conv_gy"]))
    np.testing.assert_allclose(x.grad.numpy(), g["conv_gx"], rtol=1e-5, atol=2e-6)
    for name, param in layer.named_parameters():
        want = g.get(f"conv_grad.{name}")
        if want is not None and want.shape != ():
            np.testing.assert_allclose(param.grad.numpy(), want, rtol=1e-5, atol=2e-6, err_msg=name)
    layer.eval()
    with torch.no_grad():
        assert np.array_equal(layer(torch.tensor(g["conv_eval_x"])).numpy(), g["conv_eval_y"])


def test_single_nodes_on_cpu(golden):
    """A node called on its own (the reference's node-level entry points) on CPU tensors."""
    from difflut_amd.nodes import DWNNode, ProbabilisticNode

    torch.manual_seed(4)
    node = DWNNode(input_dim=4, output_dim=2)
    x = torch.rand(9, 4, requires_grad=True)
    y = node(x)
    assert np.array_equal(y.detach().numpy(), orc.dwn_forward(x.detach().numpy(), node.luts.detach().numpy()))
    gy = torch.randn_like(y)
    y.backward(gy)
    gx, gl = orc.efd_backward(x.detach().numpy(), node.luts.detach().numpy(), gy.numpy(), np.float32(node.alpha),
                              np.float32(node.beta))
    np.testing.assert_allclose(x.grad.numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(node.luts.grad.numpy(), gl, rtol=1e-5, atol=1e-6)
    pnode = ProbabilisticNode(input_dim=3, output_dim=2)
    xp = torch.rand(7, 3)
    np.testing.assert_allclose(pnode(xp).detach().numpy(),
                               orc.prob_forward(xp.numpy(), pnode.raw_weights.detach().numpy(), 1.0), rtol=1e-5, atol=1e-6)


def test_bank_adam_matches_torch_adam_on_cpu():
    from difflut_amd.utils import BankAdam

    torch.manual_seed(2)
    a = [torch.randn(7, 1, 16, requires_grad=True), torch.randn(33, requires_grad=True)]
    b = [t.detach().clone().requires_grad_() for t in a]
    ours, ref = BankAdam(a, lr=0.01, weight_decay=0.1), torch.optim.Adam(b, lr=0.01, weight_decay=0.1)
    for _ in range(4):
        for x, y in zip(a, b):
            g = torch.randn_like(x)
            x.grad, y.grad = g.clone(), g.clone()
        ours.step()
        ref.step()
    for x, y in zip(a, b):
        np.testing.assert_allclose(x.detach().numpy(), y.detach().numpy(), rtol=1e-6, atol=1e-7)
