"""GPU tests through the public layer/node API, shaped after the reference's own tests
(tests/test_layers/test_fused_kernels.py, test_layer_functionality.py,
tests/test_nodes/test_node_functionality.py, test_residual_initialization.py) with the CPU oracle
standing in for the reference's CPU path, plus size-independent properties at the full benchmark
shape (batch 4096 x 16384 inputs x 8192 nodes)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu


def _api():
    from difflut_amd import REGISTRY
    from difflut_amd.nodes import NodeConfig
    from difflut_amd.nodes.utils import residual_init, uniform_init
    return REGISTRY, NodeConfig, uniform_init, residual_init


def stacked(layer, name):
    return torch.stack([getattr(n, name).detach() for n in layer.nodes]).cpu().numpy()


def test_basic_functionality_fused_shapes():
    """test_fused_kernels.py:16-49: I=25, N=36, k=6, batch 100 of randn inputs."""
    REGISTRY, NodeConfig, _, _ = _api()
    layer = REGISTRY.get_layer("random")(input_size=25, output_size=36, node_type=REGISTRY.get_node("dwn"),
                                         node_kwargs=NodeConfig(input_dim=6, output_dim=1), seed=42).cuda()
    x = torch.randn(100, 25).cuda()
    out = layer(x)
    assert out.shape == (100, 36) and not torch.isnan(out).any()
    assert hasattr(layer.nodes[0], "forward_with_mapping")
    want = orc.dwn_layer_forward(x.cpu().numpy(), layer._mapping_indices.cpu().numpy(), stacked(layer, "luts"))
    assert np.array_equal(out.detach().cpu().numpy(), want[:, :, 0])
    # the fused layer call equals the per-node path on the gathered inputs (test_fused_kernels.py:98-156)
    mapped = layer.get_mapping(x)
    per_node = torch.cat([node(mapped[:, i, :]) for i, node in enumerate(layer.nodes)], dim=1)
    assert torch.equal(per_node, out)
    shared = layer.nodes[3].forward_with_mapping(x, layer.get_mapping_indices())
    assert shared.shape == (100, 36, 1)
    want = orc.dwn_layer_forward(x.cpu().numpy(), layer._mapping_indices.cpu().numpy(),
                                 np.repeat(stacked(layer, "luts")[3:4], 36, 0))
    assert np.array_equal(shared.detach().cpu().numpy(), want)


def test_gradient_flow_every_parameter():
    """test_fused_kernels.py:52-95: I=16, N=25, k=4, batch 10; every luts gets a non-zero gradient."""
    REGISTRY, NodeConfig, _, _ = _api()
    layer = REGISTRY.get_layer("random")(input_size=16, output_size=25, node_type=REGISTRY.get_node("dwn"),
                                         node_kwargs=NodeConfig(input_dim=4, output_dim=1), seed=42).cuda()
    x = torch.randn(10, 16, device="cuda", requires_grad=True)
    out = layer(x)
    assert out.shape == (10, 25)
    out.sum().backward()
    assert x.grad is not None and x.grad.abs().sum() > 0
    count = 0
    for name, p in layer.named_parameters():
        assert p.grad is not None and p.grad.abs().sum() > 0, name
        count += 1
    assert count == 25
    gx, gl = orc.dwn_layer_backward(x.detach().cpu().numpy(), layer._mapping_indices.cpu().numpy(),
                                    stacked(layer, "luts"), np.ones((10, 25, 1), np.float32),
                                    np.float32(0.5 * 0.75 ** 3), np.float32(1 / 3))
    np.testing.assert_allclose(x.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(torch.stack([n.luts.grad for n in layer.nodes]).cpu().numpy(), gl, rtol=1e-6)


@pytest.mark.parametrize("layer_name", ["random", "learnable"])
@pytest.mark.parametrize("node_name", ["dwn", "probabilistic"])
def test_layer_shape_range_grads_and_device_roundtrip(layer_name, node_name):
    """test_layer_functionality.py:37-123 (input 256, 128 nodes, k=4, batch 8) for every layer x node."""
    REGISTRY, NodeConfig, _, _ = _api()
    torch.manual_seed(42)
    kwargs = dict(input_size=256, output_size=128, node_type=REGISTRY.get_node(node_name),
                  node_kwargs=NodeConfig(input_dim=4, output_dim=1))
    cpu_layer = REGISTRY.get_layer(layer_name)(**kwargs)
    torch.manual_seed(42)
    layer = REGISTRY.get_layer(layer_name)(**kwargs).cuda()
    layer.load_state_dict(cpu_layer.state_dict())  # state built on the host loads into the device layer
    for k, v in cpu_layer.state_dict().items():
        assert torch.equal(v, layer.state_dict()[k].cpu()), k
    torch.manual_seed(42)
    x = torch.rand(8, 256, device="cuda", requires_grad=True)
    layer.train()
    out = layer(x)
    assert out.shape == (8, 128)
    out.sum().backward()
    for name, p in layer.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), name
    assert any(p.grad.abs().sum() > 0 for p in layer.parameters())
    layer.eval()
    for seed in (42, 123, 456):
        torch.manual_seed(seed)
        with torch.no_grad():
            e = layer(torch.rand(8, 256, device="cuda"))
        assert e.min() >= 0.0 and e.max() <= 1.0 and set(e.unique().tolist()) <= {0.0, 1.0}


def test_learnable_layer_train_and_eval_against_oracle():
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    torch.manual_seed(7)
    layer = REGISTRY.get_layer("learnable")(
        input_size=60, output_size=20, node_type=REGISTRY.get_node("dwn"),
        node_kwargs=NodeConfig(input_dim=3, output_dim=1, init_fn=uniform_init, init_kwargs={"a": -1.0, "b": 1.0}),
        tau=1.0, tau_start=1.0, tau_min=1e-4, tau_decay_iters=1000.0, use_cuda_soft=False).cuda()
    x = torch.rand(33, 60, device="cuda", requires_grad=True)
    W = layer.mapping.W.detach().cpu().numpy()
    luts = stacked(layer, "luts")
    ident = np.arange(60).reshape(20, 3)
    layer.train()
    out = layer(x)
    m = orc.soft_mapping_forward(x.detach().cpu().numpy(), W, 1.0)
    mt = layer.get_mapping(x)
    np.testing.assert_allclose(mt.detach().cpu().numpy().reshape(33, -1), m, rtol=1e-5, atol=1e-6)
    # node stage checked on the device's own mapped values (thresholding is discontinuous)
    want = orc.dwn_layer_forward(mt.detach().cpu().numpy().reshape(33, -1), ident, luts)[:, :, 0]
    assert np.array_equal(out.detach().cpu().numpy(), want)
    gy = torch.randn_like(out)
    out.backward(gy)
    gmap, gl = orc.dwn_layer_backward(mt.detach().cpu().numpy().reshape(33, -1), ident, luts,
                                      gy.cpu().numpy()[:, :, None], np.float32(0.5 * 0.75 ** 2), np.float32(1 / 3))
    gx, gW = orc.soft_mapping_backward(x.detach().cpu().numpy(), W, gmap, 1.0)
    np.testing.assert_allclose(x.grad.cpu().numpy(), gx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(layer.mapping.W.grad.cpu().numpy(), gW, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(torch.stack([n.luts.grad for n in layer.nodes]).cpu().numpy(), gl, rtol=1e-5, atol=1e-5)
    layer.eval()
    xb = torch.randint(0, 2, (12, 60), device="cuda").float()
    hm, sel = orc.hard_mapping(xb.cpu().numpy(), W)
    assert np.array_equal(layer.get_mapping_matrix().cpu().numpy(), sel.reshape(20, 3))
    want = np.stack([orc.dwn_eval_forward(hm[:, 3 * n:3 * n + 3], luts[n]) for n in range(20)], 1)[:, :, 0]
    assert np.array_equal(layer(xb).cpu().numpy(), want)


def test_residual_initialisation_known_answers():
    """tests/test_nodes/test_residual_initialization.py:56-232 for DWN and Probabilistic nodes."""
    REGISTRY, _, _, residual_init = _api()
    corners = torch.tensor(list(itertools.product([0, 1], repeat=6)), dtype=torch.float32, device="cuda")
    for name in ("dwn", "probabilistic"):
        node = REGISTRY.get_node(name)(input_dim=6, output_dim=1, init_fn=residual_init,
                                       init_kwargs={"node_type": name, "noise_factor": 0.0, "logit_clarity": 5.0,
                                                    "input_dim": 6}).cuda()
        node.eval()
        with torch.no_grad():
            assert torch.equal(node.forward_eval(corners).squeeze(), corners[:, 0])  # passes input 0 through
        if name == "probabilistic":
            node.train()
            with torch.no_grad():
                lo = node.forward_train(torch.zeros(50, 6, device="cuda")).mean().item()
                hi = node.forward_train(torch.ones(50, 6, device="cuda")).mean().item()
                a = torch.zeros(1, 6, device="cuda"); b = a.clone(); b[0, 1:] = 1.0
                diff = (node.forward_train(a) - node.forward_train(b)).abs().item()
            assert abs(lo - 1 / (1 + np.exp(5.0))) < 1e-5 and abs(hi - 1 / (1 + np.exp(-5.0))) < 1e-5 and diff < 1e-5
        assert node.export_bitstream() == [int(c[0]) for c in corners.cpu().tolist()]


def test_smallest_training_configuration_end_to_end(golden):
    """thermometer -> RandomLayer+DWN -> GroupSum -> cross-entropy against the reference's numbers."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.utils import GroupSum
    g = golden
    x = torch.tensor(g["e2e_x"]).cuda()
    enc = REGISTRY.build_encoder("thermometer", num_bits=4).fit(x)
    bits = enc.encode(x).requires_grad_()
    assert np.array_equal(bits.detach().cpu().numpy(), g["e2e_bits"])
    layer = REGISTRY.get_layer("random")(80, 30, REGISTRY.get_node("dwn"),
                                         NodeConfig(input_dim=6, output_dim=1, init_fn=uniform_init,
                                                    init_kwargs={"a": -1.0, "b": 1.0}), seed=42).cuda()
    assert np.array_equal(layer._mapping_indices.cpu().numpy(), g["e2e_idx"])
    with torch.no_grad():
        for n, node in enumerate(layer.nodes):
            node.luts.copy_(torch.tensor(g["e2e_luts"][n]))
    logits = GroupSum(k=10, tau=1.0, use_randperm=False)(layer(bits))
    np.testing.assert_allclose(logits.detach().cpu().numpy(), g["e2e_logits"], rtol=1e-6, atol=1e-6)
    loss = torch.nn.functional.cross_entropy(logits, torch.tensor(g["e2e_labels"]).cuda())
    assert loss.item() == pytest.approx(float(g["e2e_loss"]), rel=1e-6)
    loss.backward()
    np.testing.assert_allclose(bits.grad.cpu().numpy(), g["e2e_gbits"], rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(torch.stack([n.luts.grad for n in layer.nodes]).cpu().numpy(), g["e2e_gluts"],
                               rtol=1e-5, atol=1e-7)


def test_first_benchmark_configuration_full_size_against_oracle():
    """The reference's CPU-runnable configuration at its full size: U[0,1] inputs [256, 784] -> thermometer with 4
    thresholds -> 3136 bits -> RandomLayer(seed 42, k = 6) -> 2000 DWN nodes, tables U[-1,1] -> GroupSum into 10
    classes -> cross-entropy on random labels, one forward + backward.  Module by module and as one DWNStack
    (thermometer and GroupSum folded into the layer's kernels) against the oracle: bits, mapping table, layer output
    and logits bit-exact / to 1e-6, table gradients to rtol 1e-5."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum
    torch.manual_seed(0)
    B, F, NB, N, k, G = 256, 784, 4, 2000, 6, 10
    x = torch.rand(B, F)
    labels = torch.randint(0, G, (B,))
    thr = orc.thermometer_fit(x.numpy(), NB)
    bits = orc.thermometer_encode(x.numpy(), thr).reshape(B, F * NB).astype(np.float32)
    layer = REGISTRY.get_layer("random")(F * NB, N, REGISTRY.get_node("dwn"),
                                         NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init,
                                                    init_kwargs={"a": -1.0, "b": 1.0}), seed=42).cuda()
    idx = layer._mapping_indices.cpu().numpy().astype(np.int64)
    assert np.array_equal(idx, orc.random_mapping(F * NB, N, k, seed=42).numpy().astype(np.int64))
    luts = stacked(layer, "luts")
    alpha, beta = float(layer.nodes[0].alpha), float(layer.nodes[0].beta)
    # oracle: forward, logits, loss and the gradient that reaches the tables
    want_y = c_oracle.dwn_layer_forward(bits, idx, luts).reshape(B, N)
    want_logits = orc.group_sum(want_y, G, 1.0)
    lt = torch.tensor(want_logits, dtype=torch.float64, requires_grad=True)
    want_loss = torch.nn.functional.cross_entropy(lt, labels)
    want_loss.backward()
    g_y = np.repeat(lt.grad.numpy(), N // G, axis=1).astype(np.float32).reshape(B, N, 1)
    _, want_gl = c_oracle.dwn_layer_backward(bits, idx, luts, g_y, alpha, beta)
    # module by module
    xd = x.cuda()
    enc = REGISTRY.build_encoder("thermometer", num_bits=NB).fit(xd)
    got_bits = enc.encode(xd)
    assert np.array_equal(got_bits.cpu().numpy().reshape(B, -1), bits)
    y = layer(got_bits)
    assert np.array_equal(y.detach().cpu().numpy(), want_y)
    head = GroupSum(k=G, tau=1.0, use_randperm=False)
    logits = head(y)
    np.testing.assert_allclose(logits.detach().cpu().numpy(), want_logits, rtol=1e-6, atol=1e-5)  # sums of 200 values
    loss = torch.nn.functional.cross_entropy(logits, labels.cuda())
    assert loss.item() == pytest.approx(want_loss.item(), rel=1e-6)
    loss.backward()
    got_gl = torch.stack([n.luts.grad for n in layer.nodes]).cpu().numpy()
    np.testing.assert_allclose(got_gl, want_gl, rtol=1e-5, atol=1e-8)  # a bin holds ~4 terms of size ~1e-3
    # the same step as one chained call
    layer._banks["luts"].flat.grad = None
    for n in layer.nodes:
        n.luts.grad = None
    stack = DWNStack([layer], encoder=enc, head=head).train()
    logits2 = stack(xd)
    np.testing.assert_allclose(logits2.detach().cpu().numpy(), want_logits, rtol=1e-6, atol=1e-5)
    torch.nn.functional.cross_entropy(logits2, labels.cuda()).backward()
    np.testing.assert_allclose(layer._banks["luts"].flat.grad.cpu().numpy().reshape(want_gl.shape), want_gl,
                               rtol=1e-5, atol=1e-8)


def test_adam_steps_change_tables_in_place():
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    layer = REGISTRY.get_layer("random")(64, 40, REGISTRY.get_node("dwn"), NodeConfig(input_dim=6, output_dim=1),
                                         seed=1).cuda()
    opt = torch.optim.Adam(layer.parameters(), lr=0.01)
    before = stacked(layer, "luts").copy()
    x = torch.randint(0, 2, (128, 64), device="cuda").float()
    target = torch.rand(128, 40, device="cuda")
    losses = []
    for _ in range(5):
        opt.zero_grad()
        loss = ((layer(x) - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0] and not np.array_equal(before, stacked(layer, "luts"))
    assert layer._banks["luts"].tied()
    # one leaf per node parameter: same memory as the per-node views, one optimizer tensor
    (flat,) = layer.bank_parameters()
    assert flat.shape == (40, 1, 64) and flat.is_leaf and flat.requires_grad
    opt = torch.optim.Adam([flat], lr=0.01)
    before = stacked(layer, "luts").copy()
    opt.zero_grad()
    ((layer(x) - target) ** 2).mean().backward()
    assert torch.equal(flat.grad[3], layer.nodes[3].luts.grad)
    opt.step()
    assert not np.array_equal(before, stacked(layer, "luts"))
    assert np.array_equal(flat.detach().cpu().numpy(), stacked(layer, "luts"))


# ------------------------------------------------------------------------------ benchmark shape
def test_full_size_properties_dwn_k6_b4096_n8192():
    from difflut_amd import ops
    torch.manual_seed(0)
    B, I, N, k = 4096, 16384, 8192, 6
    x = torch.bernoulli(torch.full((B, I), 0.5, device="cuda"))
    idx = orc.random_mapping(I, N, k, seed=42)
    plan = ops.MappingPlan(idx.cuda(), I)
    luts = (torch.rand(N, 1, 64, device="cuda") * 2 - 1).requires_grad_()
    gy = torch.randn(B, N, device="cuda")
    alpha, beta = 0.5 * 0.75 ** 5, 1 / 3
    xg = x.clone().requires_grad_()
    y = ops.DWNLayerFunction.apply(xg, luts, plan, alpha, beta)
    y.backward(gy)
    gx1, gl1 = xg.grad.clone(), luts.grad.clone()
    # every output is one of the node's own table entries, and the lookup is deterministic
    lo, hi = luts.detach().amin(dim=(1, 2)), luts.detach().amax(dim=(1, 2))
    assert bool(((y.detach() >= lo) & (y.detach() <= hi)).all())
    y2 = ops.DWNLayerFunction.apply(x, luts.detach(), plan, alpha, beta)
    assert torch.equal(y.detach(), y2)
    # table gradient conserves the upstream gradient per node: sum_e gl[n,e] = sum_b gy[b,n]
    torch.testing.assert_close(gl1.sum(dim=(1, 2)), gy.sum(dim=0), rtol=1e-4, atol=2e-3)
    # backward is linear in gy; the input gradient is run-to-run identical (fixed summation order)
    xg2 = x.clone().requires_grad_(); l2 = luts.detach().clone().requires_grad_()
    ops.DWNLayerFunction.apply(xg2, l2, plan, alpha, beta).backward(2.0 * gy)
    assert torch.equal(xg2.grad, 2.0 * gx1)
    torch.testing.assert_close(l2.grad, 2.0 * gl1, rtol=1e-5, atol=1e-4)
    # first rows against the C restatement of the reference loops
    rows = 24
    xs, idn = x[:rows].cpu().numpy(), idx.numpy()
    ln = luts.detach().cpu().numpy()
    assert np.array_equal(y[:rows].detach().cpu().numpy(), c_oracle.dwn_layer_forward(xs, idn, ln)[:, :, 0])
    cgx, _ = c_oracle.dwn_layer_backward(xs, idn, ln, gy[:rows].cpu().numpy()[:, :, None], np.float32(alpha),
                                         np.float32(beta))
    np.testing.assert_allclose(gx1[:rows].cpu().numpy(), cgx, rtol=1e-5, atol=2e-6)
    # the table gradient is a histogram of gy by address: recompute it from the outputs' addresses
    addr = torch.zeros(B, N, dtype=torch.long, device="cuda")
    for j in range(k):
        addr |= (x[:, idx[:, j].long().cuda()] >= 0.5).long() << j
    want = torch.zeros(N, 64, device="cuda", dtype=torch.float64)
    want.scatter_add_(1, addr.t().contiguous(), gy.t().double().contiguous())
    torch.testing.assert_close(gl1[:, 0, :].double(), want, rtol=1e-5, atol=1e-4)


def test_full_size_probabilistic_k4_b1024_n4096():
    """The probabilistic benchmark shape against a float64 torch restatement of the same fold (the checker runs on
    the GPU; the first nodes also go through the numpy oracle)."""
    from difflut_amd import ops
    torch.manual_seed(1)
    B, I, N, k, T = 1024, 4096, 4096, 4, 1.0
    x = torch.sigmoid(torch.randn(B, I, device="cuda"))
    idx = orc.random_mapping(I, N, k, seed=42)
    plan = ops.MappingPlan(idx.cuda(), I)
    raw = torch.rand(N, 1 << k, 1, device="cuda")
    gy = torch.randn(B, N, device="cuda")
    xg = x.clone().requires_grad_(); wg = raw.clone().requires_grad_()
    y = ops.ProbLayerFunction.apply(xg, wg, plan, T)
    y.backward(gy)
    # float64 reference: multilinear interpolation of the sigmoid table, folded input by input
    xd = x.double().requires_grad_(); wd = raw.double().requires_grad_()
    m = xd[:, idx.long().cuda()]                                   # [B,N,k]
    v = torch.sigmoid(wd[:, :, 0] / T)[None].expand(B, N, 1 << k)
    for j in range(k):
        v = v[..., 0::2] + m[..., j:j + 1] * (v[..., 1::2] - v[..., 0::2])
    yd = v[..., 0]
    yd.backward(gy.double())
    torch.testing.assert_close(y.detach().double(), yd.detach(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(xg.grad.double(), xd.grad, rtol=1e-5, atol=2e-6)
    # a table gradient sums 1024 terms of size <= |gy| p_a sigmoid'(w) <= 0.25 |gy|
    torch.testing.assert_close(wg.grad.double(), wd.grad, rtol=1e-5, atol=2e-5)
    # first nodes through the numpy oracle as well
    n0 = 64
    want = orc.prob_layer_forward(x.cpu().numpy(), idx.numpy()[:n0], raw.cpu().numpy()[:n0], T, dtype=torch.float64)
    np.testing.assert_allclose(y.detach().cpu().numpy()[:, :n0], want[:, :, 0], rtol=1e-5, atol=1e-6)
    # deterministic: fixed summation orders everywhere
    xg2 = x.clone().requires_grad_(); wg2 = raw.clone().requires_grad_()
    ops.ProbLayerFunction.apply(xg2, wg2, plan, T).backward(gy)
    assert torch.equal(xg2.grad, xg.grad) and torch.equal(wg2.grad, wg.grad)


@pytest.mark.parametrize("precision", [0, 1])
def test_full_size_soft_mapping_b512_i3136_m48000(precision):
    """The soft-connectivity benchmark shape against float64 torch autograd of softmax + matmul (learnable_layer.py:254-255).
    fp32 operands: rtol 1e-4 on sums of 3136 .. 48000 terms; bf16 operands: 1e-2 of the tensor's largest value."""
    from difflut_amd import ops
    torch.manual_seed(2)
    B, I, M, tau = 512, 3136, 48000, 1.0
    x = torch.rand(B, I, device="cuda")
    W = torch.randn(M, I, device="cuda") * 0.01
    gm = torch.randn(B, M, device="cuda")
    xg = x.clone().requires_grad_(); Wg = W.clone().requires_grad_()
    m = ops.SoftMapFunction.apply(xg, Wg, tau, precision)
    m.backward(gm)
    xd = x.double().requires_grad_(); Wd = W.double().requires_grad_()
    md = xd @ torch.softmax(Wd / tau, dim=-1).t()
    md.backward(gm.double())
    if precision == 0:
        torch.testing.assert_close(m.detach().double(), md.detach(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(xg.grad.double(), xd.grad, rtol=1e-4, atol=2e-5 * float(xd.grad.abs().max()))
        torch.testing.assert_close(Wg.grad.double(), Wd.grad, rtol=1e-4, atol=2e-5 * float(Wd.grad.abs().max()))
    else:
        for got, want in ((m.detach(), md.detach()), (xg.grad, xd.grad), (Wg.grad, Wd.grad)):
            assert float((got.double() - want).abs().max()) <= 1e-2 * float(want.abs().max())


@pytest.mark.parametrize("shape", [((70, 50), [40, 33, 20], 6), ((130, 64), [128, 64], 4), ((64, 30), [25], 3),
                                   ((200, 96), [300, 150, 75, 10], 6),
                                   # wide hidden layer, ragged batch: the bit-sliced forward walks several tiles per block
                                   ((4100, 96), [16000, 300], 6)])
@pytest.mark.parametrize("input_grad", [True, False])
def test_dwn_stack_equals_layer_by_layer(shape, input_grad):
    """Chained execution (bit-planes forward, tile-major gradients backward) against the same layers
    called one after the other: outputs bit-exact, gradients to rtol 1e-5 (same kernels, same
    summation orders; only the layouts between the layers differ)."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.layers import DWNStack
    (B, I), widths, k = shape
    torch.manual_seed(sum(widths) + B)
    layers, width = [], I
    for li, n in enumerate(widths):
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init,
                                                              init_kwargs={"a": -1.0, "b": 2.0}), seed=li + 3).cuda())
        width = n
    x = torch.rand(B, I, device="cuda")
    gy = torch.randn(B, widths[-1], device="cuda")
    xa = x.clone().requires_grad_(input_grad)
    h = xa
    for layer in layers:
        h = layer(h)
    h.backward(gy)
    want_y = h.detach().clone()
    want_gl = [layer._banks["luts"].flat.grad.clone() for layer in layers]
    want_gx = xa.grad.clone() if input_grad else None
    for layer in layers:
        layer._banks["luts"].flat.grad = None
    stack = DWNStack(layers).train()
    xb = x.clone().requires_grad_(input_grad)
    y = stack(xb)
    assert torch.equal(y.detach(), want_y)
    y.backward(gy)
    # a bin of the table gradient sums about B / 2^k values of size ~1 and its blocks flush with atomics in any order:
    # the floor is a few fp32 ulps of that sum
    for layer, want in zip(layers, want_gl):
        torch.testing.assert_close(layer._banks["luts"].flat.grad, want, rtol=1e-5, atol=max(1e-6, 2.5e-9 * B))
    if input_grad:
        torch.testing.assert_close(xb.grad, want_gx, rtol=1e-5, atol=2e-6)
    # eval mode and non-chainable members fall back to the members' own forward
    stack.eval()
    he = x
    for layer in layers:
        layer.eval()
        he = layer(he)
    assert torch.equal(stack(x), he)


@pytest.mark.parametrize("case", [(130, 37, 4, [60, 20], 6), (64, 784, 4, [2000, 10], 6), (9, 5, 3, [7], 2),
                                  (300, 70, 1, [33, 40], 5), (65, 17, 9, [50], 4)])
def test_dwn_stack_with_thermometer_encoder(case):
    """The stack fed raw features through a fitted thermometer encoder (code written directly as
    bit-planes) against encode() followed by the layers one by one: outputs bit-exact, table
    gradients to rtol 1e-5; the planes themselves against the oracle's bits."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd import _native as nat
    from difflut_amd.layers import DWNStack
    B, F, nbits, widths, k = case
    torch.manual_seed(B + F)
    x = torch.rand(B, F, device="cuda")
    enc = REGISTRY.build_encoder("thermometer", num_bits=nbits).fit(x)
    layers, width = [], F * nbits
    for li, n in enumerate(widths):
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init,
                                                              init_kwargs={"a": -1.0, "b": 2.0}), seed=li + 9).cuda())
        width = n
    # the planes against the oracle: bit r of word (t, c) is bit c of row 64 t + r
    lib = nat.lib()
    planes = torch.zeros(lib.dl_dwn_planes_bytes(B, F * nbits) // 8, dtype=torch.int64, device="cuda")
    nat.check(lib.dl_thermometer_planes(x.data_ptr(), enc.thresholds.contiguous().data_ptr(), planes.data_ptr(), B, F, nbits,
                                        nat.stream()))
    bits = orc.thermometer_encode(x.cpu().numpy(), enc.thresholds.cpu().numpy()).reshape(B, F * nbits)
    BT = (B + 63) // 64
    padded = np.zeros((BT * 64, F * nbits), dtype=np.uint64)
    padded[:B] = bits.astype(np.uint64)
    want = (padded.reshape(BT, 64, -1) << np.arange(64, dtype=np.uint64)[None, :, None]).sum(1, dtype=np.uint64)
    got = planes.cpu().numpy().view(np.uint64)[:BT * F * nbits].reshape(BT, F * nbits)
    assert np.array_equal(got, want)
    gy = torch.randn(B, widths[-1], device="cuda")
    h = enc.encode(x)
    for layer in layers:
        h = layer(h)
    h.backward(gy)
    want_y = h.detach().clone()
    want_gl = [layer._banks["luts"].flat.grad.clone() for layer in layers]
    for layer in layers:
        layer._banks["luts"].flat.grad = None
    stack = DWNStack(layers, encoder=enc).train()
    y = stack(x)
    assert torch.equal(y.detach(), want_y)
    y.backward(gy)
    for layer, want_g in zip(layers, want_gl):
        torch.testing.assert_close(layer._banks["luts"].flat.grad, want_g, rtol=1e-5, atol=1e-6)
    stack.eval()
    he = enc.encode(x)
    for layer in layers:
        layer.eval()
        he = layer(he)
    assert torch.equal(stack(x), he)


def test_more_than_2_31_output_elements():
    """A layer whose output has more than 2^31 elements (131109 rows x 16400 nodes; about 30 GB of device memory in
    all): sampled rows of the forward and of the input gradient against the oracle, and the mass of every node's
    table gradient against the column sums of the upstream gradient.  Guards the 64-bit offsets."""
    from difflut_amd import ops
    B, I, N, k, O = 131072 + 37, 512, 16400, 6, 1
    assert B * N > 2 ** 31
    torch.manual_seed(0)
    x = torch.rand(B, I, device="cuda")
    idx = orc.random_mapping(I, N, k, seed=3)
    plan = ops.MappingPlan(idx.cuda(), I)
    luts = (torch.rand(N, O, 64, device="cuda") * 2 - 1).requires_grad_()
    xt = x.clone().requires_grad_()
    y = ops.DWNLayerFunction.apply(xt, luts, plan, 0.1, 1.0 / 3.0)
    rows = torch.tensor([0, 1, 63, 64, 65535, 65536, 131071, 131072, B - 1])
    idx_np, luts_np = idx.numpy().astype(np.int64), luts.detach().cpu().numpy()
    want = orc.dwn_layer_forward(x[rows].cpu().numpy(), idx_np, luts_np).reshape(len(rows), -1)
    assert np.array_equal(y[rows].detach().cpu().numpy(), want)
    gy = torch.randn(B, N, device="cuda")
    y.backward(gy)
    mass = luts.grad.double().sum(-1).view(-1)
    col = gy.double().sum(0)
    torch.testing.assert_close(mass, col, rtol=1e-4, atol=1e-4 * float(col.abs().max()))
    gxs, _ = orc.dwn_layer_backward(x[rows].cpu().numpy(), idx_np, luts_np, gy[rows].cpu().numpy().reshape(len(rows), N, 1),
                                    np.float32(0.1), np.float32(1.0 / 3.0))
    np.testing.assert_allclose(xt.grad[rows].cpu().numpy(), gxs, rtol=1e-5, atol=2e-5)  # ~190 terms per input


def test_full_size_deep_stack_b8192():
    """The deep-stack configuration at its full size (8192 x 784 -> thermometer 4 bits -> 16000/8000/4000/2000
    DWN k=6 nodes -> GroupSum 10 -> cross-entropy): the chained run against the layers one by one (logits and
    loss to rtol 1e-5, every table gradient to rtol 1e-5 with a floor of a few ulps of its scale), two chained
    runs bit-identical in the logits, conservation of each table's gradient mass, and eval mode chained ==
    eval mode layer by layer, bit for bit."""
    REGISTRY, NodeConfig, _, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum
    B, F, k = 8192, 784, 6
    widths = [16000, 8000, 4000, 2000]
    torch.manual_seed(0)
    x = torch.rand(B, F, device="cuda")
    labels = torch.randint(0, 10, (B,), device="cuda")
    enc = REGISTRY.build_encoder("thermometer", num_bits=4).fit(x)
    layers, width = [], F * 4
    for n in widths:
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=1), seed=42).cuda())
        width = n
    head = GroupSum(k=10, tau=1.0, use_randperm=False)
    h = enc.encode(x)
    for layer in layers:
        h = layer(h)
    logits = head(h)
    loss = torch.nn.functional.cross_entropy(logits, labels)
    loss.backward()
    want_gl = [layer._banks["luts"].flat.grad.clone() for layer in layers]
    for layer in layers:
        layer._banks["luts"].flat.grad = None
    stack = DWNStack(layers, encoder=enc, head=head).train()
    got = stack(x)
    torch.testing.assert_close(got.detach(), logits.detach(), rtol=1e-5, atol=1e-4)
    loss2 = torch.nn.functional.cross_entropy(got, labels)
    torch.testing.assert_close(loss2.detach(), loss.detach(), rtol=1e-5, atol=0)
    loss2.backward()
    for layer, want in zip(layers, want_gl):
        g = layer._banks["luts"].flat.grad
        torch.testing.assert_close(g, want, rtol=1e-5, atol=float(want.abs().max()) * 4e-6)
    assert torch.equal(stack(x).detach(), got.detach())
    # the last layer's table gradient: every node's bins add up to the sum of its output gradient over the batch
    p = torch.softmax(got.detach().double(), dim=1)
    p[torch.arange(B), labels] -= 1.0
    per_group = (p / B).sum(0)                                  # d loss / d logit, summed over the batch
    mass = layers[-1]._banks["luts"].flat.grad.double().view(widths[-1], -1).sum(1)
    torch.testing.assert_close(mass, per_group.repeat_interleave(widths[-1] // 10), rtol=1e-4, atol=1e-7)
    # inference
    stack.eval()
    he = enc.encode(x)
    for layer in layers:
        layer.eval()
        he = layer(he)
    assert torch.equal(stack(x), head(he))


@pytest.mark.parametrize("case", [(130, 37, [60, 640], 6, 10, 1.0), (64, 100, [2000], 6, 10, 2.5), (700, 50, [300, 768], 4, 3, 0.5),
                                  (65, 30, [90, 130], 5, 2, 1.0), (256, 64, [512], 6, 8, 1.0), (33, 40, [1000], 6, 7, 1.0),
                                  (100, 48, [70, 192], 4, 3, 1.0, 2),
                                  # the head's gradient expanded inside the chained gather (at most 16 groups, short lists):
                                  # inputs read three times, twice, unevenly; 16 groups; 20 groups (written out first)
                                  (200, 40, [1280, 640], 6, 10, 1.0), (130, 33, [1000, 500], 4, 5, 2.0), (70, 20, [704, 520], 5, 8, 1.0),
                                  (90, 20, [2048, 1024], 6, 16, 0.5), (90, 20, [2560, 1280], 6, 20, 1.0), (4100, 64, [1024, 512], 6, 8, 1.0)])
def test_dwn_stack_with_group_sum_head(case):
    """DWNStack(..., head=GroupSum): the last layer sums its columns per group itself.  Against the
    layers one by one followed by GroupSum: logits to rtol 1e-5 (fp32 sums in another order), and
    against the oracle's group_sum of the bit-exact layer output; table and input gradients to
    rtol 1e-5; two runs give identical bits (fixed summation order).  The last case has groups that
    do not divide the width and takes the unfused head."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum
    import warnings
    B, I, widths, k, groups, tau = case[:6]
    O = case[6] if len(case) > 6 else 1  # outputs per node: the last case has two, groups run over node-major columns
    torch.manual_seed(B + I + groups)
    layers, width = [], I
    for li, n in enumerate(widths):
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=O, init_fn=uniform_init,
                                                              init_kwargs={"a": -1.0, "b": 2.0}), seed=li + 21).cuda())
        width = n * O
    head = GroupSum(k=groups, tau=tau, use_randperm=False)
    x = torch.rand(B, I, device="cuda")
    glog = torch.randn(B, groups, device="cuda")
    xa = x.clone().requires_grad_()
    h = xa
    for layer in layers:
        h = layer(h)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        logits = head(h)
    logits.backward(glog)
    want_gl = [layer._banks["luts"].flat.grad.clone() for layer in layers]
    want_gx = xa.grad.clone()
    for layer in layers:
        layer._banks["luts"].flat.grad = None
    stack = DWNStack(layers, head=head).train()
    assert stack._fusable_head() == (widths[-1] * O % groups == 0)
    xb = x.clone().requires_grad_()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        got = stack(xb)
    assert got.shape == (B, groups)
    torch.testing.assert_close(got.detach(), logits.detach(), rtol=1e-5, atol=1e-5)
    want = orc.group_sum(h.detach().cpu().numpy(), groups, tau)
    np.testing.assert_allclose(got.detach().cpu().numpy(), want, rtol=1e-5, atol=1e-5)
    got.backward(glog)
    for layer, want_g in zip(layers, want_gl):  # bins are sums of up to B values of size ~1/tau with cancellation
        torch.testing.assert_close(layer._banks["luts"].flat.grad, want_g, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(xb.grad, want_gx, rtol=1e-5, atol=5e-6)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        again = stack(x)
    assert torch.equal(again, got.detach())
    # eval mode: members one by one, then the head
    stack.eval()
    he = x
    for layer in layers:
        layer.eval()
        he = layer(he)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        assert torch.equal(stack(x), head(he))


@pytest.mark.parametrize("case", [(130, 37, 4, [60, 640], 6, 10, 1), (64, 25, 4, [2000], 6, 10, 1), (700, 50, 1, [300, 768], 4, 3, 1),
                                  (65, 30, 3, [90, 130], 5, None, 1), (100, 12, 4, [70, 192], 4, 3, 2), (33, 40, 2, [1000], 6, 7, 1)])
def test_dwn_stack_eval_runs_chained_on_binary_input(case):
    """Eval mode of DWNStack behind a thermometer encoder (or on 0/1 input with binary_input=True): bit-planes
    between the layers, (table >= 0.5) outputs, GroupSum as a count.  Against the oracle's eval forward layer by
    layer (bit-exact 0/1 outputs; the group sums are integers divided by tau) and against the members run
    one by one."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum
    import warnings
    B, F, nbits, widths, k, groups, O = case
    torch.manual_seed(B * 3 + F)
    x = torch.rand(B, F, device="cuda")
    enc = REGISTRY.build_encoder("thermometer", num_bits=nbits).fit(x)
    layers, width = [], F * nbits
    for li, n in enumerate(widths):
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=O, init_fn=uniform_init,
                                                              init_kwargs={"a": 0.0, "b": 1.0}), seed=li + 31).cuda())
        width = n * O
    head = GroupSum(k=groups, tau=1.5, use_randperm=False) if groups else None
    # oracle: encode, then every layer's eval forward on the mapped bits
    h = orc.thermometer_encode(x.cpu().numpy(), enc.thresholds.cpu().numpy()).reshape(B, -1).astype(np.float32)
    for layer in layers:
        idx = layer._mapping_indices.cpu().numpy().astype(np.int64)
        luts = layer._banks["luts"].tensor().detach().cpu().numpy()
        h = np.stack([orc.dwn_eval_forward(h[:, idx[n]], luts[n]) for n in range(idx.shape[0])], axis=1).reshape(B, -1)
    want = h if head is None else orc.group_sum(h, groups, 1.5)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        stack = DWNStack(layers, encoder=enc, head=head).eval()
        got = stack(x)
        # the members one by one
        he = enc.encode(x)
        for layer in layers:
            layer.eval()
            he = layer(he)
        loop = he if head is None else head(he)
        # the same stack without the encoder, fed the code itself
        code = enc.encode(x)
        plain = DWNStack(layers, head=head, binary_input=True).eval()
        got_code = plain(code)
    assert not got.requires_grad
    if head is None:
        assert np.array_equal(got.cpu().numpy(), want)
    else:
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-6, atol=0)
    assert torch.equal(got, loop) and torch.equal(got_code, got)


def test_group_head_entry_points_reject_bad_arguments():
    """Error codes: -1 null pointer, -2 shape, -3 unsupported, -4 workspace too small."""
    from difflut_amd import _native as nat
    lib = nat.lib()
    one = torch.zeros(4096, device="cuda")
    p = one.data_ptr()
    args = (64, 32, 128, 6, 1)
    # groups narrower than 64 columns are not supported by the fused head
    assert lib.dl_dwn_layer_fwd_planes_groups(p, p, p, p, p, p, 1 << 20, *args, 4, 1.0, nat.stream()) == -3
    assert lib.dl_dwn_layer_fwd_planes_groups(p, p, p, p, p, p, 1 << 20, *args, 0, 1.0, nat.stream()) == -2
    assert lib.dl_dwn_layer_fwd_planes_groups(p, p, p, p, p, p, 1 << 20, *args, 2, 0.0, nat.stream()) == -2
    assert lib.dl_dwn_layer_fwd_planes_groups(p, p, p, p, p, p, 16, *args, 2, 1.0, nat.stream()) == -4
    assert lib.dl_dwn_layer_fwd_planes_groups(p, p, p, None, p, p, 1 << 20, *args, 2, 1.0, nat.stream()) == -1
    assert lib.dl_dwn_layer_bwd_groups(p, p, p, p, None, 2, 1.0, 0.1, 0.3, p, 0, p, p, 1 << 20, *args, nat.stream()) == -1
    assert lib.dl_dwn_layer_bwd_groups(p, p, p, p, p, 2, -1.0, 0.1, 0.3, p, 0, p, p, 1 << 20, *args, nat.stream()) == -2


def test_dwn_layer_step_replays_from_a_hip_graph():
    """The library never allocates or synchronises, and clears buffers with kernels, so a forward +
    backward can be captured once and replayed; every replay is checked against an eager run on
    the same inputs (eager work and synchronisations in between)."""
    from difflut_amd import ops
    torch.manual_seed(5)
    B, I, N, k = 192, 96, 80, 6
    idx = orc.random_mapping(I, N, k, seed=7)
    plan = ops.MappingPlan(idx.cuda(), I)
    alpha, beta = 0.5 * 0.75 ** 5, 1 / 3
    x = torch.rand(B, I, device="cuda").requires_grad_()
    luts = (torch.rand(N, 1, 64, device="cuda") * 2 - 1).requires_grad_()
    gy = torch.randn(B, N, device="cuda")

    def eager(xv, lv, gv):
        xa, la = xv.clone().requires_grad_(), lv.clone().requires_grad_()
        y = ops.DWNLayerFunction.apply(xa, la, plan, alpha, beta)
        y.backward(gv)
        return y.detach(), xa.grad, la.grad

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture
        for _ in range(2):
            y = ops.DWNLayerFunction.apply(x, luts, plan, alpha, beta)
            gxs, gls = torch.autograd.grad(y, (x, luts), gy)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = ops.DWNLayerFunction.apply(x, luts, plan, alpha, beta)
        gxs, gls = torch.autograd.grad(y, (x, luts), gy)
    for rep in range(3):
        with torch.no_grad():
            x.copy_(torch.rand(B, I, device="cuda"))
            luts.copy_(torch.rand(N, 1, 64, device="cuda") * 2 - 1)
            gy.copy_(torch.randn(B, N, device="cuda"))
        graph.replay()
        torch.cuda.synchronize()
        wy, wgx, wgl = eager(x.detach(), luts.detach(), gy)
        assert torch.equal(y, wy) and torch.equal(gxs, wgx)
        torch.testing.assert_close(gls, wgl, rtol=1e-5, atol=1e-6)  # float atomics: order may differ


def test_training_stack_step_replays_from_a_hip_graph():
    """Forward + backward of a chained stack (thermometer planes in, GroupSum head out) captured once and replayed on
    new inputs and upstream gradients; logits bit-equal to eager, table gradients to rtol 1e-5 (atomic adds)."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum
    torch.manual_seed(13)
    B, F = 300, 40
    xs = [torch.rand(B, F, device="cuda") for _ in range(3)]
    gs = [torch.randn(B, 4, device="cuda") for _ in range(3)]
    enc = REGISTRY.build_encoder("thermometer", num_bits=2).fit(xs[0])
    layers, width = [], F * 2
    for li, n in enumerate([120, 240, 256]):
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=6, output_dim=1, init_fn=uniform_init,
                                                              init_kwargs={"a": -1.0, "b": 2.0}), seed=li + 51).cuda())
        width = n
    stack = DWNStack(layers, encoder=enc, head=GroupSum(k=4, tau=2.0, use_randperm=False)).train()
    banks = [layer._banks["luts"].flat for layer in layers]
    static_x, static_g = xs[0].clone(), gs[0].clone()

    def step(x, g):
        out = stack(x)
        grads = torch.autograd.grad(out, banks, g)
        return out.detach(), grads

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(static_x, static_g)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_c, grads_c = step(static_x, static_g)
    for i, (x, g) in enumerate(zip(xs, gs)):
        static_x.copy_(x)
        static_g.copy_(g)
        graph.replay()
        torch.cuda.synchronize()
        want_out, want_grads = step(x, g)
        torch.cuda.synchronize()
        assert torch.equal(out_c, want_out), f"replay {i}"
        for got, want in zip(grads_c, want_grads):
            torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def test_inference_stack_replays_from_a_hip_graph():
    """Chained inference (thermometer planes -> eval lookups -> GroupSum count) and a single layer's eval forward
    (device-side check of its input, both kernels launched) captured once and replayed on new inputs, with
    eager runs and synchronisations in between; every replay equals the eager result."""
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum
    torch.manual_seed(11)
    B, F = 200, 30
    xs = [torch.rand(B, F, device="cuda") for _ in range(4)]
    enc = REGISTRY.build_encoder("thermometer", num_bits=3).fit(xs[0])
    layers, width = [], F * 3
    for li, n in enumerate([150, 128]):
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=6, output_dim=1, init_fn=uniform_init,
                                                              init_kwargs={"a": 0.0, "b": 1.0}), seed=li + 41).cuda())
        width = n
    stack = DWNStack(layers, encoder=enc, head=GroupSum(k=2, tau=1.0, use_randperm=False)).eval()
    single = layers[0].eval()
    static_x = xs[0].clone()
    static_bits = enc.encode(xs[0]).clone()
    static_bits[0, 0] = 0.5                      # not binary: the generic kernel must answer for this input
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        for _ in range(2):
            stack(static_x)
            single(static_bits)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        out_stack = stack(static_x)
        out_single = single(static_bits)
    for i, x in enumerate(xs):
        bits = enc.encode(x)
        if i % 2 == 0:
            bits[0, 0] = 0.5
        static_x.copy_(x)
        static_bits.copy_(bits)
        graph.replay()
        torch.cuda.synchronize()
        with torch.no_grad():
            want_stack = stack(x)
            want_single = single(bits)
        torch.cuda.synchronize()
        assert torch.equal(out_stack, want_stack), f"replay {i}: stack"
        assert torch.equal(out_single, want_single), f"replay {i}: single layer ({'mixed' if i % 2 == 0 else 'binary'} input)"


def test_legacy_extension_names_and_signatures(golden):
    """tests/test_layers/test_fused_kernels.py:159-179 imports efd_cuda / efd_fused_cuda by bare name;
    the shims answer with the reference's signatures."""
    import difflut_amd.compat as compat
    compat.install()
    import efd_cuda
    import efd_fused_cuda
    import learnable_mapping_cuda
    import mapping_cuda
    import probabilistic_cuda

    g = golden
    dev = "cuda"
    x = torch.tensor(g["dwn_k6o2_x"], device=dev); luts = torch.tensor(g["dwn_k6o2_luts"], device=dev)
    gy = torch.tensor(g["dwn_k6o2_gy"], device=dev)
    a, b = (float(v) for v in g["dwn_k6o2_ab"])
    assert np.array_equal(efd_cuda.forward(x, luts).cpu().numpy(), g["dwn_k6o2_y"])
    gx, gl = efd_cuda.backward(x, luts, gy, a, b)
    np.testing.assert_allclose(gx.cpu().numpy(), g["dwn_k6o2_gx"], rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(gl.cpu().numpy(), g["dwn_k6o2_gl"], rtol=1e-5, atol=1e-6)
    rng = np.random.default_rng(0)
    xin = torch.tensor(rng.random((50, 30)).astype(np.float32), device=dev)
    mapping = orc.random_mapping(30, 12, 4, seed=3).to(dev).long()
    l3 = torch.tensor(rng.uniform(-1, 1, (12, 2, 16)).astype(np.float32), device=dev)
    y = efd_fused_cuda.forward(xin, mapping, l3)
    assert y.shape == (50, 12, 2)
    assert np.array_equal(y.cpu().numpy(), orc.dwn_layer_forward(xin.cpu().numpy(), mapping.cpu().numpy(), l3.cpu().numpy()))
    m = mapping_cuda.forward(xin, mapping.to(torch.int16))
    assert np.array_equal(m.cpu().numpy(), orc.gather_forward(xin.cpu().numpy(), mapping.cpu().numpy()))
    gm = torch.randn_like(m)
    np.testing.assert_allclose(mapping_cuda.backward(gm, mapping.to(torch.int16), 30).cpu().numpy(),
                               orc.gather_backward(gm.cpu().numpy(), mapping.cpu().numpy(), 30), rtol=1e-6, atol=1e-6)
    T = torch.tensor(float(g["prob_k4o2_T"][0]), device=dev)
    px = torch.tensor(g["prob_k4o2_x"], device=dev); pw = torch.tensor(g["prob_k4o2_w"], device=dev)
    np.testing.assert_allclose(probabilistic_cuda.forward(px, pw, T).cpu().numpy(), g["prob_k4o2_y"], rtol=1e-5, atol=1e-6)
    pgx, pgw = probabilistic_cuda.backward(px, pw, T, torch.tensor(g["prob_k4o2_gy"], device=dev))
    np.testing.assert_allclose(pgx.cpu().numpy(), g["prob_k4o2_gx"], rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(pgw.cpu().numpy(), g["prob_k4o2_gw"], rtol=1e-5, atol=2e-6)
    sx = torch.tensor(g["soft_x"], device=dev); sW = torch.tensor(g["soft_W"], device=dev)
    np.testing.assert_allclose(learnable_mapping_cuda.soft_forward(sx, sW, 1.0).cpu().numpy(), g["soft_m"].reshape(5, -1),
                               rtol=1e-5, atol=1e-6)
    sel = torch.tensor(g["hard_idx"].reshape(-1), device=dev, dtype=torch.int32)
    assert np.array_equal(learnable_mapping_cuda.forward(sx, sel).cpu().numpy(), g["hard_m"].reshape(5, -1))
