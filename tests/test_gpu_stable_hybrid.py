"""GPU parity of the gradient-stabilised DWN node and the hybrid node against the CPU oracle, through the
C ABI (ops) and through the layer / node classes.  Lookups must be bit-exact given the table; sums of
floating-point terms are held to rtol 1e-5 with an absolute floor of a few fp32 ulps of the operand scale."""
import itertools
import warnings

import numpy as np
import pytest
import torch

from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _ops():
    from difflut_amd import ops
    return ops


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to(DEV, dtype)


def make_case(seed, B, I, N, k, O, interior=False):
    rng = np.random.default_rng(seed)
    x = rng.random((B, I)).astype(np.float32)
    if interior:
        x = (0.02 + 0.96 * x).astype(np.float32)
    idx = orc.random_mapping(I, N, k, seed=seed + 1).numpy().astype(np.int64)
    raw = rng.standard_normal((N, O, 1 << k)).astype(np.float32)
    gy = rng.standard_normal((B, N, O)).astype(np.float32)
    scale = (0.5 + rng.random(N)).astype(np.float32)
    return x, idx, raw, gy, scale


SHAPES = [  # (B, I, N, k, O)
    (100, 25, 36, 6, 1),   # shapes of the reference's fused-kernel tests (tests/test_layers/test_fused_kernels.py:26-72)
    (10, 16, 25, 4, 1),
    (8, 256, 128, 4, 1),
    (70, 40, 33, 3, 2),
    (130, 300, 77, 5, 3),
    (1, 7, 5, 1, 1),
    (65, 9, 300, 2, 1),
    (200, 1030, 515, 6, 2),
    (9, 30, 11, 7, 2),     # k > 6: generic kernels
]


def test_table_sigmoid_forward_backward():
    ops = _ops()
    rng = np.random.default_rng(0)
    raw = (rng.standard_normal((37, 2, 64)) * 4).astype(np.float32)
    g = rng.standard_normal(raw.shape).astype(np.float32)
    rt = dev(raw).requires_grad_()
    luts = ops.TableSigmoidFunction.apply(rt)
    want = orc.table_sigmoid(raw)
    np.testing.assert_allclose(luts.detach().cpu().numpy(), want, rtol=3e-7, atol=1e-9)  # 2 ulp of expf + divide
    luts.backward(dev(g))
    # like torch's sigmoid backward the adjoint is g * y * (1 - y) on the fp32 y: near saturation 1 - y
    # carries half an ulp of 1 (6e-8) absolute, so the floor is |g| * 6e-8 ~ 3e-7
    np.testing.assert_allclose(rt.grad.cpu().numpy(), g * want * (1 - want), rtol=1e-5, atol=3e-7)


@pytest.mark.parametrize("shape", SHAPES)
def test_stable_layer_forward_backward(shape):
    B, I, N, k, O = shape
    ops = _ops()
    x, idx, raw, gy, scale = make_case(sum(shape), *shape)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_()
    rt = dev(raw).requires_grad_()
    luts = ops.TableSigmoidFunction.apply(rt)
    y = ops.DWNStableLayerFunction.apply(xt, luts, dev(scale), plan)
    # the lookup itself is exact: every output is the table entry the oracle addresses
    want = orc.dwn_layer_forward(x, idx, luts.detach().cpu().numpy()).reshape(B, N * O)
    assert np.array_equal(y.detach().cpu().numpy(), want)
    y.backward(dev(gy.reshape(B, N * O)))
    gx, graw = orc.stable_layer_backward(x, idx, raw, gy, scale)
    # gx sums fan-in * O terms of size scale*|gy|*|D| ~ 1: rtol 1e-5, floor 2e-6
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(rt.grad.cpu().numpy(), graw, rtol=1e-5, atol=2e-6)


def test_stable_no_input_grad_and_scalar_scale():
    ops = _ops()
    shape = (40, 50, 3, 2, 1)
    B, I, N, k, O = shape
    x, idx, raw, gy, _ = make_case(4, *shape)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    rt = dev(raw).requires_grad_()
    y = ops.DWNStableLayerFunction.apply(dev(x), ops.TableSigmoidFunction.apply(rt), torch.full((N,), 1.25, device=DEV), plan)
    y.backward(dev(gy.reshape(B, -1)))
    _, graw = orc.stable_layer_backward(x, idx, raw, gy, 1.25)
    np.testing.assert_allclose(rt.grad.cpu().numpy(), graw, rtol=1e-5, atol=2e-6)
    with pytest.raises(RuntimeError):
        ops.DWNStableLayerFunction.apply(dev(x), dev(orc.table_sigmoid(raw)), torch.ones(N + 1, device=DEV), plan)


@pytest.mark.parametrize("shape", SHAPES)
def test_hybrid_layer_forward_backward(shape):
    B, I, N, k, O = shape
    ops = _ops()
    x, idx, raw, gy, _ = make_case(sum(shape) + 1, *shape, interior=True)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_()
    rt = dev(raw).requires_grad_()
    luts = ops.TableSigmoidFunction.apply(rt)
    y = ops.HybridLayerFunction.apply(xt, luts, plan)
    want = orc.dwn_layer_forward(x, idx, luts.detach().cpu().numpy()).reshape(B, N * O)
    assert np.array_equal(y.detach().cpu().numpy(), want)
    y.backward(dev(gy.reshape(B, N * O)))
    gx, graw = orc.hybrid_layer_backward(x, idx, raw, gy)
    # terms are |gy| * |table| * product weights <= 1 in size: rtol 1e-5, floor 2e-6
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(rt.grad.cpu().numpy(), graw, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("shape", [(66, 20, 30, 4, 1), (12, 30, 8, 7, 1)])
def test_hybrid_binary_inputs_get_zero_gradient(shape):
    """x_j (1 - x_j) = 0 at a binary input, so the reference's factor (a_j - x_j) / (x_j (1 - x_j) + 1e-8)
    multiplies a weight that is itself zero: the input gradient is exactly 0 there."""
    B, I, N, k, O = shape
    ops = _ops()
    x, idx, raw, gy, _ = make_case(21, *shape)
    x = (x >= 0.5).astype(np.float32)
    x[:, 3] = 0.3  # one real-valued input among the binary ones keeps its gradient
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_()
    rt = dev(raw).requires_grad_()
    ops.HybridLayerFunction.apply(xt, ops.TableSigmoidFunction.apply(rt), plan).backward(dev(gy.reshape(B, -1)))
    gx, graw = orc.hybrid_layer_backward(x, idx, raw, gy)
    got = xt.grad.cpu().numpy()
    assert np.all(np.delete(got, 3, axis=1) == 0.0)
    np.testing.assert_allclose(got, gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(rt.grad.cpu().numpy(), graw, rtol=1e-5, atol=2e-6)


# ------------------------------------------------------------------------------ node and layer classes
def _api():
    from difflut_amd.nodes import NodeConfig
    from difflut_amd.nodes.utils import residual_init, uniform_init
    from difflut_amd.registry import REGISTRY
    return REGISTRY, NodeConfig, uniform_init, residual_init


@pytest.mark.parametrize("name", ["dwn_stable", "hybrid"])
def test_node_alone_matches_oracle(name):
    """A node called on its own, with the signature of the reference's node classes."""
    REGISTRY, _, _, _ = _api()
    torch.manual_seed(3)
    kw = {"gradient_scale": 1.6} if name == "dwn_stable" else {}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        node = REGISTRY.get_node(name)(input_dim=5, output_dim=2, **kw).to(DEV)
    node.train()
    rng = np.random.default_rng(2)
    x = (0.02 + 0.96 * rng.random((50, 5))).astype(np.float32)
    gy = rng.standard_normal((50, 2)).astype(np.float32)
    xt = dev(x).requires_grad_()
    y = node(xt)
    raw = node.raw_luts.detach().cpu().numpy()
    luts = node._get_luts().detach().cpu().numpy()
    assert np.array_equal(y.detach().cpu().numpy(), orc.dwn_forward(x, luts))
    y.backward(dev(gy))
    idx = np.arange(5)[None]
    if name == "dwn_stable":
        gx, graw = orc.stable_layer_backward(x, idx, raw[None], gy[:, None, :], 1.6)
        assert node.gradient_scale.grad is None  # the scale is a Parameter that never gets a gradient
    else:
        gx, graw = orc.hybrid_layer_backward(x, idx, raw[None], gy[:, None, :])
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(node.raw_luts.grad.cpu().numpy(), graw[0], rtol=1e-5, atol=2e-6)
    node.eval()
    xb = dev((x >= 0.5).astype(np.float32))
    assert np.array_equal(node(xb).cpu().numpy(), orc.dwn_eval_forward(xb.cpu().numpy(), luts))


@pytest.mark.parametrize("name", ["dwn_stable", "hybrid"])
def test_residual_initialisation_known_answers(name):
    """tests/test_nodes/test_residual_initialization.py:42-173 for the two node types: with
    noise_factor = 0 the node passes its first input through, in eval mode exactly and in training
    mode as sigmoid(+-logit_clarity)."""
    REGISTRY, _, _, residual_init = _api()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        node = REGISTRY.get_node(name)(input_dim=6, output_dim=1, init_fn=residual_init,
                                       init_kwargs={"node_type": name, "noise_factor": 0.0, "logit_clarity": 5.0,
                                                    "input_dim": 6}).to(DEV)
    corners = torch.tensor(list(itertools.product([0, 1], repeat=6)), dtype=torch.float32, device=DEV)
    node.eval()
    with torch.no_grad():
        assert torch.equal(node.forward_eval(corners).squeeze(), corners[:, 0])
    node.train()
    with torch.no_grad():
        out = node.forward_train(corners).squeeze()
    assert torch.all((out > 0.5) == (corners[:, 0] > 0.5))
    for first in (0.0, 1.0):  # the output depends on the first input only
        assert out[corners[:, 0] == first].std().item() < 1e-6


@pytest.mark.parametrize("name", ["dwn_stable", "hybrid"])
def test_random_layer_fused_equals_oracle_and_state_dict_roundtrip(name):
    REGISTRY, NodeConfig, uniform_init, _ = _api()
    torch.manual_seed(11)
    B, I, N, k = 96, 64, 48, 4
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        cfg = NodeConfig(input_dim=k, output_dim=1, init_fn=uniform_init, init_kwargs={"a": -2.0, "b": 2.0})
        layer = REGISTRY.get_layer("random")(I, N, REGISTRY.get_node(name), cfg, seed=5).to(DEV)
        clone = REGISTRY.get_layer("random")(I, N, REGISTRY.get_node(name), cfg, seed=5).to(DEV)
    assert layer._fused == name
    layer.train()
    rng = np.random.default_rng(12)
    x = (0.02 + 0.96 * rng.random((B, I))).astype(np.float32)
    gy = rng.standard_normal((B, N)).astype(np.float32)
    xt = dev(x).requires_grad_()
    y = layer(xt)
    assert y.shape == (B, N)
    y.backward(dev(gy))
    idx = layer._mapping_indices.cpu().numpy().astype(np.int64)
    raw = np.stack([n.raw_luts.detach().cpu().numpy() for n in layer.nodes])
    if name == "dwn_stable":
        gx, graw = orc.stable_layer_backward(x, idx, raw, gy[:, :, None], 1.25)  # the constructor's default scale
    else:
        gx, graw = orc.hybrid_layer_backward(x, idx, raw, gy[:, :, None])
    luts = orc.table_sigmoid(raw).astype(np.float32)
    np.testing.assert_allclose(y.detach().cpu().numpy(), orc.dwn_layer_forward(x, idx, luts)[:, :, 0], rtol=3e-7)
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    for n in (0, 17, N - 1):  # per-node parameters see their row of the fused gradient
        np.testing.assert_allclose(layer.nodes[n].raw_luts.grad.cpu().numpy(), graw[n], rtol=1e-5, atol=2e-6)
    assert all(p.grad is not None for p in layer.bank_parameters() if p.dim() == 3)
    # state dict keys are the reference's per-node names
    keys = set(layer.state_dict().keys())
    assert "nodes.0.raw_luts" in keys and f"nodes.{N - 1}.raw_luts" in keys and "_mapping_indices" in keys
    assert ("nodes.0.gradient_scale" in keys) == (name == "dwn_stable")
    assert ("nodes.0.binary_combinations" in keys) == (name == "hybrid")
    clone.load_state_dict(layer.state_dict())
    clone.eval(); layer.eval()
    xb = dev((x >= 0.5).astype(np.float32))
    with torch.no_grad():
        assert torch.equal(clone(xb), layer(xb))
        m = orc.gather_forward(xb.cpu().numpy(), idx)
        want = np.stack([orc.dwn_eval_forward(m[:, n], luts[n])[:, 0] for n in range(N)], 1)
        assert np.array_equal(layer(xb).cpu().numpy(), want)


def test_legacy_extension_names_and_signatures():
    """dwn_stable_cuda / hybrid_cuda by bare name with the reference's call signatures
    (nodes/cuda/dwn_stable_cuda.cpp:19-43, hybrid_cuda.cpp:19-44): post-sigmoid tables, a float scale."""
    import difflut_amd.compat as compat
    compat.install()
    import dwn_stable_cuda
    import hybrid_cuda

    rng = np.random.default_rng(31)
    x = (0.02 + 0.96 * rng.random((40, 6))).astype(np.float32)
    luts = rng.random((2, 64)).astype(np.float32)
    gy = rng.standard_normal((40, 2)).astype(np.float32)
    xt, lt, gt = dev(x), dev(luts), dev(gy)
    want_y = orc.dwn_forward(x, luts)
    assert np.array_equal(dwn_stable_cuda.forward(xt, lt).cpu().numpy(), want_y)
    assert np.array_equal(hybrid_cuda.forward(xt, lt).cpu().numpy(), want_y)
    gx, gl = dwn_stable_cuda.backward(xt, lt, gt, 1.25)
    wx, wl = orc.stable_backward(x, luts, gy, 1.25)
    np.testing.assert_allclose(gx.cpu().numpy(), wx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(gl.cpu().numpy(), wl, rtol=1e-5, atol=2e-6)
    combos = torch.tensor([[(a >> j) & 1 for j in range(6)] for a in range(64)], dtype=torch.float32, device=DEV)
    gx, gl = hybrid_cuda.backward(xt, lt, combos, gt)
    wx, wl = orc.hybrid_backward(x, luts, gy)
    np.testing.assert_allclose(gx.cpu().numpy(), wx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(gl.cpu().numpy(), wl, rtol=1e-5, atol=2e-6)
    with pytest.raises(RuntimeError):
        hybrid_cuda.backward(xt.cpu(), lt, combos, gt)


def test_full_size_properties_stable_and_hybrid_k6_b4096_n8192():
    """The headline layer shape with the two node types, through size-independent properties:
    exact lookups, histogram mass (table gradients of a node sum to scale * sum of gy, resp. sum of gy
    because the product weights sum to one), linearity in gy, and zero input gradient for a constant table."""
    ops = _ops()
    B, I, N, k = 4096, 16384, 8192, 6
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.rand((B, I), generator=g).to(DEV)
    idx = orc.random_mapping(I, N, k, seed=42).to(DEV, torch.int32)
    plan = ops.MappingPlan(idx, I)
    raw = torch.randn((N, 1, 64), generator=g).to(DEV)
    gy = torch.randn((B, N), generator=g).to(DEV)
    scale = torch.full((N,), 1.25, device=DEV)
    luts = ops.TableSigmoidFunction.apply(raw)
    addr = ((x[:, idx.long()] >= 0.5).long() << torch.arange(k, device=DEV)).sum(-1)  # [B,N]
    want_y = torch.gather(luts[:, 0, :].T, 0, addr)
    for kind in ("stable", "hybrid"):
        def run(table, grad):
            xt = x.clone().requires_grad_()
            tt = table.clone().requires_grad_()
            if kind == "stable":
                y = ops.DWNStableLayerFunction.apply(xt, tt, scale, plan)
            else:
                y = ops.HybridLayerFunction.apply(xt, tt, plan)
            y.backward(grad)
            return y.detach(), xt.grad, tt.grad
        y, gx, gl = run(luts, gy)
        assert torch.equal(y, want_y)
        mass = gy.double().sum(0) * (1.25 if kind == "stable" else 1.0)
        torch.testing.assert_close(gl[:, 0, :].double().sum(1), mass, rtol=1e-5, atol=2e-4)
        _, gx2, gl2 = run(luts, 2.0 * gy)
        assert torch.equal(gx2, 2.0 * gx)  # scaling by two is exact in fp32 and gx is summed in a fixed order
        torch.testing.assert_close(gl2, 2.0 * gl, rtol=1e-5, atol=1e-4)  # bins are flushed with atomics
        _, gx0, _ = run(torch.full_like(luts, 0.3), gy)
        assert gx0.abs().max().item() <= 2e-5  # constant table: every difference vanishes
        assert torch.isfinite(gx).all() and gx.abs().max().item() > 0


@pytest.mark.parametrize("kind", ["stable", "dwn two outputs per node"])
def test_backward_in_chunks_of_rows_equals_the_halves(kind):
    """From about 6000 rows on the backward of a big layer runs chunk after chunk of rows inside one call.  Against the
    two half batches on their own (too small for chunks): the input gradient is the same rows bit for bit (a row's
    sums do not depend on the rows around it), the table gradient the sum of the two (other grouping of the same
    terms: rtol 1e-5).  The stabilised node (its scale enters where the chunks' partial sums are added, once) and a
    DWN layer with two outputs per node (columns are not nodes)."""
    ops = _ops()
    B, k = 8200, 6
    I, N, O = (16384, 8192, 1) if kind == "stable" else (8192, 4096, 2)
    g = torch.Generator(device="cpu").manual_seed(3)
    x = torch.rand((B, I), generator=g).to(DEV)
    idx = orc.random_mapping(I, N, k, seed=11).to(DEV, torch.int32)
    plan = ops.MappingPlan(idx, I)
    luts = (torch.rand((N, O, 64), generator=g) * 2 - 1).to(DEV)
    gy = torch.randn((B, N * O), generator=g).to(DEV)
    scale = (torch.rand((N,), generator=g) + 0.5).to(DEV)

    def run(rows):
        xt = x[rows].clone().requires_grad_()
        tt = luts.clone().requires_grad_()
        if kind == "stable":
            y = ops.DWNStableLayerFunction.apply(xt, tt, scale, plan)
        else:
            y = ops.DWNLayerFunction.apply(xt, tt, plan, 0.1, 1.0 / 3.0)
        y.backward(gy[rows])
        return xt.grad, tt.grad

    gx, gl = run(slice(0, B))
    half = 4096  # a multiple of 64: the halves' batch tiles are the whole batch's
    gx_a, gl_a = run(slice(0, half))
    gx_b, gl_b = run(slice(half, B))
    assert torch.equal(gx[:half], gx_a) and torch.equal(gx[half:], gx_b)
    torch.testing.assert_close(gl, gl_a + gl_b, rtol=1e-5, atol=2e-5 * float(gl.abs().max()))


@pytest.mark.parametrize("name,kind", [("dwn_stable", "stable"), ("hybrid", "hybrid")])
@pytest.mark.parametrize("tag", ["k6o1", "k3o2"])
def test_nodes_against_reference_vectors(golden_next, name, kind, tag):
    """Same inputs the reference's own CPU path was run on (tests/golden): training output, gradients down to
    the raw tables, eval output."""
    REGISTRY, _, _, _ = _api()
    g = golden_next
    raw = g[f"{kind}_{tag}_raw"]
    O, L = raw.shape
    kw = {"gradient_scale": 1.6} if kind == "stable" else {}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        node = REGISTRY.get_node(name)(input_dim=L.bit_length() - 1, output_dim=O, **kw)
    with torch.no_grad():
        node.raw_luts.copy_(torch.tensor(raw))
    node = node.to(DEV).train()
    xt = dev(g[f"{kind}_{tag}_x"]).requires_grad_()
    y = node(xt)
    np.testing.assert_allclose(y.detach().cpu().numpy(), g[f"{kind}_{tag}_y"], rtol=3e-7, atol=1e-8)  # sigmoid: 2 ulp
    y.backward(dev(g[f"{kind}_{tag}_gy"]))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), g[f"{kind}_{tag}_gx"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(node.raw_luts.grad.cpu().numpy(), g[f"{kind}_{tag}_graw"], rtol=2e-5, atol=2e-6)
    node.eval()
    with torch.no_grad():
        assert np.array_equal(node(dev(g[f"{kind}_{tag}_eval_x"])).cpu().numpy(), g[f"{kind}_{tag}_eval_y"])
