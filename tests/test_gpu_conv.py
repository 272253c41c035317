"""GPU parity of the convolutional LUT layer (all trees of a depth level as one block-diagonal layer call)
against the CPU oracle's chunk / tree loops over the same tables and index tables."""
import warnings

import numpy as np
import pytest
import torch

from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _build(node_name, depth, in_ch, out_ch, rf, stride, padding, chunk, n=6, grouped=False, seed=42, **node_kw):
    from difflut_amd import REGISTRY
    from difflut_amd.layers import ConvolutionConfig
    from difflut_amd.nodes import NodeConfig
    from difflut_amd.nodes.utils import uniform_init
    cfg = ConvolutionConfig(tree_depth=depth, in_channels=in_ch, out_channels=out_ch, receptive_field=rf, stride=stride,
                            padding=padding, chunk_size=chunk, seed=seed)
    lo, hi = (-1.0, 2.0) if node_name == "dwn" else (-2.0, 2.0)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        node_cfg = NodeConfig(input_dim=n, output_dim=1, init_fn=uniform_init, init_kwargs={"a": lo, "b": hi}, **node_kw)
        layer = REGISTRY.get_convolutional_layer("convolutional")(
            convolution_config=cfg, node_type=REGISTRY.get_node(node_name), node_kwargs=node_cfg,
            layer_type=REGISTRY.get_layer("random"), n_inputs_per_node=n, grouped_connections=grouped,
            ensure_full_coverage=grouped)
    return layer.to(DEV)


def _tables(layer, pname):
    """(chunks, trees) as the oracle wants them: [(idx, tables)] and per tree [(idx, tables)]."""
    def one(sub):
        idx = sub._mapping_indices.cpu().numpy().astype(np.int64)
        tab = np.stack([getattr(node, pname).detach().cpu().numpy() for node in sub.nodes])
        return idx, tab
    return [one(c) for c in layer.first_layer_chunks], [[one(l) for l in tree] for tree in layer.trees]


def _oracle_fns(kind, scale=1.25):
    if kind == "dwn":
        alpha, beta = np.float32(0.5 * 0.75 ** 5), np.float32(0.25 / 0.75)
        return ("luts", lambda x, i, t: orc.dwn_layer_forward(x, i, t)[:, :, 0],
                lambda x, i, t, g: orc.dwn_layer_backward(x, i, t, g[:, :, None], alpha, beta))
    if kind == "probabilistic":
        return ("raw_weights", lambda x, i, t: orc.prob_layer_forward(x, i, t)[:, :, 0],
                lambda x, i, t, g: orc.prob_layer_backward(x, i, t, g[:, :, None]))
    fwd = lambda x, i, t: orc.dwn_layer_forward(x, i, orc.table_sigmoid(t).astype(np.float32))[:, :, 0]
    if kind == "dwn_stable":
        return "raw_luts", fwd, lambda x, i, t, g: orc.stable_layer_backward(x, i, t, g[:, :, None], scale)
    return "raw_luts", fwd, lambda x, i, t, g: orc.hybrid_layer_backward(x, i, t, g[:, :, None])


GEOMS = [  # (B, C, H, W), (KH, KW, SH, SW, PH, PW)
    ((2, 3, 5, 6), (3, 2, 1, 2, 1, 0)),
    ((3, 1, 10, 10), (3, 3, 1, 1, 0, 0)),
    ((1, 4, 28, 28), (5, 5, 1, 1, 0, 0)),
    ((5, 2, 9, 7), (2, 3, 2, 3, 1, 2)),
    ((70, 1, 4, 4), (4, 4, 1, 1, 0, 0)),   # one row per image
    ((2, 2, 6, 6), (1, 1, 1, 1, 0, 0)),
]


@pytest.mark.parametrize("case", GEOMS)
def test_unfold_rows_planes_and_fold(case):
    """Patch matrix bit-exact against torch's unfold (CPU), its bit-planes against the packed oracle bits,
    and the fold of row-major and tile-major gradients against torch's fold."""
    from difflut_amd import _native as nat
    from difflut_amd import ops
    shape, geom = case
    rng = np.random.default_rng(sum(shape) + sum(geom))
    x = rng.random(shape).astype(np.float32)
    want = orc.conv_unfold(x, geom[0:2], geom[2:4], geom[4:6])
    xt = torch.tensor(x, device=DEV, requires_grad=True)
    patches = ops.UnfoldFunction.apply(xt, geom)
    assert np.array_equal(patches.detach().cpu().numpy(), want)
    rows, cols = want.shape
    lib = nat.lib()
    assert lib.dl_unfold_rows(shape[0], shape[2], shape[3], *geom) == rows
    planes = torch.zeros(lib.dl_dwn_planes_bytes(rows, cols) // 8, dtype=torch.int64, device=DEV)
    nat.check(lib.dl_unfold(xt.data_ptr(), None, planes.data_ptr(), *shape, *geom, nat.stream()))
    BT = (rows + 63) // 64
    bits = np.zeros((BT * 64, cols), dtype=np.uint64)
    bits[:rows] = (want >= 0.5).astype(np.uint64)
    packed = (bits.reshape(BT, 64, cols) << np.arange(64, dtype=np.uint64)[None, :, None]).sum(1, dtype=np.uint64)
    assert np.array_equal(planes.cpu().numpy().view(np.uint64)[:BT * cols].reshape(BT, cols), packed)
    g = rng.standard_normal(want.shape).astype(np.float32)
    patches.backward(torch.tensor(g, device=DEV))
    folded = orc.conv_fold(g, shape, geom[0:2], geom[2:4], geom[4:6])
    np.testing.assert_allclose(xt.grad.cpu().numpy(), folded, rtol=1e-6, atol=1e-6)  # <= KH*KW terms per pixel
    tiled = np.zeros((BT * 64, cols), dtype=np.float32)
    tiled[:rows] = g
    tiled = np.ascontiguousarray(tiled.reshape(BT, 64, cols).transpose(0, 2, 1))
    gx = torch.empty(shape, device=DEV)
    nat.check(lib.dl_fold(torch.tensor(tiled, device=DEV).data_ptr(), 1, gx.data_ptr(), *shape, *geom, nat.stream()))
    assert torch.equal(gx, xt.grad)  # same terms in the same order


def test_unfold_rejects_bad_geometry():
    from difflut_amd import ops
    with pytest.raises(RuntimeError):
        ops.UnfoldFunction.apply(torch.rand(1, 1, 3, 3, device=DEV), (5, 5, 1, 1, 0, 0))
    with pytest.raises(RuntimeError):
        ops.UnfoldFunction.apply(torch.rand(1, 1, 3, 3), (3, 3, 1, 1, 0, 0))  # CPU tensor


CASES = [  # (kind, depth, in_ch, out_ch, rf, stride, padding, chunk, image)
    ("dwn", 1, 1, 16, 3, 1, 0, 8, (4, 10, 10)),          # tests/test_layers/test_convolutional_learning.py:186-195
    ("dwn", 2, 2, 5, 3, 1, 1, 2, (3, 7, 6)),             # ragged last chunk, padding
    ("dwn", 2, 3, 4, (3, 2), (2, 1), (0, 1), 32, (2, 9, 8)),
    ("probabilistic", 1, 1, 16, 3, 1, 0, 8, (3, 8, 8)),
    ("probabilistic", 2, 2, 3, 2, 2, 0, 2, (2, 6, 6)),
    ("dwn_stable", 2, 2, 4, 3, 1, 0, 3, (2, 6, 7)),
    ("hybrid", 2, 1, 3, 3, 2, 1, 1, (3, 7, 7)),
]


@pytest.mark.parametrize("case", CASES)
def test_conv_layer_forward_backward_against_tree_loops(case):
    kind, depth, in_ch, out_ch, rf, stride, padding, chunk, (B, H, W) = case
    torch.manual_seed(sum(case[1:4]) + B)
    layer = _build(kind, depth, in_ch, out_ch, rf, stride, padding, chunk)
    assert layer._kind == kind
    layer.train()
    pname, fwd, bwd = _oracle_fns(kind)
    rng = np.random.default_rng(H * W + out_ch)
    x = (0.02 + 0.96 * rng.random((B, in_ch, H, W))).astype(np.float32)
    xt = torch.tensor(x, device=DEV, requires_grad=True)
    y = layer(xt)
    pair = lambda v: (v, v) if isinstance(v, int) else v
    rf2, st2, pd2 = pair(rf), pair(stride), pair(padding)
    oh, ow = (H + 2 * pd2[0] - rf2[0]) // st2[0] + 1, (W + 2 * pd2[1] - rf2[1]) // st2[1] + 1
    assert y.shape == (B, out_ch, oh, ow)
    chunks, trees = _tables(layer, pname)
    patches = orc.conv_unfold(x, rf2, st2, pd2)
    out, acts = orc.conv_trees_forward(patches, chunks, trees, layer.hidden_layers[0], fwd)
    want = out.reshape(B, oh * ow, out_ch).transpose(0, 2, 1).reshape(B, out_ch, oh, ow)
    if kind == "dwn":
        assert np.array_equal(y.detach().cpu().numpy(), want)  # lookups only: bit-exact
    else:
        np.testing.assert_allclose(y.detach().cpu().numpy(), want, rtol=1e-5, atol=1e-6)
    gy = rng.standard_normal(want.shape).astype(np.float32)
    y.backward(torch.tensor(gy, device=DEV))
    gout = gy.reshape(B, out_ch, oh * ow).transpose(0, 2, 1).reshape(-1, out_ch)
    gp, gch, gtr = orc.conv_trees_backward(patches, chunks, trees, layer.hidden_layers[0], acts, gout, bwd)
    gx = orc.conv_fold(gp, x.shape, rf2, st2, pd2)
    # gradients pass through up to three levels; terms are O(1): rtol 1e-5 with a floor of 5e-6
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=5e-6)
    for c, (sub, want_g) in enumerate(zip(layer.first_layer_chunks, gch)):
        got = np.stack([getattr(node, pname).grad.cpu().numpy() for node in sub.nodes])
        np.testing.assert_allclose(got, want_g, rtol=1e-5, atol=5e-6, err_msg=f"chunk {c}")
    for t in (0, out_ch - 1):
        for l, sub in enumerate(layer.trees[t]):
            got = np.stack([getattr(node, pname).grad.cpu().numpy() for node in sub.nodes])
            np.testing.assert_allclose(got, gtr[t][l], rtol=1e-5, atol=5e-6, err_msg=f"tree {t} layer {l}")


@pytest.mark.parametrize("kind", ["dwn", "probabilistic", "hybrid"])
def test_conv_layer_eval_and_state_dict_roundtrip(kind):
    torch.manual_seed(5)
    a = _build(kind, 2, 2, 5, 3, 1, 0, 2)
    b = _build(kind, 2, 2, 5, 3, 1, 0, 2)
    keys = set(a.state_dict().keys())
    pname = _oracle_fns(kind)[0]
    assert {f"first_layer_chunks.0.nodes.0.{pname}", f"first_layer_chunks.2.nodes.35.{pname}",
            f"trees.4.1.nodes.0.{pname}", "trees.0.0._mapping_indices", "first_layer_chunks.1._mapping_indices"} <= keys
    b.load_state_dict(a.state_dict())
    a.eval(); b.eval()
    x = torch.randint(0, 2, (3, 2, 6, 6), device=DEV).float()
    with torch.no_grad():
        ya, yb = a(x), b(x)
    assert torch.equal(ya, yb) and set(ya.unique().tolist()) <= {0.0, 1.0}
    # eval semantics level by level: every layer binarises its output
    chunks, trees = _tables(a, pname)
    if kind == "dwn":
        ev = lambda m, i, t: np.stack([orc.dwn_eval_forward(m[:, i[n]], t[n])[:, 0] for n in range(len(t))], 1)
    elif kind == "probabilistic":
        ev = lambda m, i, t: np.stack([orc.prob_eval_forward(m[:, i[n]], t[n])[:, 0] for n in range(len(t))], 1)
    else:
        ev = lambda m, i, t: np.stack([orc.dwn_eval_forward(m[:, i[n]], orc.table_sigmoid(t[n]).astype(np.float32))[:, 0]
                                       for n in range(len(t))], 1)
    patches = orc.conv_unfold(x.cpu().numpy(), (3, 3), (1, 1), (0, 0))
    out, _ = orc.conv_trees_forward(patches, chunks, trees, 36, ev)
    assert np.array_equal(ya.cpu().numpy(), out.reshape(3, 16, 5).transpose(0, 2, 1).reshape(3, 5, 4, 4))


@pytest.mark.parametrize("seed", [42, 43, 100])
def test_grouped_connections_cover_every_channel(seed):
    """tests/test_layers/test_grouped_convolutional_connections.py:25-94: with grouped connections and full
    coverage the first inputs of the first-layer nodes touch all 64 channels; every node stays inside one channel."""
    layer = _build("probabilistic", 1, 64, 16, 3, 1, 0, 128, grouped=True, seed=seed)
    table = layer.first_layer_chunks[0]._mapping_indices.cpu().long()
    assert (table[:, 0] // 9).unique().numel() == 64
    assert torch.all((table // 9) == (table[:, :1] // 9))
    x = torch.rand(2, 64, 8, 8, device=DEV)
    layer.train()
    y = layer(x)
    assert y.shape == (2, 16, 6, 6) and torch.isfinite(y).all()


def test_conv_bank_parameters_train_in_place():
    """An optimizer over bank_parameters() (one tensor per depth level) updates the per-node parameters the
    state dict shows."""
    torch.manual_seed(9)
    layer = _build("dwn", 2, 1, 6, 3, 1, 0, 4)
    layer.train()
    banks = layer.bank_parameters()
    assert [tuple(t.shape) for t in banks] == [(216, 1, 64), (36, 1, 64), (6, 1, 64)]
    opt = torch.optim.SGD(banks, lr=0.1)
    before = layer.trees[5][1].nodes[0].luts.detach().clone()
    x = torch.rand(4, 1, 8, 8, device=DEV)
    layer(x).sum().backward()
    assert all(t.grad is not None for t in banks)
    opt.step()
    after = layer.state_dict()["trees.5.1.nodes.0.luts"]
    assert not torch.equal(before, after)
    assert torch.equal(after, banks[2][5].detach())


def test_conv_layer_against_reference_vectors(golden_next):
    """The reference layer's own state dict loaded into this layer; outputs, input gradient, every table
    gradient and the eval outputs against what the reference's CPU path produced (tests/golden)."""
    from difflut_amd.layers import ConvolutionalLayer, ConvolutionConfig, RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig

    g = golden_next
    cfg = ConvolutionConfig(tree_depth=2, in_channels=2, out_channels=3, receptive_field=2, stride=1, padding=0,
                            chunk_size=2, seed=42)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        layer = ConvolutionalLayer(cfg, DWNNode, NodeConfig(input_dim=2, output_dim=1), RandomLayer, n_inputs_per_node=2)
    state = {k[len("conv_state."):]: torch.tensor(v) for k, v in g.items() if k.startswith("conv_state.")}
    layer.load_state_dict(state)
    layer = layer.to(DEV).train()
    x = torch.tensor(g["conv_x"], device=DEV, requires_grad=True)
    y = layer(x)
    assert np.array_equal(y.detach().cpu().numpy(), g["conv_y"])
    y.backward(torch.tensor(g["conv_gy"], device=DEV))
    np.testing.assert_allclose(x.grad.cpu().numpy(), g["conv_gx"], rtol=1e-5, atol=2e-6)
    checked = 0
    for name, param in layer.named_parameters():
        want = g.get(f"conv_grad.{name}")
        if want is not None and want.shape != ():
            np.testing.assert_allclose(param.grad.cpu().numpy(), want, rtol=1e-5, atol=2e-6, err_msg=name)
            checked += 1
    assert checked == 12 + 6 + 3
    layer.eval()
    with torch.no_grad():
        assert np.array_equal(layer(torch.tensor(g["conv_eval_x"], device=DEV)).cpu().numpy(), g["conv_eval_y"])


@pytest.mark.parametrize("kind", ["dwn", "hybrid"])
def test_conv_layer_with_grouped_connections_against_tree_loops(kind):
    """Grouped first-layer connections (every node inside one channel) through the fused levels."""
    torch.manual_seed(13)
    B, in_ch, H, W, out_ch = 3, 4, 7, 7, 5
    layer = _build(kind, 2, in_ch, out_ch, 3, 1, 0, 2, grouped=True, seed=7)
    layer.train()
    pname, fwd, bwd = _oracle_fns(kind)
    table = layer.first_layer_chunks[0]._mapping_indices.cpu().long()
    assert torch.all((table // 9) == (table[:, :1] // 9))
    rng = np.random.default_rng(14)
    x = (0.02 + 0.96 * rng.random((B, in_ch, H, W))).astype(np.float32)
    xt = torch.tensor(x, device=DEV, requires_grad=True)
    y = layer(xt)
    chunks, trees = _tables(layer, pname)
    patches = orc.conv_unfold(x, (3, 3), (1, 1), (0, 0))
    out, acts = orc.conv_trees_forward(patches, chunks, trees, layer.hidden_layers[0], fwd)
    want = out.reshape(B, 25, out_ch).transpose(0, 2, 1).reshape(B, out_ch, 5, 5)
    np.testing.assert_allclose(y.detach().cpu().numpy(), want, rtol=1e-6, atol=1e-7)
    gy = rng.standard_normal(want.shape).astype(np.float32)
    y.backward(torch.tensor(gy, device=DEV))
    gout = gy.reshape(B, out_ch, 25).transpose(0, 2, 1).reshape(-1, out_ch)
    gp, gch, _ = orc.conv_trees_backward(patches, chunks, trees, layer.hidden_layers[0], acts, gout, bwd)
    np.testing.assert_allclose(xt.grad.cpu().numpy(), orc.conv_fold(gp, x.shape, (3, 3), (1, 1), (0, 0)), rtol=1e-5, atol=5e-6)
    got = np.stack([getattr(node, pname).grad.cpu().numpy() for node in layer.first_layer_chunks[2].nodes])
    np.testing.assert_allclose(got, gch[2], rtol=1e-5, atol=5e-6)


# ------------------------------------------------------------------------------ bit-flip augmentation, gradient rescaling
def _conv_oracle(layer, kind, x, flip_mask, gy):
    """Forward and backward of the tree loops on the patch matrix with `flip_mask` applied (None: no flip)."""
    pname, fwd, bwd = _oracle_fns(kind)
    B, C, H, W = x.shape
    rf2, st2, pd2 = layer.receptive_field, layer.stride, layer.padding
    oh, ow = (H + 2 * pd2[0] - rf2[0]) // st2[0] + 1, (W + 2 * pd2[1] - rf2[1]) // st2[1] + 1
    chunks, trees = _tables(layer, pname)
    patches = orc.conv_unfold(x, rf2, st2, pd2)
    if flip_mask is not None:  # x + (1 - 2 x) in fp32, as base_layer.py:214-221 computes the flipped value
        patches = np.where(flip_mask, patches + (np.float32(1.0) - np.float32(2.0) * patches), patches).astype(np.float32)
    out, acts = orc.conv_trees_forward(patches, chunks, trees, layer.hidden_layers[0], fwd)
    want = out.reshape(B, oh * ow, layer.out_channels).transpose(0, 2, 1).reshape(B, layer.out_channels, oh, ow)
    gout = gy.reshape(B, layer.out_channels, oh * ow).transpose(0, 2, 1).reshape(-1, layer.out_channels)
    gp, gch, gtr = orc.conv_trees_backward(patches, chunks, trees, layer.hidden_layers[0], acts, gout, bwd)
    return want, orc.conv_fold(gp, x.shape, rf2, st2, pd2), gch, gtr


def _check_conv_grads(layer, kind, xt, gx, gch, gtr):
    pname = _oracle_fns(kind)[0]
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=5e-6)
    for c, (sub, want_g) in enumerate(zip(layer.first_layer_chunks, gch)):
        got = np.stack([getattr(node, pname).grad.cpu().numpy() for node in sub.nodes])
        np.testing.assert_allclose(got, want_g, rtol=1e-5, atol=5e-6, err_msg=f"chunk {c}")
    for t in (0, layer.out_channels - 1):
        for l, sub in enumerate(layer.trees[t]):
            got = np.stack([getattr(node, pname).grad.cpu().numpy() for node in sub.nodes])
            np.testing.assert_allclose(got, gtr[t][l], rtol=1e-5, atol=5e-6, err_msg=f"tree {t} layer {l}")


@pytest.mark.parametrize("kind,prob", [("dwn", 0.3), ("dwn", 0.02), ("probabilistic", 0.3), ("hybrid", 0.1)])
def test_conv_layer_with_bit_flip_against_tree_loops_on_the_same_mask(kind, prob):
    """flip_probability > 0 (convolutional.py:205-207): the mask the layer draws is reproduced from the same seed with
    the same generator calls and handed to the oracle.  For DWN trees the chained bit-plane path stays on (the flip is
    applied where the patch bits are formed); outputs bit-exact, gradients flow as if nothing had been flipped."""
    torch.manual_seed(11)
    layer = _build(kind, 2, 2, 5, 3, 1, 1, 2)
    layer.flip_probability = prob
    layer.train()
    B, C, H, W = 3, 2, 7, 6
    rng = np.random.default_rng(8)
    x = rng.integers(0, 2, (B, C, H, W)).astype(np.float32) if kind != "probabilistic" else \
        (0.02 + 0.96 * rng.random((B, C, H, W))).astype(np.float32)
    if kind == "dwn":
        x[0, 0, 0, :3] = [0.5, 0.49999997, 0.50000006]  # values whose flipped form sits at the threshold
    rows, cols = B * 7 * 6, C * 9   # padding 1: output 7 x 6
    xt = torch.tensor(x, device=DEV, requires_grad=True)
    torch.manual_seed(77)
    y = layer(xt)
    torch.manual_seed(77)
    if prob < 0.05:
        mask = torch.zeros(rows * cols, dtype=torch.bool, device=DEV)
        mask[torch.randperm(rows * cols, device=DEV)[:int(rows * cols * prob)]] = True
        mask = mask.view(rows, cols)
    else:
        mask = torch.bernoulli(torch.full((rows, cols), prob, device=DEV, dtype=torch.float32)).bool()
    assert 0 < int(mask.sum()) < rows * cols
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(torch.tensor(gy, device=DEV))
    want, gx, gch, gtr = _conv_oracle(layer, kind, x, mask.cpu().numpy(), gy)
    if kind == "dwn":
        assert layer._chained()
        assert np.array_equal(y.detach().cpu().numpy(), want)
    else:
        np.testing.assert_allclose(y.detach().cpu().numpy(), want, rtol=1e-5, atol=1e-6)
    _check_conv_grads(layer, kind, xt, gx, gch, gtr)
    # and the flip really changed something: the unflipped oracle differs
    plain = _conv_oracle(layer, kind, x, None, gy)[0]
    assert not np.array_equal(plain, want)
    # eval mode never flips
    layer.eval()
    with torch.no_grad():
        assert torch.equal(layer(xt), layer(xt))


@pytest.mark.parametrize("mode", ["layerwise", "batchwise"])
@pytest.mark.parametrize("subtract_mean", [False, True])
@pytest.mark.parametrize("kind", ["dwn", "probabilistic"])
def test_conv_layer_gradient_stabilization_against_formula(kind, mode, subtract_mean):
    """grad_stabilization (base_layer.py:266-339 through the hook of convolutional.py:252-265): the gradient that
    reaches the trees is (g - mean) * sqrt(target / (mean((g - mean)^2) + eps)), over the whole output or per image.
    The oracle's tree loops are fed the rescaled gradient computed in float64 from that formula."""
    torch.manual_seed(13)
    layer = _build(kind, 2, 2, 4, 3, 1, 0, 3)
    layer.grad_stabilization, layer.grad_target_std, layer.grad_subtract_mean, layer.grad_epsilon = mode, 0.7, subtract_mean, 1e-8
    layer.train()
    B, C, H, W = 4, 2, 6, 7
    rng = np.random.default_rng(3)
    x = (0.02 + 0.96 * rng.random((B, C, H, W))).astype(np.float32)
    xt = torch.tensor(x, device=DEV, requires_grad=True)
    y = layer(xt)
    gy = (rng.standard_normal(tuple(y.shape)) * 3.0 + 0.5).astype(np.float32)
    y.backward(torch.tensor(gy, device=DEV))
    g = gy.reshape(B, -1).astype(np.float64)
    axis = None if mode == "layerwise" else 1
    if subtract_mean:
        g = g - g.mean(axis=axis, keepdims=axis is not None)
    var = (g ** 2).mean(axis=axis, keepdims=axis is not None)
    g = (g * np.sqrt(0.7 / (var + 1e-8))).astype(np.float32).reshape(gy.shape)
    want, gx, gch, gtr = _conv_oracle(layer, kind, x, None, g)
    _check_conv_grads(layer, kind, xt, gx, gch, gtr)
