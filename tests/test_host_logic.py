"""CPU-only checks: the C-ABI library exports every declared symbol, the host-side mirror of the
reference interface builds the same state (mapping table, per-node tables, generator position,
state-dict keys) and refuses to compute on CPU tensors."""
import ctypes
import os
import re
import warnings

import numpy as np
import pytest
import torch

warnings.filterwarnings("ignore")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from difflut_amd import _native as nat

    if not nat.is_built():
        import difflut_amd.build as b
        b.build()
    header = open(os.path.join(ROOT, "include", "difflut_hip.h")).read()
    declared = set(re.findall(r"\b(dl_[a-z0-9_]+)\s*\(", header))
    assert declared == set(nat.SIGNATURES), declared ^ set(nat.SIGNATURES)
    handle = ctypes.CDLL(nat.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    assert handle.dl_version() >= 100
    nat.lib()
    assert nat.lib().dl_error_string(-4).decode().startswith("workspace")
    # size queries are host-only arithmetic: callable without a GPU
    assert nat.lib().dl_dwn_saved_bytes(4096, 16384, 8192, 6, 1) == 4096 * 8192
    assert nat.lib().dl_dwn_fwd_workspace_bytes(4096, 16384, 8192, 6, 1) == 64 * 16384 * 8


def test_registry_names_and_errors():
    from difflut_amd import REGISTRY
    from difflut_amd.layers import LearnableLayer, RandomLayer
    from difflut_amd.nodes import DWNNode, ProbabilisticNode

    assert REGISTRY.get_node("dwn") is DWNNode and REGISTRY.get_node("probabilistic") is ProbabilisticNode
    assert REGISTRY.get_layer("random") is RandomLayer and REGISTRY.get_layer("learnable") is LearnableLayer
    assert "thermometer" in REGISTRY.list_encoders() and "uniform" in REGISTRY.list_initializers()
    with pytest.raises(ValueError, match="not found"):
        REGISTRY.get_node("nope")
    enc = REGISTRY.build_encoder("thermometer", num_bits=3)
    assert enc.num_bits == 3 and not enc.is_fitted


@pytest.mark.parametrize("tag", ["fused_a", "fused_b", "layer_fn", "exact3", "cfg1", "nocover"])
def test_random_layer_construction_matches_reference(golden, tag):
    from difflut_amd.layers import RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig

    I, N, k, seed, cover = (int(v) for v in golden[f"map_{tag}_meta"])
    torch.manual_seed(1234)
    layer = RandomLayer(I, N, DWNNode, NodeConfig(input_dim=k, output_dim=1), seed=seed,
                        ensure_full_input_coverage=bool(cover))
    assert layer._mapping_indices.dtype == torch.int16
    assert np.array_equal(layer._mapping_indices.numpy(), golden[f"map_{tag}_idx"])
    assert np.array_equal(layer.nodes[0].luts.detach().numpy(), golden[f"map_{tag}_lut_first"])
    assert np.array_equal(layer.nodes[N - 1].luts.detach().numpy(), golden[f"map_{tag}_lut_last"])
    assert np.array_equal(torch.rand(4).numpy(), golden[f"map_{tag}_next_rand"])  # generator position
    assert layer.n == k and layer.output_dim_per_node == 1 and len(layer.nodes) == N


def test_state_dict_keys_and_parameter_views():
    from difflut_amd.layers import LearnableLayer, RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig, ProbabilisticNode

    layer = RandomLayer(20, 6, DWNNode, NodeConfig(input_dim=3, output_dim=2), seed=1)
    keys = set(layer.state_dict().keys())
    assert {"_mapping_indices", "nodes.0.luts", "nodes.0.alpha", "nodes.0.beta", "nodes.5.luts"} <= keys
    assert layer.nodes[2].luts.shape == (2, 8) and len(list(layer.parameters())) == 6
    flat = layer._banks["luts"].tensor()
    with torch.no_grad():
        layer.nodes[4].luts.fill_(0.25)  # a per-node parameter is a view of the layer's table tensor
    assert torch.all(flat[4] == 0.25)
    other = RandomLayer(20, 6, DWNNode, NodeConfig(input_dim=3, output_dim=2), seed=1)
    other.load_state_dict(layer.state_dict())
    assert torch.equal(other._banks["luts"].tensor().detach(), flat.detach())
    # gradients: one tensor for the layer, per-node .grad are its rows; zero_grad clears it
    flat.grad = torch.ones_like(flat)
    assert torch.all(layer.nodes[1].luts.grad == 1)
    opt = torch.optim.SGD(layer.parameters(), lr=0.5)
    opt.step()
    assert torch.allclose(layer.nodes[4].luts.detach(), torch.full((2, 8), -0.25))
    opt.zero_grad()
    assert layer.nodes[1].luts.grad is None and flat.grad is None
    moved = layer.double()  # Module._apply re-allocates every parameter: the layer re-ties them
    assert moved._banks["luts"].tied() and moved.nodes[4].luts.dtype == torch.float64

    p = RandomLayer(16, 4, ProbabilisticNode, NodeConfig(input_dim=2, output_dim=1), seed=1)
    assert {"nodes.0.raw_weights", "nodes.0.temperature", "nodes.0.binary_combinations"} <= set(p.state_dict())
    assert p.nodes[0].raw_weights.shape == (4, 1)
    assert p.nodes[0].binary_combinations.tolist() == [[0, 0], [1, 0], [0, 1], [1, 1]]  # LSB first
    torch.manual_seed(3)
    l = LearnableLayer(20, 7, DWNNode, NodeConfig(input_dim=3, output_dim=1), tau=1.0, tau_start=1.0, tau_min=1e-4,
                       tau_decay_iters=1000.0, use_cuda_soft=False)
    assert l.mapping.W.shape == (21, 20) and "mapping.W" in l.state_dict()
    l.update_tau(500)
    assert l.tau == pytest.approx(10 ** -0.5) and l.mapping.tau == l.tau
    l.update_tau(10 ** 9)
    assert l.tau == 1e-4


def test_learnable_layer_W_matches_reference_draw(golden):
    from difflut_amd.layers import LearnableLayer
    from difflut_amd.nodes import DWNNode, NodeConfig

    torch.manual_seed(3)
    l = LearnableLayer(20, 7, DWNNode, NodeConfig(input_dim=3, output_dim=1), tau=1.0, tau_start=1.0, tau_min=1e-4,
                       tau_decay_iters=1000.0, use_cuda_soft=False)
    assert np.array_equal(l.mapping.W.detach().numpy(), golden["soft_W"])


def test_constructor_validation_and_cpu_refusal():
    from difflut_amd.layers import LayerConfig, RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig
    from difflut_amd.utils import GroupSum

    cfg = NodeConfig(input_dim=2, output_dim=1)
    with pytest.raises(ValueError):
        RandomLayer(0, 4, DWNNode, cfg)
    with pytest.raises(ValueError):
        RandomLayer(8, -1, DWNNode, cfg)
    with pytest.raises(ValueError):
        DWNNode(input_dim=0, output_dim=1)
    with pytest.raises(TypeError):
        DWNNode(input_dim=2, output_dim=1, init_fn=3)
    with pytest.raises(ValueError):
        LayerConfig(flip_probability=1.5)
    with pytest.raises(TypeError):
        RandomLayer(8, 4, DWNNode, cfg, layer_config={"flip_probability": 0.1})
    with pytest.raises(ValueError):
        GroupSum(k=0)
    layer = RandomLayer(8, 4, DWNNode, cfg)
    with pytest.raises(ValueError, match="2D input"):
        layer(torch.zeros(8))
    with pytest.raises(ValueError, match="expected input with 8 features"):
        layer(torch.zeros(2, 9))
    assert layer(torch.zeros(2, 8)).shape == (2, 4)  # CPU tensors take the plain-torch branch
    assert DWNNode(input_dim=6, output_dim=1).alpha.item() == pytest.approx(0.5 * 0.75 ** 5)


def test_residual_initialiser_known_answer(golden):
    from difflut_amd.nodes import DWNNode, ProbabilisticNode
    from difflut_amd.nodes.utils import residual_init

    kw = {"node_type": "dwn", "noise_factor": 0.0, "logit_clarity": 5.0, "input_dim": 6}
    node = DWNNode(input_dim=6, output_dim=1, init_fn=residual_init, init_kwargs=kw)
    assert np.array_equal(node.luts.detach().numpy(), golden["dwn_residual_luts"])
    p = ProbabilisticNode(input_dim=3, output_dim=2, init_fn=residual_init,
                          init_kwargs={"node_type": "probabilistic", "noise_factor": 0.0, "logit_clarity": 5.0,
                                       "input_dim": 3})
    assert p.raw_weights[:, 0].tolist() == [-5, 5, -5, 5, -5, 5, -5, 5]


def test_stable_and_hybrid_nodes_consume_the_generator_like_the_reference(golden_next):
    """Same constructor calls in the same order as the script that wrote the vectors: default `raw_luts`
    (randn * 0.1), initialised tables, inputs and the generator position afterwards all agree."""
    from difflut_amd.nodes import DWNStableNode, HybridNode
    from difflut_amd.nodes.utils import uniform_init

    g = golden_next
    torch.manual_seed(21)
    for cls, kind in ((DWNStableNode, "stable"), (HybridNode, "hybrid")):
        for tag, B, k, O in (("k6o1", 12, 6, 1), ("k3o2", 9, 3, 2)):
            kw = {"gradient_scale": 1.6} if kind == "stable" else {}
            node = cls(input_dim=k, output_dim=O, use_cuda=False, **kw)
            assert np.array_equal(node.raw_luts.detach().numpy(), g[f"{kind}_{tag}_default_raw"])
            node = cls(input_dim=k, output_dim=O, use_cuda=False, init_fn=uniform_init, init_kwargs={"a": -2.0, "b": 2.0}, **kw)
            assert np.array_equal(node.raw_luts.detach().numpy(), g[f"{kind}_{tag}_raw"])
            assert tuple(node.raw_luts.shape) == (O, 2 ** k)
            if kind == "stable":
                assert abs(float(node.gradient_scale) - 1.6) < 1e-7 and isinstance(node.gradient_scale, torch.nn.Parameter)
            else:
                assert np.array_equal(node.binary_combinations.numpy()[5][:3], [1.0, 0.0, 1.0])  # input 0 = LSB
            x = 0.02 + 0.96 * torch.rand(B, k)
            assert np.array_equal(x.numpy(), g[f"{kind}_{tag}_x"])
            torch.randn(B, O); torch.randint(0, 2, (B, k))
    assert np.array_equal(torch.rand(3).numpy(), g["next_rand_after_nodes"])


@pytest.mark.parametrize("tag,cover", [("cover", True), ("nocover", False)])
def test_grouped_input_mapping_matches_reference(golden_next, tag, cover):
    from difflut_amd.layers import GroupedInputConfig

    g = golden_next
    torch.manual_seed(77)
    cfg = GroupedInputConfig(n_groups=4, input_size=36, output_trees=5, luts_per_tree=6, bits_per_node=6, seed=42,
                             ensure_full_coverage=cover)
    assert np.array_equal(cfg.mapping_indices.numpy(), g[f"grouped_{tag}_table"])
    assert np.array_equal(cfg.get_mapping_indices(1, 3).numpy(), g[f"grouped_{tag}_chunk_1_3"])
    assert np.array_equal(torch.rand(2).numpy(), g[f"grouped_{tag}_next_rand"])
    groups = cfg.mapping_indices // 9
    assert torch.all(groups == groups[:, :1])  # a node stays inside one group
    if cover:
        assert sorted(groups[:28, 0].tolist()) == sorted(list(range(4)) * 7)  # dealt out as permutations


def test_convolutional_layer_construction_matches_reference(golden_next):
    """Sub-module layout, state-dict keys, index tables and per-node tables of a seeded layer."""
    from difflut_amd import REGISTRY
    from difflut_amd.layers import ConvolutionalLayer, ConvolutionConfig, RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig, ProbabilisticNode
    from difflut_amd.nodes.utils import uniform_init

    g = golden_next
    assert REGISTRY.get_convolutional_layer("convolutional") is ConvolutionalLayer
    torch.manual_seed(31)
    cfg = ConvolutionConfig(tree_depth=2, in_channels=2, out_channels=3, receptive_field=2, stride=1, padding=0,
                            chunk_size=2, seed=42)
    layer = ConvolutionalLayer(cfg, DWNNode, NodeConfig(input_dim=2, output_dim=1, init_fn=uniform_init,
                                                        init_kwargs={"a": -1.0, "b": 2.0}), RandomLayer, n_inputs_per_node=2)
    want = {k[len("conv_state."):]: v for k, v in g.items() if k.startswith("conv_state.")}
    state = layer.state_dict()
    assert set(state) == set(want)
    for name, value in want.items():
        assert np.array_equal(state[name].numpy(), value), name
    assert layer.hidden_layers == [4, 2, 1] and len(layer.first_layer_chunks) == 2 and len(layer.trees) == 3
    assert [tuple(t.shape) for t in layer.bank_parameters()] == [(12, 1, 4), (6, 1, 4), (3, 1, 4)]
    assert np.array_equal(torch.rand(4, 2, 4, 4)[:2].numpy(), g["conv_x"])  # generator position after construction
    assert layer(torch.rand(2, 2, 4, 4)).shape == (2, 3, 3, 3)  # CPU tensors take the plain-torch branch
    torch.manual_seed(32)
    gcfg = ConvolutionConfig(tree_depth=1, in_channels=4, out_channels=5, receptive_field=3, stride=1, padding=0,
                             chunk_size=2, seed=43)
    glayer = ConvolutionalLayer(gcfg, ProbabilisticNode, NodeConfig(input_dim=6, output_dim=1), RandomLayer,
                                n_inputs_per_node=6, grouped_connections=True, ensure_full_coverage=True)
    for c, chunk in enumerate(glayer.first_layer_chunks):
        assert np.array_equal(chunk._mapping_indices.numpy(), g[f"gconv_chunk{c}_idx"])
    assert np.array_equal(glayer.trees[0][0]._mapping_indices.numpy(), g["gconv_tree0_idx"])
    assert np.array_equal(glayer.trees[4][0]._mapping_indices.numpy(), g["gconv_tree4_idx"])
    assert np.array_equal(glayer.first_layer_chunks[0].nodes[0].raw_weights.detach().numpy(), g["gconv_first_raw"])
    assert np.array_equal(glayer.trees[4][0].nodes[0].raw_weights.detach().numpy(), g["gconv_last_raw"])


def test_argument_checks_of_the_later_entry_points_need_no_gpu():
    """Null pointers, bad sizes and unsupported geometries are refused before anything is launched."""
    from difflut_amd import _native as nat

    lib = nat.lib()
    one = ctypes.c_void_p(64)  # any non-null value: the checks below fail before it is dereferenced
    assert lib.dl_unfold(None, one, None, 1, 1, 4, 4, 2, 2, 1, 1, 0, 0, None) == -1
    assert lib.dl_unfold(one, None, None, 1, 1, 4, 4, 2, 2, 1, 1, 0, 0, None) == -1        # no output asked for
    assert lib.dl_unfold(one, one, None, 1, 1, 4, 4, 5, 5, 1, 1, 0, 0, None) == -2         # window larger than image
    assert lib.dl_unfold(one, one, None, 1, 1, 4, 4, 2, 2, 0, 1, 0, 0, None) == -2         # zero stride
    assert lib.dl_unfold(one, one, None, 1, 64, 20, 20, 9, 9, 1, 1, 0, 0, None) == -3      # 5184 columns > 4096
    assert lib.dl_fold(None, 0, one, 1, 1, 4, 4, 2, 2, 1, 1, 0, 0, None) == -1
    assert lib.dl_unfold_rows(3, 28, 28, 5, 5, 1, 1, 0, 0) == 3 * 24 * 24
    assert lib.dl_unfold_rows(3, 28, 28, 5, 5, 2, 2, 2, 2) == 3 * 14 * 14
    assert lib.dl_unfold_rows(3, 4, 4, 5, 5, 1, 1, 0, 0) == 0
    assert lib.dl_table_sigmoid_fwd(one, one, 0, None) == -2 and lib.dl_table_sigmoid_fwd(None, one, 8, None) == -1
    assert lib.dl_table_sigmoid_bwd(one, None, one, 8, None) == -1
    assert lib.dl_dwn_stable_layer_bwd(None, one, one, one, one, one, one, None, one, one, one, 1 << 30,
                                       64, 8, 4, 2, 1, None) == -1                          # no gradient scale
    assert lib.dl_dwn_stable_layer_bwd(None, one, one, one, one, one, one, one, one, one, one, 0,
                                       64, 8, 4, 2, 1, None) == -4                          # workspace too small
    assert lib.dl_hybrid_layer_bwd(one, one, one, one, one, one, one, one, one, 0, 64, 8, 4, 2, 1, None) == -4
    assert lib.dl_hybrid_layer_bwd(one, one, one, one, one, one, one, one, one, 1 << 30, 64, 8, 4, 0, 1, None) == -2
    assert lib.dl_thermometer_planes(one, None, one, 4, 4, 2, None) == -1
    assert lib.dl_thermometer_planes(one, one, one, 4, 0, 2, None) == -2
    dims = (4096, 16384, 8192, 6, 1)
    assert lib.dl_hybrid_bwd_workspace_bytes(*dims) < lib.dl_prob_bwd_workspace_bytes(*dims)
    assert lib.dl_hybrid_bwd_workspace_bytes(*dims) >= 4096 * (16384 + 8192 + 6 * 8192) * 4


# ------------------------------------------------------------------------------ parameter and scalar banks
def _small_dwn_layer(n=12, k=3, inputs=20):
    from difflut_amd.layers import RandomLayer
    from difflut_amd.nodes import DWNNode, NodeConfig
    return RandomLayer(inputs, n, DWNNode, NodeConfig(input_dim=k, output_dim=1), seed=5)


@pytest.mark.parametrize("how", ["deepcopy", "pickle"])
def test_parameters_are_final_after_copy_so_an_optimizer_built_at_once_trains(how):
    """copy.deepcopy / pickle hand back a layer whose per-node Parameters are already views of the bank: an optimizer
    built before any forward holds the tensors the layer uses, and a step moves the bank."""
    import copy
    import pickle
    layer = _small_dwn_layer()
    twin = copy.deepcopy(layer) if how == "deepcopy" else pickle.loads(pickle.dumps(layer))
    params = list(twin.parameters())
    ids = [id(p) for p in params]
    opt = torch.optim.SGD(params, lr=0.5)
    bank = twin._banks["luts"]
    flat = bank.tensor()                      # what the first forward asks for
    assert [id(p) for p in twin.parameters()] == ids and bank.tensor() is flat
    assert bank.nodes[3]._parameters["luts"].data_ptr() == flat[3].data_ptr()
    before = flat.detach().clone()
    flat.grad = torch.ones_like(flat)         # what a backward leaves
    assert params[3].grad is not None and torch.equal(params[3].grad, torch.ones_like(params[3]))
    opt.step()
    assert torch.equal(flat.detach(), before - 0.5)
    assert torch.equal(twin.nodes[3].luts.detach(), before[3] - 0.5)
    # the original is untouched and still tied to its own bank
    assert layer._banks["luts"].tied() and not torch.equal(layer._banks["luts"].flat.detach(), flat.detach())


def test_bank_notices_nodes_taken_over_or_replaced():
    """A bank whose nodes were re-tied by another bank (a sub-layer called on its own inside a convolutional level) or
    whose parameter was reassigned is stale, whichever node it was - not only the first or the last."""
    from difflut_amd.layers.base_layer import ParameterBank
    layer = _small_dwn_layer()
    bank = layer._banks["luts"]
    assert bank.tied()
    middle = ParameterBank(list(layer.nodes)[4:8], "luts")   # takes nodes 4..7 away
    assert middle.tied() and not bank.tied()
    flat = bank.tensor()                                      # re-ties all twelve
    assert bank.tied() and not middle.tied()
    assert layer.nodes[5].luts.data_ptr() == flat[5].data_ptr()
    layer.nodes[6].luts = torch.nn.Parameter(torch.zeros(1, 8))
    assert not bank.tied()
    assert torch.equal(bank.tensor()[6], torch.zeros(1, 8))


def test_scalar_buffers_are_banked_and_differences_are_seen():
    layer = _small_dwn_layer()
    alpha, beta = layer._scalars["alpha"], layer._scalars["beta"]
    alpha_n, beta_n, beta_max = layer.efd_scalars()
    assert alpha_n.shape == beta_n.shape == (12,) and alpha_n.dtype == torch.float32
    assert float(alpha_n[3]) == pytest.approx(0.5 * 0.75 ** 2) and beta_max == pytest.approx(1 / 3)
    assert set(layer.state_dict()) >= {"nodes.0.alpha", "nodes.11.beta"} and layer.state_dict()["nodes.0.alpha"].shape == ()
    # a state dict with another value for one node in the middle lands in the array the kernels are handed
    state = layer.state_dict()
    state["nodes.7.alpha"] = torch.tensor(0.25)
    layer.load_state_dict(state)
    assert alpha.tied() and float(layer.efd_scalars()[0][7]) == 0.25 and float(layer.efd_scalars()[0][6]) != 0.25
    # in-place edits too
    with torch.no_grad():
        layer.nodes[4].beta.fill_(0.75)
    assert float(layer.efd_scalars()[1][4]) == 0.75 and layer.efd_scalars()[2] == pytest.approx(0.75)
    # replacing a node's buffer object re-ties on the next use
    layer.nodes[2].beta = torch.tensor(0.9)
    assert not beta.tied()
    assert layer.efd_scalars()[2] == pytest.approx(0.9)
    assert layer.nodes[2].beta.data_ptr() == beta.flat[2].data_ptr()
    # a buffer entry swapped behind the module's back (no __setattr__) is noticed as well
    layer.nodes[5]._buffers["alpha"] = torch.tensor(0.5)
    assert not alpha.tied()
    assert float(layer.efd_scalars()[0][5]) == 0.5 and alpha.tied()


def test_writes_that_bypass_the_version_counter():
    """`buffer.data.fill_` does not bump the version the host-side summary is keyed on: the kernels still get the
    value (they are handed the array itself), and `invalidate_scalars()` refreshes max |beta|, which selects the
    form of the coefficient table."""
    layer = _small_dwn_layer()
    assert layer.efd_scalars()[2] == pytest.approx(1 / 3)
    layer.nodes[1].beta.data.fill_(0.9)
    assert float(layer.efd_scalars()[1][1]) == pytest.approx(0.9)  # the value itself is never stale
    assert layer.efd_scalars()[2] == pytest.approx(1 / 3)          # the cached maximum is
    layer.invalidate_scalars()
    assert layer.efd_scalars()[2] == pytest.approx(0.9)


def test_scalar_banks_keep_the_buffers_dtype():
    layer = _small_dwn_layer().double()
    assert layer.nodes[3].alpha.dtype == torch.float64 and layer.nodes[3].luts.dtype == torch.float64
    alpha_n, beta_n, _ = layer.efd_scalars()
    assert alpha_n.dtype == beta_n.dtype == torch.float32  # the kernels' view
    assert layer.state_dict()["nodes.3.beta"].dtype == torch.float64


def test_probabilistic_layer_hands_over_per_node_temperatures():
    from difflut_amd.layers import RandomLayer
    from difflut_amd.nodes import NodeConfig, ProbabilisticNode
    layer = RandomLayer(16, 8, ProbabilisticNode, NodeConfig(input_dim=2, output_dim=1), seed=1)
    assert torch.equal(layer.temperatures(), torch.ones(8))
    with torch.no_grad():
        layer.nodes[5].temperature.fill_(2.0)
    assert float(layer.temperatures()[5]) == 2.0 and float(layer.temperatures()[4]) == 1.0


def test_size_limits_and_argument_errors_are_reported_before_any_launch():
    """Error codes of the C ABI on the host side: nothing below reaches a kernel launch, so it runs without a GPU."""
    from difflut_amd import _native as nat
    lib = nat.lib()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    NULL, SHAPE, UNSUPPORTED, WORKSPACE = -1, -2, -3, -4
    assert lib.dl_gather_fwd(None, p, 16, p, 4, 4, 4, 2, None) == NULL
    assert lib.dl_gather_fwd(p, p, 8, p, 4, 4, 4, 2, None) == UNSUPPORTED            # index width
    assert lib.dl_gather_bwd(p, p, p, p, 0, 4, 4, 2, None) == SHAPE
    assert lib.dl_dwn_layer_fwd(p, p, p, p, p, p, 64, 4, 4, 4, 17, 1, None) == UNSUPPORTED   # k > DL_MAX_K
    assert lib.dl_dwn_layer_fwd(p, p, p, p, p, p, 8, 4096, 16384, 8192, 6, 1, None) == WORKSPACE
    assert lib.dl_dwn_layer_bwd(None, p, p, p, p, p, p, 0.1, 0.3, p, p, p, 8, 4096, 16384, 8192, 6, 1, None) == WORKSPACE
    assert lib.dl_prob_layer_fwd(p, p, p, 1.0, p, p, 64, 4000001, 4, 4, 2, 1, None) == UNSUPPORTED  # batch tiles > grid.y
    assert lib.dl_thermometer_planes(p, p, p, 4000001, 4, 2, None) == UNSUPPORTED
    # 256 channels with a 5x5 field: more patch columns than the per-block offset table holds
    assert lib.dl_unfold(p, p, None, 1, 256, 8, 8, 5, 5, 1, 1, 0, 0, None) == UNSUPPORTED
    assert lib.dl_unfold(p, p, None, 1, 1, 3, 3, 5, 5, 1, 1, 0, 0, None) == SHAPE           # field larger than the image
    assert lib.dl_unfold_rows(2, 8, 8, 3, 3, 1, 1, 0, 0) == 2 * 36
    assert lib.dl_dwn_layer_fwd_static(p, p, p, p, p, 4097, 16384, 8, 6, 1, None) == -6
    for code in (NULL, SHAPE, UNSUPPORTED, WORKSPACE, -5, -6):
        assert len(lib.dl_error_string(code)) > 10
