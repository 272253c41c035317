"""The benchmark configurations at their full sizes against the CPU restatements on ALL rows.

  * single DWN layer (4096 x 16384 -> 8192 nodes, k = 6): outputs, input gradient and table gradient of every row
    against the C restatement of the reference's loops (oracle/dwn_oracle.c);
  * deep stack (8192 x 784 -> thermometer 4 -> 16000/8000/4000/2000 DWN nodes -> GroupSum 10 -> cross-entropy):
    the C restatement runs all four layers forward and backward; logits, loss and every layer's table gradient of
    the chained device run are compared with it, then one Adam(lr=0.01) step on the tables with torch's CPU Adam
    fed the restatement's gradients;
  * LearnableLayer (3136 -> 8000 DWN nodes, k = 6, B = 512): soft connectivity against float64 softmax + matmul,
    the node stage against the C restatement on the device's own mapped values, all three gradients.

Tolerances: outputs and addresses bit-exact; gradients rtol 1e-5 with an absolute floor of a few fp32 ulps of the
sums' scale (written at each comparison); soft-connectivity gradients rtol 1e-4 (sums of 3136..48000 terms).
"""
import warnings

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu
warnings.filterwarnings("ignore")


def _api():
    from difflut_amd import REGISTRY
    from difflut_amd.nodes import NodeConfig
    from difflut_amd.nodes.utils import uniform_init
    return REGISTRY, NodeConfig, uniform_init


def test_single_dwn_layer_all_rows_against_c_restatement():
    from difflut_amd import ops
    from difflut_amd.layers.random_layer import draw_mapping
    torch.manual_seed(0)
    B, I, N, k = 4096, 16384, 8192, 6
    x = torch.bernoulli(torch.full((B, I), 0.5, device="cuda"))
    idx = draw_mapping(I, N, k, seed=42)
    plan = ops.MappingPlan(idx.cuda(), I)
    luts = (torch.rand(N, 1, 64, device="cuda") * 2 - 1).requires_grad_()
    gy = torch.randn(B, N, device="cuda")
    alpha, beta = 0.5 * 0.75 ** 5, 1 / 3
    xg = x.clone().requires_grad_()
    y = ops.DWNLayerFunction.apply(xg, luts, plan, alpha, beta)
    y.backward(gy)
    xs, idn, ln = x.cpu().numpy(), idx.numpy(), luts.detach().cpu().numpy()
    assert np.array_equal(y.detach().cpu().numpy(), c_oracle.dwn_layer_forward(xs, idn, ln)[:, :, 0])  # bit exact
    cgx, cgl = c_oracle.dwn_layer_backward(xs, idn, ln, gy.cpu().numpy()[:, :, None], np.float32(alpha), np.float32(beta))
    # three terms of size alpha * |gy| * |dS| ~ 0.1 .. 1 per input
    np.testing.assert_allclose(xg.grad.cpu().numpy(), cgx, rtol=1e-5, atol=2e-6)
    # a bin sums about B / 64 = 64 values of size ~1
    np.testing.assert_allclose(luts.grad.cpu().numpy(), cgl, rtol=1e-5, atol=2e-5)
    # both gradients are summed in a fixed order (no floating-point atomics): a second run gives the same bits
    x2, l2 = x.clone().requires_grad_(), luts.detach().clone().requires_grad_()
    ops.DWNLayerFunction.apply(x2, l2, plan, alpha, beta).backward(gy)
    assert torch.equal(l2.grad, luts.grad) and torch.equal(x2.grad, xg.grad)


@pytest.mark.parametrize("mapping,B,beta,shape", [
    ("whole permutations", 4096, 1 / 3, (16384, 8192, 6)), ("independent draws", 4096, 1 / 3, (16384, 8192, 6)),
    ("whole permutations", 4100, 1 / 3, (16384, 8192, 6)), ("whole permutations", 4096, 0.9, (16384, 8192, 6)),
    ("independent draws", 4100, 0.9, (16384, 8192, 6)),
    # fewer inputs per node: rows of 4 and 8 values, two of them per register all the same
    ("whole permutations", 2100, 1 / 3, (16384, 16384, 3)), ("whole permutations", 2048, 0.9, (16384, 12288, 4)),
    # 8000 inputs fit one XCD's resident blocks at 16 inputs per wavefront: the walking gather without the packing
    ("whole permutations", 2100, 1 / 3, (8000, 8000, 3)),
    # widths that are no multiple of a block's 128 inputs or of four (scalar stores, a last block with two inputs)
    ("whole permutations", 2100, 1 / 3, (16386, 8193, 6)),
    # more than 6000 rows: the backward is taken in chunks of about 4096 rows (two here, the last tile with eight rows;
    # three of 53 or 54 tiles each), and the table gradient adds the chunks' partial sums one after the other
    ("whole permutations", 8200, 1 / 3, (16384, 8192, 6)), ("independent draws", 10250, 0.9, (16384, 8192, 6)),
    # equal widths, every input read six times: sixteen inputs per wavefront with the packed rows; and the in-order
    # gather in chunks of rows (8192 inputs: the walking gather does not apply)
    ("whole permutations", 2100, 1 / 3, (12288, 12288, 6)), ("whole permutations", 2050, 0.9, (12288, 12288, 6)),
    ("whole permutations", 8200, 1 / 3, (8192, 8192, 6))])
def test_row_major_input_gradient_of_a_big_layer_equals_the_tile_major_one(mapping, B, beta, shape):
    """At this size the row-major input gradient is taken by the walking, paced gather (two entries' rows of table
    differences per register, 32 inputs per wavefront), the tile-major one by the one-block-per-(slab, tile) gather:
    the same terms in the same order, so the same bits - with every input read exactly three times (the unrolled path
    with the coefficient rows in registers) and with the same number of connections drawn independently (uneven lists:
    the general loop inside the walking kernel).  Three calls in a row (the pace of the walking gather moves between
    launches; the sums must not)."""
    from difflut_amd import _native as nat
    from difflut_amd import ops
    from difflut_amd.layers.random_layer import draw_mapping
    lib = nat.lib()
    torch.manual_seed(1)
    I, N, k = shape  # B = 4100: a last batch tile of four rows
    if mapping == "whole permutations":
        idx = draw_mapping(I, N, k, seed=7)
    else:
        idx = torch.randint(0, I, (N, k))
    plan = ops.MappingPlan(idx.to("cuda", torch.int32), I)
    x = torch.rand(B, I, device="cuda")
    luts = torch.rand(N, 1, 1 << k, device="cuda") * 2 - 1
    gy = torch.randn(B, N, device="cuda")
    dims = (B, I, N, k, 1)
    y = torch.empty(B, N, device="cuda")
    saved = torch.empty(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device="cuda")
    wf = torch.empty(lib.dl_dwn_fwd_workspace_bytes(*dims), dtype=torch.uint8, device="cuda")
    wb = torch.empty(lib.dl_dwn_bwd_workspace_bytes(*dims), dtype=torch.uint8, device="cuda")
    nat.check(lib.dl_dwn_layer_fwd(x.data_ptr(), plan.idx32.data_ptr(), luts.data_ptr(), y.data_ptr(), saved.data_ptr(),
                                   wf.data_ptr(), wf.numel(), *dims, nat.stream()))
    alpha = 0.5 * 0.75 ** 5  # beta = 0.9: the other form of the coefficient table (one row per slot)
    BT = (B + 63) // 64

    def backward(tiled):
        gx = torch.zeros(BT * 64 * I if tiled else B * I, device="cuda")
        gl = torch.empty_like(luts)
        nat.check(lib.dl_dwn_layer_bwd_tiled(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(),
                                             luts.data_ptr(), gy.data_ptr(), 0, alpha, beta, gx.data_ptr(), tiled, gl.data_ptr(),
                                             wb.data_ptr(), wb.numel(), *dims, nat.stream()))
        return gx, gl

    tiles, gl_t = backward(1)
    want = tiles.view(BT, I, 64).permute(0, 2, 1).reshape(BT * 64, I)[:B]
    for _ in range(3):
        rows, gl_r = backward(0)
        assert torch.equal(rows.view(B, I), want)
        if BT < 96:
            assert torch.equal(gl_r, gl_t)
        else:  # the same terms, grouped by chunk of rows: bins of about B / 64 values of size ~1
            torch.testing.assert_close(gl_r, gl_t, rtol=1e-5, atol=2e-5)
        del rows


def test_deep_stack_against_c_restatement_and_adam_step():
    REGISTRY, NodeConfig, _ = _api()
    from difflut_amd.layers import DWNStack
    from difflut_amd.utils import GroupSum, cross_entropy
    B, F, k = 8192, 784, 6
    widths = [16000, 8000, 4000, 2000]
    torch.manual_seed(0)
    x = torch.rand(B, F, device="cuda")
    labels = torch.randint(0, 10, (B,), device="cuda")
    # fitted on the host like the reference's CPU path (a device fit may contract min + j * step into one fma and
    # land one ulp away)
    enc = REGISTRY.build_encoder("thermometer", num_bits=4).fit(x.cpu())
    layers, width = [], F * 4
    for n in widths:
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=1), seed=42).cuda())
        width = n
    head = GroupSum(k=10, tau=1.0, use_randperm=False)
    stack = DWNStack(layers, encoder=enc, head=head).train()
    banks = [layer.bank_parameters()[0] for layer in layers]
    before = [b.detach().cpu().clone() for b in banks]
    opt = torch.optim.Adam(banks, lr=0.01)
    opt.zero_grad(set_to_none=True)
    logits = stack(x)
    loss = cross_entropy(logits, labels)
    loss.backward()
    got_gl = [b.grad.detach().cpu().numpy().copy() for b in banks]
    opt.step()
    after = [b.detach().cpu() for b in banks]

    # ---- the restatement, layer by layer on the host
    alpha, beta = np.float32(0.5 * 0.75 ** (k - 1)), np.float32(0.25 / 0.75)
    thr = orc.thermometer_fit(x.cpu().numpy(), 4)
    np.testing.assert_array_equal(thr, enc.thresholds.cpu().numpy())
    acts = [orc.thermometer_encode(x.cpu().numpy(), thr)]
    tabs = [t.numpy() for t in before]
    maps = [layer._mapping_indices.cpu().numpy().astype(np.int32) for layer in layers]
    for idx, tab in zip(maps, tabs):
        acts.append(c_oracle.dwn_layer_forward(acts[-1], idx, tab)[:, :, 0])
    want_logits = orc.group_sum(acts[-1], 10, 1.0)
    # sums of 200 table values of size <= 1 in another order
    np.testing.assert_allclose(logits.detach().cpu().numpy(), want_logits, rtol=1e-5, atol=2e-5)
    lt = torch.tensor(want_logits, dtype=torch.float64, requires_grad=True)
    want_loss = torch.nn.functional.cross_entropy(lt, labels.cpu())
    want_loss.backward()
    np.testing.assert_allclose(loss.item(), want_loss.item(), rtol=1e-5)
    g = np.repeat(lt.grad.numpy().astype(np.float32), widths[-1] // 10, axis=1)  # GroupSum backward, tau = 1
    want_gl = [None] * 4
    for li in range(3, -1, -1):
        g, want_gl[li] = c_oracle.dwn_layer_backward(acts[li], maps[li], tabs[li], g[:, :, None], alpha, beta)
    for li in range(4):
        scale = float(np.abs(want_gl[li]).max())
        # every bin adds ~B/64 = 128 terms; the floor is a few fp32 ulps of the largest bin
        np.testing.assert_allclose(got_gl[li], want_gl[li], rtol=1e-5, atol=4e-6 * scale, err_msg=f"layer {li}")

    # ---- one Adam(lr=0.01) step: torch's CPU Adam on the restatement's gradients
    cpu_params = [t.clone().requires_grad_() for t in before]
    cpu_opt = torch.optim.Adam(cpu_params, lr=0.01)
    for p, gl in zip(cpu_params, want_gl):
        p.grad = torch.from_numpy(gl.copy())
    cpu_opt.step()
    for li in range(4):
        got, want = after[li].numpy(), cpu_params[li].detach().numpy()
        assert not np.array_equal(got, before[li].numpy())
        # the first Adam step moves an entry by lr * g / (|g| + 1e-8): where |g| is far above 1e-8 that is +-lr for both
        # runs; entries whose gradient is within a few orders of 1e-8 may differ by a fraction of lr
        clear = np.abs(want_gl[li]) > 1e-5
        np.testing.assert_allclose(got[clear], want[clear], rtol=1e-5, atol=1e-6, err_msg=f"layer {li}")
        assert np.abs(got - want).max() <= 0.0101


def test_learnable_layer_full_size_against_restatements():
    REGISTRY, NodeConfig, _ = _api()
    B, I, N, k = 512, 3136, 8000, 6
    torch.manual_seed(3)
    layer = REGISTRY.get_layer("learnable")(I, N, REGISTRY.get_node("dwn"), NodeConfig(input_dim=k, output_dim=1),
                                            tau=1.0, tau_start=1.0, tau_min=1e-4, tau_decay_iters=1000,
                                            use_cuda_soft=False).cuda().train()
    with torch.no_grad():
        layer.mapping.W.normal_(0, 0.01)
    x = torch.rand(B, I, device="cuda", requires_grad=True)
    gy = torch.randn(B, N, device="cuda")
    out = layer(x)
    out.backward(gy)
    mapped = layer.get_mapping(x).detach().reshape(B, N * k)
    # soft connectivity against float64 softmax + matmul (learnable_layer.py:254-255)
    xd = x.detach().double().requires_grad_()
    Wd = layer.mapping.W.detach().double().requires_grad_()
    md = xd @ torch.softmax(Wd / 1.0, dim=-1).t()
    torch.testing.assert_close(mapped.double(), md.detach(), rtol=1e-5, atol=1e-6)
    # node stage on the device's own mapped values (thresholding is discontinuous)
    m_host = mapped.cpu().numpy()
    ident = np.arange(N * k, dtype=np.int32).reshape(N, k)
    luts = layer._banks["luts"].flat.detach().cpu().numpy()
    assert np.array_equal(out.detach().cpu().numpy(), c_oracle.dwn_layer_forward(m_host, ident, luts)[:, :, 0])
    gmap, gl = c_oracle.dwn_layer_backward(m_host, ident, luts, gy.cpu().numpy()[:, :, None],
                                           np.float32(0.5 * 0.75 ** (k - 1)), np.float32(0.25 / 0.75))
    np.testing.assert_allclose(layer._banks["luts"].flat.grad.cpu().numpy(), gl, rtol=1e-5, atol=1e-5)
    md.backward(torch.from_numpy(gmap).cuda().double())
    torch.testing.assert_close(x.grad.double(), xd.grad, rtol=1e-4, atol=2e-5 * float(xd.grad.abs().max()))
    torch.testing.assert_close(layer.mapping.W.grad.double(), Wd.grad, rtol=1e-4, atol=2e-5 * float(Wd.grad.abs().max()))
