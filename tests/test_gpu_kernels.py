"""GPU parity: every kernel family, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Integer/selection work (addresses, gathered values, table lookups, eval outputs,
thermometer bits, argmax) must be bit-exact; floating-point sums are held to rtol 1e-5 with an
absolute floor of a few fp32 ulps of the operand scale (stated per test)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _ops():
    from difflut_amd import ops
    return ops


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to(DEV, dtype)


def make_case(seed, B, I, N, k, O, lo=-1.0, hi=1.0, binary=False):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 2, (B, I)).astype(np.float32) if binary else rng.random((B, I)).astype(np.float32)
    idx = orc.random_mapping(I, N, k, seed=seed + 1).numpy().astype(np.int64)
    tab = rng.uniform(lo, hi, (N, O, 1 << k)).astype(np.float32)
    gy = rng.standard_normal((B, N, O)).astype(np.float32)
    return x, idx, tab, gy


DWN_SHAPES = [  # (B, I, N, k, O)
    (100, 25, 36, 6, 1),   # reference tests/test_layers/test_fused_kernels.py:26-36
    (10, 16, 25, 4, 1),    # test_fused_kernels.py:62-72
    (8, 256, 128, 4, 1),   # tests/test_layers/test_layer_functionality.py:37-55
    (70, 40, 33, 3, 2),
    (64, 128, 256, 6, 1),
    (130, 300, 77, 5, 3),
    (1, 7, 5, 1, 1),
    (322, 52, 80, 1, 1),   # k = 1: the S-form table (2 floats per node) is larger than the D form (1 float)
    (65, 9, 300, 2, 1),
    (200, 1030, 515, 6, 2),
    (9, 30, 11, 7, 2),     # k > 6: generic kernels
    (5, 64, 6, 9, 1),
    (21, 1031, 1100, 7, 1),  # k > 6 from 1024 columns on: the row of x through the LDS (odd width: scalar staging)
    (6, 512, 520, 8, 2),     # the same with two outputs per node
]


@pytest.mark.parametrize("shape", DWN_SHAPES)
def test_dwn_layer_forward_backward(shape):
    B, I, N, k, O = shape
    ops = _ops()
    x, idx, luts, gy = make_case(sum(shape), *shape)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_()
    lt = dev(luts).requires_grad_()
    alpha, beta = 0.5 * 0.75 ** (k - 1), 1.0 / 3.0
    y = ops.DWNLayerFunction.apply(xt, lt, plan, alpha, beta)
    want = orc.dwn_layer_forward(x, idx, luts).reshape(B, N * O)
    assert np.array_equal(y.detach().cpu().numpy(), want)  # bit exact
    y.backward(dev(gy.reshape(B, N * O)))
    gx, gl = orc.dwn_layer_backward(x, idx, luts, gy, np.float32(alpha), np.float32(beta))
    # gx sums <= fan-in terms of size alpha*|gy|*|D| ~ 0.1..1: rtol 1e-5, floor 2e-6
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    # table gradients are plain sums of gy over the rows that hit an entry
    np.testing.assert_allclose(lt.grad.cpu().numpy(), gl, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", [(33000, 50, 300, 6, 1), (40000, 7, 40, 2, 1)])
def test_dwn_backward_few_inputs_many_rows(shape):
    """Few inputs read by many nodes over many rows (the shape of the first level of a convolutional layer:
    CSR lists of ~36 entries per input, hundreds of batch tiles) against the C restatement on all rows."""
    B, I, N, k, O = shape
    ops = _ops()
    x, idx, luts, gy = make_case(sum(shape) % 1000, *shape)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    alpha, beta = 0.5 * 0.75 ** (k - 1), 1.0 / 3.0
    xt = dev(x).requires_grad_()
    lt = dev(luts).requires_grad_()
    y = ops.DWNLayerFunction.apply(xt, lt, plan, alpha, beta)
    y.backward(dev(gy.reshape(B, N * O)))
    assert np.array_equal(y.detach().cpu().numpy(), c_oracle.dwn_layer_forward(x, idx, luts).reshape(B, N * O))
    wx, wl = c_oracle.dwn_layer_backward(x, idx, luts, gy, alpha, beta)
    # up to N*k/I (~36) terms of size alpha*|gy|*|D| per input: rtol 1e-5, floor 5e-6
    np.testing.assert_allclose(xt.grad.cpu().numpy(), wx, rtol=1e-5, atol=5e-6)
    np.testing.assert_allclose(lt.grad.cpu().numpy(), wl, rtol=1e-5, atol=2e-4)  # ~B/2^k terms per bin


@pytest.mark.parametrize("shape", [(700, 20, 200, 6, 1), (130, 50, 64, 5, 1), (260, 9, 40, 6, 1), (65, 100, 50, 6, 1)])
def test_dwn_backward_tile_major_output_all_list_lengths(shape):
    """The tile-major form of the input gradient (what a chained layer or the fold of a convolutional layer
    reads) through the C entry point, for average CSR list lengths of 60, 6.4, 27 and 3: the gather runs with
    1, 4, 4 and 16 inputs per wavefront.  Every tile against the row-major result of the same call sequence
    and against the oracle."""
    from difflut_amd import _native as nat
    B, I, N, k, O = shape
    ops = _ops()
    lib = nat.lib()
    x, idx, luts, gy = make_case(sum(shape) % 997, *shape)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    alpha, beta = 0.5 * 0.75 ** (k - 1), 1.0 / 3.0
    dims = (B, I, N, k, O)
    xd, ld, gd = dev(x), dev(luts), dev(gy.reshape(B, N * O))
    y = torch.empty(B, N * O, device=DEV)
    saved = torch.empty(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device=DEV)
    wf = torch.empty(lib.dl_dwn_fwd_workspace_bytes(*dims), dtype=torch.uint8, device=DEV)
    wb = torch.empty(lib.dl_dwn_bwd_workspace_bytes(*dims), dtype=torch.uint8, device=DEV)
    nat.check(lib.dl_dwn_layer_fwd(xd.data_ptr(), plan.idx32.data_ptr(), ld.data_ptr(), y.data_ptr(), saved.data_ptr(),
                                   wf.data_ptr(), wf.numel(), *dims, nat.stream()))
    BT = (B + 63) // 64
    results = []
    for tiled in (0, 1):
        gx = torch.zeros(BT * I * 64 if tiled else B * I, device=DEV)
        gl = torch.empty_like(ld)
        nat.check(lib.dl_dwn_layer_bwd_tiled(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                             gd.data_ptr(), 0, alpha, beta, gx.data_ptr(), tiled, gl.data_ptr(), wb.data_ptr(),
                                             wb.numel(), *dims, nat.stream()))
        results.append((gx, gl))
    row_major = results[0][0].view(B, I)
    tile_major = results[1][0].view(BT, I, 64).permute(0, 2, 1).reshape(BT * 64, I)[:B]
    assert torch.equal(tile_major, row_major)  # same sums in the same order, another layout
    wx, wl = orc.dwn_layer_backward(x, idx, luts, gy, np.float32(alpha), np.float32(beta))
    np.testing.assert_allclose(row_major.cpu().numpy(), wx, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(results[1][1].cpu().numpy(), wl, rtol=1e-5, atol=2e-4)


FUSED_CHAIN_SHAPES = [  # (B, I0, k_front, I = nodes of the front layer, N, k)
    (200, 40, 6, 128, 64, 6),    # every input read three times: the unrolled path; fewer batch tiles than XCDs
    (1100, 64, 4, 256, 128, 6),  # 18 batch tiles: XCDs with three and with two; 16 bins per column
    (333, 30, 5, 100, 45, 5),    # lists of two and three entries, a last slab of 36 inputs
    (130, 16, 3, 20, 40, 6),     # twelve entries per input: four inputs per wavefront
    (64, 12, 6, 70, 35, 2),      # every input read once
    (150, 20, 4, 96, 32, 6),     # every input read twice
    (300, 16, 6, 48, 48, 6),     # every input read six times: four inputs per wavefront, unrolled
    (150, 16, 4, 24, 48, 6),     # twelve times
    (200, 24, 5, 64, 32, 6),     # three reads per input on average only (see the test)
]


@pytest.mark.parametrize("shape", FUSED_CHAIN_SHAPES)
def test_dwn_chained_backward_fills_the_table_gradient_of_the_layer_in_front(shape):
    """dl_dwn_layer_bwd_chain_fused against the two calls it replaces (the layer's own backward with a tile-major
    input gradient, then the front layer's histogram over that gradient) and against the oracle.  The input
    gradient and the layer's own table gradient keep their order of additions: bit-equal.  The front layer's
    bins are summed per block and then over blocks: rtol 1e-5 with a floor of 2e-5 of the largest bin."""
    from difflut_amd import _native as nat
    B, I0, kf, I, N, k = shape
    ops = _ops()
    lib = nat.lib()
    x0, idx_f, luts_f, _ = make_case(sum(shape) % 991, B, I0, I, kf, 1, lo=0.0)
    _, idx, luts, gy = make_case(sum(shape) % 983, B, I, N, k, 1)
    if shape == FUSED_CHAIN_SHAPES[-1]:
        # N k = 3 I, but drawn independently: the lists are uneven although the host sees a whole fan-in
        idx = np.random.default_rng(5).integers(0, I, (N, k)).astype(np.int64)
    plan_f = ops.MappingPlan(dev(idx_f, torch.int32), I0)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    front, dims = (B, I0, I, kf, 1), (B, I, N, k, 1)
    rng = np.random.default_rng(7)
    alpha_n = dev(rng.uniform(0.1, 0.6, N).astype(np.float32))
    beta_n = dev(rng.uniform(-0.4, 0.45, N).astype(np.float32))
    beta_max = float(beta_n.abs().max())

    def forward(xin, pl, tab, d):
        y = torch.empty(d[0], d[2], device=DEV)
        saved = torch.empty(lib.dl_dwn_saved_bytes(*d), dtype=torch.uint8, device=DEV)
        ws = torch.empty(lib.dl_dwn_fwd_workspace_bytes(*d), dtype=torch.uint8, device=DEV)
        nat.check(lib.dl_dwn_layer_fwd(xin.data_ptr(), pl.idx32.data_ptr(), tab.data_ptr(), y.data_ptr(), saved.data_ptr(),
                                       ws.data_ptr(), ws.numel(), *d, nat.stream()))
        return y, saved

    lf, ld, gd = dev(luts_f), dev(luts), dev(gy.reshape(B, N))
    h, saved_f = forward(dev(x0), plan_f, lf, front)
    _, saved = forward(h, plan, ld, dims)
    BT = (B + 63) // 64
    assert lib.dl_dwn_chain_fusable(*dims, kf, beta_max) == 1
    # the two calls
    ws = torch.empty(lib.dl_dwn_bwd_workspace_bytes(*dims), dtype=torch.uint8, device=DEV)
    gx_ref = torch.zeros(BT * I * 64, device=DEV)
    gl_ref = torch.empty_like(ld)
    nat.check(lib.dl_dwn_layer_bwd_chain_nodes(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                               gd.data_ptr(), 0, 1, 1.0, alpha_n.data_ptr(), beta_n.data_ptr(), beta_max,
                                               gx_ref.data_ptr(), 1, gl_ref.data_ptr(), ws.data_ptr(), ws.numel(), *dims,
                                               nat.stream()))
    wsf = torch.empty(lib.dl_dwn_bwd_workspace_bytes(*front), dtype=torch.uint8, device=DEV)
    glf_ref = torch.empty_like(lf)
    nat.check(lib.dl_dwn_layer_bwd_tiled(saved_f.data_ptr(), None, None, lf.data_ptr(), gx_ref.data_ptr(), 1, 0.3, 0.3, None, 0,
                                         glf_ref.data_ptr(), wsf.data_ptr(), wsf.numel(), *front, nat.stream()))
    # the one call
    wsx = torch.empty(lib.dl_dwn_bwd_fused_workspace_bytes(*dims, kf), dtype=torch.uint8, device=DEV)
    gx = torch.zeros(BT * I * 64, device=DEV)
    gl = torch.empty_like(ld)
    glf = torch.full_like(lf, 7.0)
    nat.check(lib.dl_dwn_layer_bwd_chain_fused(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                               gd.data_ptr(), 0, 1, 1.0, alpha_n.data_ptr(), beta_n.data_ptr(), beta_max,
                                               gx.data_ptr(), 1, gl.data_ptr(), saved_f.data_ptr(), kf, glf.data_ptr(),
                                               wsx.data_ptr(), wsx.numel(), *dims, nat.stream()))
    assert torch.equal(gx, gx_ref)
    assert torch.equal(gl, gl_ref)
    floor = 2e-5 * float(glf_ref.abs().max())
    np.testing.assert_allclose(glf.cpu().numpy(), glf_ref.cpu().numpy(), rtol=1e-5, atol=floor)
    # the oracle on the front layer, fed with the input gradient just computed (rows past B carry zeros)
    rows = gx.view(BT, I, 64).permute(0, 2, 1).reshape(BT * 64, I)[:B].cpu().numpy()
    _, want = orc.dwn_layer_backward(x0, idx_f, luts_f, rows.reshape(B, I, 1), np.float32(0.3), np.float32(0.3))
    np.testing.assert_allclose(glf.cpu().numpy(), want, rtol=1e-5, atol=floor)
    # the layer's own table gradient already there: gy tile-major, no gluts
    gyT = torch.zeros(BT * 64, N, device=DEV)
    gyT[:B] = gd
    gyT = gyT.view(BT, 64, N).permute(0, 2, 1).contiguous()
    gx2 = torch.zeros_like(gx)
    glf2 = torch.empty_like(lf)
    nat.check(lib.dl_dwn_layer_bwd_chain_fused(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                               gyT.data_ptr(), 1, 1, 1.0, alpha_n.data_ptr(), beta_n.data_ptr(), beta_max,
                                               gx2.data_ptr(), 1, None, saved_f.data_ptr(), kf, glf2.data_ptr(),
                                               wsx.data_ptr(), wsx.numel(), *dims, nat.stream()))
    assert torch.equal(gx2, gx_ref)
    assert torch.equal(glf2, glf)  # fixed order of additions: the same bits on every call
    # no buffer for the input gradient (nobody behind the front layer reads it): the same bins, the same bits, and the
    # layer's own table gradient as before
    glf4, gl4 = torch.empty_like(lf), torch.empty_like(ld)
    nat.check(lib.dl_dwn_layer_bwd_chain_fused(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                               gd.data_ptr(), 0, 1, 1.0, alpha_n.data_ptr(), beta_n.data_ptr(), beta_max,
                                               None, 1, gl4.data_ptr(), saved_f.data_ptr(), kf, glf4.data_ptr(),
                                               wsx.data_ptr(), wsx.numel(), *dims, nat.stream()))
    assert torch.equal(glf4, glf) and torch.equal(gl4, gl_ref)
    # and without a front layer it is the plain chained backward
    gx3 = torch.zeros_like(gx)
    nat.check(lib.dl_dwn_layer_bwd_chain_fused(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                               gyT.data_ptr(), 1, 1, 1.0, alpha_n.data_ptr(), beta_n.data_ptr(), beta_max,
                                               gx3.data_ptr(), 1, None, None, 0, None, ws.data_ptr(), ws.numel(), *dims,
                                               nat.stream()))
    assert torch.equal(gx3, gx_ref)


def test_dwn_chained_backward_refuses_what_it_cannot_fuse():
    from difflut_amd import _native as nat
    lib = nat.lib()
    assert lib.dl_dwn_chain_fusable(64, 9, 64, 6, 1, 6, 0.3) == 0    # 42 entries per input: the one-input gather
    assert lib.dl_dwn_chain_fusable(64, 128, 64, 6, 1, 6, 0.75) == 0  # |beta| > 1/2: the other coefficient form
    assert lib.dl_dwn_chain_fusable(64, 128, 64, 6, 2, 6, 0.3) == 0   # two outputs per node
    assert lib.dl_dwn_chain_fusable(64, 128, 64, 6, 1, 7, 0.3) == 0   # front layer on the generic path
    assert lib.dl_dwn_chain_fusable(64, 128, 64, 6, 1, 4, 0.3) == 1
    buf = torch.zeros(1 << 16, device=DEV)
    rc = lib.dl_dwn_layer_bwd_chain_fused(buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), 0, 1,
                                          1.0, buf.data_ptr(), buf.data_ptr(), 0.75, buf.data_ptr(), 1, buf.data_ptr(),
                                          buf.data_ptr(), 6, buf.data_ptr(), buf.data_ptr(), buf.numel() * 4, 64, 128, 64, 6, 1,
                                          nat.stream())
    assert rc == -3  # DL_ERR_UNSUPPORTED


@pytest.mark.parametrize("shape", [(300, 12, 128, 6, 1), (1300, 7, 80, 6, 1), (90, 5, 64, 5, 1)])
def test_dwn_backward_tile_major_output_uneven_long_lists(shape):
    """Inputs read by 40 to 90 nodes each, drawn independently (lists of very different lengths, some beyond what the
    gather for long lists keeps in registers): the tile-major input gradient against the row-major one of the same
    entry point (same terms in the same order: bit-equal) and against the oracle."""
    from difflut_amd import _native as nat
    B, I, N, k, O = shape
    ops = _ops()
    lib = nat.lib()
    rng = np.random.default_rng(sum(shape))
    x = rng.random((B, I)).astype(np.float32)
    idx = rng.integers(0, I, (N, k)).astype(np.int64)
    idx[:, 0] = np.where(rng.random(N) < 0.5, 0, idx[:, 0])  # input 0 is read far more often than the others
    luts = rng.uniform(-1, 1, (N, O, 1 << k)).astype(np.float32)
    gy = rng.standard_normal((B, N, O)).astype(np.float32)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    alpha, beta = 0.5 * 0.75 ** (k - 1), 1.0 / 3.0
    dims = (B, I, N, k, O)
    xd, ld, gd = dev(x), dev(luts), dev(gy.reshape(B, N * O))
    y = torch.empty(B, N * O, device=DEV)
    saved = torch.empty(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device=DEV)
    wf = torch.empty(lib.dl_dwn_fwd_workspace_bytes(*dims), dtype=torch.uint8, device=DEV)
    wb = torch.empty(lib.dl_dwn_bwd_workspace_bytes(*dims), dtype=torch.uint8, device=DEV)
    nat.check(lib.dl_dwn_layer_fwd(xd.data_ptr(), plan.idx32.data_ptr(), ld.data_ptr(), y.data_ptr(), saved.data_ptr(),
                                   wf.data_ptr(), wf.numel(), *dims, nat.stream()))
    BT = (B + 63) // 64
    results = []
    for tiled in (0, 1):
        gx = torch.zeros(BT * I * 64 if tiled else B * I, device=DEV)
        gl = torch.empty_like(ld)
        nat.check(lib.dl_dwn_layer_bwd_tiled(saved.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), ld.data_ptr(),
                                             gd.data_ptr(), 0, alpha, beta, gx.data_ptr(), tiled, gl.data_ptr(), wb.data_ptr(),
                                             wb.numel(), *dims, nat.stream()))
        results.append((gx, gl))
    row_major = results[0][0].view(B, I)
    tile_major = results[1][0].view(BT, I, 64).permute(0, 2, 1).reshape(BT * 64, I)[:B]
    assert torch.equal(tile_major, row_major)
    assert torch.equal(results[0][1], results[1][1])
    wx, wl = orc.dwn_layer_backward(x, idx, luts, gy, np.float32(alpha), np.float32(beta))
    # up to ~100 terms of size alpha*|gy|*|D| per input: rtol 1e-5, floor 2e-5
    np.testing.assert_allclose(row_major.cpu().numpy(), wx, rtol=1e-5, atol=2e-5)
    np.testing.assert_allclose(results[1][1].cpu().numpy(), wl, rtol=1e-5, atol=2e-4)


def test_dwn_threshold_is_inclusive_and_exact_at_half():
    ops = _ops()
    x = np.array([[0.5, 0.49999997, 0.50000006, 0.0, 1.0, -3.0]], dtype=np.float32)
    idx = np.arange(6)[None]
    luts = np.arange(64, dtype=np.float32)[None, None]
    plan = ops.MappingPlan(dev(idx, torch.int32), 6)
    y = ops.DWNLayerFunction.apply(dev(x), dev(luts), plan, 0.1, 0.3)
    assert y.item() == float(0b010101)


@pytest.mark.parametrize("beta", [0.0, 1.0, 0.9])
def test_dwn_backward_other_alpha_beta(beta):
    ops = _ops()
    shape = (33, 20, 17, 4, 2)
    x, idx, luts, gy = make_case(5, *shape)
    B, I, N, k, O = shape
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_(); lt = dev(luts).requires_grad_()
    ops.DWNLayerFunction.apply(xt, lt, plan, 0.7, beta).backward(dev(gy.reshape(B, -1)))
    gx, gl = orc.dwn_layer_backward(x, idx, luts, gy, np.float32(0.7), np.float32(beta))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(lt.grad.cpu().numpy(), gl, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("beta", [1.0 / 3.0, -0.5, 0.9])
@pytest.mark.parametrize("shape", [(70, 40, 25, 8, 1), (33, 24, 9, 7, 2), (20, 64, 5, 10, 1)])
def test_dwn_backward_more_than_six_inputs(shape, beta):
    """k > 6: the input gradient from tables smoothed once per call (|beta| <= 1/2) and from the 2^k-term sum
    (beta = 0.9), both against the oracle; the smoothed form amplifies rounding by (1 + |beta|)^k / (1 - beta) <= 52,
    hence rtol 1e-5 with a floor of 2e-5."""
    ops = _ops()
    B, I, N, k, O = shape
    x, idx, luts, gy = make_case(sum(shape), *shape)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_(); lt = dev(luts).requires_grad_()
    y = ops.DWNLayerFunction.apply(xt, lt, plan, 0.3, beta)
    assert np.array_equal(y.detach().cpu().numpy().reshape(B, N, O), orc.dwn_layer_forward(x, idx, luts))
    y.backward(dev(gy.reshape(B, -1)))
    gx, gl = orc.dwn_layer_backward(x, idx, luts, gy, np.float32(0.3), np.float32(beta))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-5 * max(1.0, float(np.abs(gx).max())))
    np.testing.assert_allclose(lt.grad.cpu().numpy(), gl, rtol=1e-5, atol=1e-5)


def test_dwn_no_input_grad_and_unused_inputs():
    ops = _ops()
    B, I, N, k, O = 40, 50, 3, 2, 1  # 44 of the 50 inputs feed no node: their gradient must be 0
    x, idx, luts, gy = make_case(11, B, I, N, k, O)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    lt = dev(luts).requires_grad_()
    ops.DWNLayerFunction.apply(dev(x), lt, plan, 0.2, 0.3).backward(dev(gy.reshape(B, -1)))
    _, gl = orc.dwn_layer_backward(x, idx, luts, gy, np.float32(0.2), np.float32(0.3))
    np.testing.assert_allclose(lt.grad.cpu().numpy(), gl, rtol=1e-5, atol=1e-5)
    xt = dev(x).requires_grad_()
    ops.DWNLayerFunction.apply(xt, dev(luts), plan, 0.2, 0.3).backward(dev(gy.reshape(B, -1)))
    unused = np.setdiff1d(np.arange(I), idx.reshape(-1))
    assert np.all(xt.grad.cpu().numpy()[:, unused] == 0.0)


@pytest.mark.parametrize("shape", [(12, 20, 9, 6, 2), (70, 33, 140, 3, 1), (4, 30, 5, 8, 1)])
def test_dwn_eval_forward(shape):
    ops = _ops()
    B, I, N, k, O = shape
    x, idx, luts, _ = make_case(3, *shape, lo=0.0, hi=1.0, binary=True)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    y = ops.dwn_layer_eval(dev(x), dev(luts), plan).cpu().numpy().reshape(B, N, O)
    m = orc.gather_forward(x, idx)
    for n in range(N):
        assert np.array_equal(y[:, n], orc.dwn_eval_forward(m[:, n], luts[n]))


@pytest.mark.parametrize("shape", [(130, 40, 150, 6, 1), (64, 36, 70, 4, 2), (257, 33, 129, 5, 1),
                                   # from 1024 columns on the literal-address kernel stages the row of x in the LDS:
                                   # odd widths, two outputs per node, two windows of columns
                                   (37, 1031, 1100, 5, 1), (5, 300, 600, 3, 2), (9, 4096, 9000, 6, 1)])
def test_dwn_eval_forward_any_input_values(shape):
    """The eval entry point with a workspace answers through the bit-plane kernels when every input is 0 or 1 and
    through the literal float address otherwise; both against the oracle, including inputs where the two
    addresses differ (0.7 counts as 0.7 * 2^j, not as a set bit) and a single odd value in a binary batch."""
    ops = _ops()
    B, I, N, k, O = shape
    xb, idx, luts, _ = make_case(11, *shape, lo=0.0, hi=1.0, binary=True)
    rng = np.random.default_rng(5)
    xf = rng.random((B, I)).astype(np.float32) * 1.2          # arbitrary values, some above 1
    xo = xb.copy()
    xo[B // 2, idx[N // 2, 0]] = 0.25                          # one value that is neither 0 nor 1
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    for x in (xb, xf, xo, xb):                                 # the flag is reset on every call
        y = ops.dwn_layer_eval(dev(x), dev(luts), plan).cpu().numpy().reshape(B, N, O)
        m = orc.gather_forward(x, idx)
        L = 1 << k
        for n in range(N):
            addr = (m[:, n] * (2.0 ** np.arange(k)).astype(np.float32)).sum(-1, dtype=np.float32).astype(np.int64)
            want = (luts[n][:, np.clip(addr, 0, L - 1)].T >= np.float32(0.5)).astype(np.float32)  # clamped like the kernel
            assert np.array_equal(y[:, n], want)
            if x is not xf:
                assert np.array_equal(want, orc.dwn_eval_forward(m[:, n], luts[n]))


@pytest.mark.parametrize("shape", [(130, 40, 150, 4, 1), (64, 36, 70, 6, 2), (200, 33, 90, 3, 1),
                                   # from 1024 columns on both literal-address kernels stage the row of x in the LDS
                                   (33, 1031, 1100, 4, 1), (7, 300, 520, 6, 2)])
def test_prob_eval_forward_any_input_values(shape):
    """Probabilistic eval through the workspace entry point (binarised sigmoid table looked up by the DWN eval
    path) against the oracle, for 0/1 inputs (bit-plane kernels), arbitrary inputs and a single odd value
    (generic kernel), and against the entry point without a workspace."""
    from difflut_amd import _native as nat
    ops = _ops()
    B, I, N, k, O = shape
    rng = np.random.default_rng(21)
    idx = orc.random_mapping(I, N, k, seed=4).numpy().astype(np.int64)
    raw = rng.standard_normal((N, 1 << k, O)).astype(np.float32)
    raw[0, 0, 0] = 0.0                                         # sigmoid(0) = 0.5 counts as 1
    xb = rng.integers(0, 2, (B, I)).astype(np.float32)
    xf = rng.random((B, I)).astype(np.float32)
    xo = xb.copy()
    xo[3, idx[1, 0]] = 0.5
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    lib = nat.lib()
    rawd = dev(raw)
    for x in (xb, xf, xo):
        xd = dev(x)
        y = ops.prob_layer_eval(xd, rawd, plan, 0.7)
        plain = torch.empty_like(y)
        nat.check(lib.dl_prob_layer_eval(xd.data_ptr(), plan.idx32.data_ptr(), rawd.data_ptr(), 0.7, plain.data_ptr(),
                                         B, I, N, k, O, nat.stream()))
        assert torch.equal(y, plain)
        m = orc.gather_forward(x, idx)
        got = y.cpu().numpy().reshape(B, N, O)
        for n in range(N):
            assert np.array_equal(got[:, n], orc.prob_eval_forward(m[:, n], raw[n], 0.7))


@pytest.mark.parametrize("tag", ["k6o2", "k4o1", "k2o3"])
def test_dwn_node_against_reference_vectors(golden, tag):
    """Same inputs the reference's own CPU path was run on (tests/golden)."""
    from difflut_amd.nodes.dwn_node import efd_forward

    g = golden
    a, b = (float(v) for v in g[f"dwn_{tag}_ab"])
    xt = dev(g[f"dwn_{tag}_x"]).requires_grad_()
    lt = dev(g[f"dwn_{tag}_luts"]).requires_grad_()
    y = efd_forward(xt, lt, a, b)
    assert np.array_equal(y.detach().cpu().numpy(), g[f"dwn_{tag}_y"])
    y.backward(dev(g[f"dwn_{tag}_gy"]))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), g[f"dwn_{tag}_gx"], rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(lt.grad.cpu().numpy(), g[f"dwn_{tag}_gl"], rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------------------ gather
@pytest.mark.parametrize("dtype", [torch.int16, torch.int32])
def test_gather_forward_backward(dtype):
    ops = _ops()
    B, I, N, k = 37, 211, 90, 5
    rng = np.random.default_rng(0)
    x = rng.standard_normal((B, I)).astype(np.float32)
    idx = orc.random_mapping(I, N, k, seed=9).numpy().astype(np.int64)
    it = dev(idx, dtype)
    xt = dev(x).requires_grad_()
    m = ops.GatherFunction.apply(xt, it, ops.MappingPlan(it, I))
    assert np.array_equal(m.detach().cpu().numpy(), orc.gather_forward(x, idx))
    gm = rng.standard_normal((B, N, k)).astype(np.float32)
    m.backward(dev(gm))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), orc.gather_backward(gm, idx, I), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(70, 1031, 700, 6, torch.int16),      # 4200 connections: one piece, odd widths (scalar staging)
                                   (33, 3136, 2000, 6, torch.int16),     # cfg 1's layer: lists of three and four
                                   (25, 4096, 4096, 4, torch.int32),     # whole permutations, four inputs per thread
                                   (9, 16384, 8192, 6, torch.int32),     # two pieces per row, sixteen inputs per thread
                                   (5, 20001, 9000, 5, torch.int32),     # two windows of inputs, pieces of odd length
                                   (3, 300, 48000, 1, torch.int32)])     # hard selection's shape: long lists, one input each
def test_gather_through_the_lds(shape):
    """From 4096 connections on the row that is read at random (x forward, gm backward) is staged in the LDS.  The
    forward is a copy: exact.  The backward adds a list in its order, like the oracle's loop: exact as well."""
    ops = _ops()
    B, I, N, k, dtype = shape
    rng = np.random.default_rng(I + N)
    x = rng.standard_normal((B, I)).astype(np.float32)
    idx = orc.random_mapping(I, N, k, seed=5).numpy().astype(np.int64)
    it = dev(idx, dtype)
    xt = dev(x).requires_grad_()
    m = ops.GatherFunction.apply(xt, it, ops.MappingPlan(it, I))
    assert np.array_equal(m.detach().cpu().numpy(), x[:, idx])
    gm = rng.standard_normal((B, N, k)).astype(np.float32)
    m.backward(dev(gm))
    want = np.zeros((B, I), np.float32)
    flat = gm.reshape(B, -1)
    for p, i in enumerate(idx.reshape(-1)):  # ascending position within every input: the order of the CSR lists
        want[:, i] += flat[:, p]
    assert np.array_equal(xt.grad.cpu().numpy(), want)


# ------------------------------------------------------------------------------ probabilistic
PROB_SHAPES = [(32, 40, 24, 4, 2), (64, 128, 300, 4, 1), (17, 30, 9, 6, 1), (20, 9, 5, 1, 1), (10, 50, 7, 2, 3),
               (6, 40, 5, 7, 2), (200, 300, 260, 4, 1), (130, 70, 33, 5, 2), (65, 1000, 515, 3, 1),
               (300, 20, 3, 4, 1)]   # last: few nodes, many batch tiles -> several table-gradient chunks


@pytest.mark.parametrize("shape", PROB_SHAPES)
@pytest.mark.parametrize("T", [1.0, 0.5])
def test_prob_layer_forward_backward(shape, T):
    ops = _ops()
    B, I, N, k, O = shape
    rng = np.random.default_rng(sum(shape))
    x = (1 / (1 + np.exp(-rng.standard_normal((B, I))))).astype(np.float32)
    idx = orc.random_mapping(I, N, k, seed=4).numpy().astype(np.int64)
    raw = rng.uniform(0, 1, (N, 1 << k, O)).astype(np.float32)
    gy = rng.standard_normal((B, N, O)).astype(np.float32)
    plan = ops.MappingPlan(dev(idx, torch.int32), I)
    xt = dev(x).requires_grad_(); wt = dev(raw).requires_grad_()
    y = ops.ProbLayerFunction.apply(xt, wt, plan, T)
    want = orc.prob_layer_forward(x, idx, raw, T, dtype=torch.float64).reshape(B, N * O)
    np.testing.assert_allclose(y.detach().cpu().numpy(), want, rtol=1e-5, atol=1e-6)  # outputs lie in (0,1)
    y.backward(dev(gy.reshape(B, -1)))
    gx, gw = orc.prob_layer_backward(x, idx, raw, gy, T)
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(wt.grad.cpu().numpy(), gw, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("tag", ["k4o2", "k6o1"])
def test_prob_node_against_reference_vectors(golden, tag):
    from difflut_amd.nodes.probabilistic_node import probabilistic_forward
    ops = _ops()

    g = golden
    T = float(g[f"prob_{tag}_T"][0])
    xt = dev(g[f"prob_{tag}_x"]).requires_grad_()
    wt = dev(g[f"prob_{tag}_w"]).requires_grad_()
    y = probabilistic_forward(xt, wt, T)
    np.testing.assert_allclose(y.detach().cpu().numpy(), g[f"prob_{tag}_y"], rtol=1e-5, atol=1e-6)
    y.backward(dev(g[f"prob_{tag}_gy"]))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), g[f"prob_{tag}_gx"], rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(wt.grad.cpu().numpy(), g[f"prob_{tag}_gw"], rtol=1e-5, atol=2e-6)
    k = g[f"prob_{tag}_x"].shape[1]
    plan = ops.MappingPlan.identity(k, DEV)
    ye = ops.prob_layer_eval(dev(g[f"prob_{tag}_eval_x"]), wt.detach().unsqueeze(0), plan, T)
    assert np.array_equal(ye.cpu().numpy(), g[f"prob_{tag}_eval_y"])


# ------------------------------------------------------------------------------ learnable mapping
@pytest.mark.parametrize("shape,tau", [((5, 20, 21), 1.0), ((70, 130, 200), 0.3), ((64, 64, 64), 1.0),
                                       ((33, 257, 18), 0.05), ((256, 384, 1000), 1.0),
                                       ((130, 260, 516), 0.5), ((129, 132, 4100), 2.0)])
def test_soft_mapping_forward_backward_fp32(shape, tau):
    ops = _ops()
    B, I, M = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.random((B, I)).astype(np.float32)
    W = (rng.standard_normal((M, I)) * 0.5).astype(np.float32)
    gm = rng.standard_normal((B, M)).astype(np.float32)
    xt = dev(x).requires_grad_(); Wt = dev(W).requires_grad_()
    m = ops.SoftMapFunction.apply(xt, Wt, tau, 0)
    np.testing.assert_allclose(m.detach().cpu().numpy(), orc.soft_mapping_forward(x, W, tau, torch.float64),
                               rtol=1e-5, atol=1e-6)  # m is a convex mix of inputs in [0,1)
    m.backward(dev(gm))
    gx, gW = orc.soft_mapping_backward(x, W, gm, tau)
    np.testing.assert_allclose(xt.grad.cpu().numpy(), gx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(Wt.grad.cpu().numpy(), gW, rtol=1e-4, atol=1e-5 / tau)


@pytest.mark.parametrize("shape,tau", [((5, 20, 21), 1.0), ((256, 384, 1000), 1.0), ((130, 260, 516), 0.5),
                                       ((129, 132, 4100), 2.0), ((128, 256, 384), 1.0)])
def test_soft_mapping_bf16_operands(shape, tau):
    """precision=1 rounds x, S and gm to bf16 (8 significant bits, relative step 2^-8) before the
    MFMA and accumulates in fp32.  Tolerance: 1e-2 of the largest reference magnitude per tensor
    (rounding errors of the summands are independent, so the sums do better than 2^-8)."""
    ops = _ops()
    B, I, M = shape
    rng = np.random.default_rng(sum(shape) + 1)
    x = rng.random((B, I)).astype(np.float32)
    W = (rng.standard_normal((M, I)) * 0.5).astype(np.float32)
    gm = rng.standard_normal((B, M)).astype(np.float32)
    xt = dev(x).requires_grad_(); Wt = dev(W).requires_grad_()
    m = ops.SoftMapFunction.apply(xt, Wt, tau, 1)
    want_m = orc.soft_mapping_forward(x, W, tau, torch.float64)
    got_m = m.detach().cpu().numpy()
    assert np.abs(got_m - want_m).max() <= 1e-2 * np.abs(want_m).max()
    assert np.abs(got_m - want_m).max() > 0  # the bf16 path ran, not the fp32 one
    m.backward(dev(gm))
    gx, gW = orc.soft_mapping_backward(x, W, gm, tau)
    assert np.abs(xt.grad.cpu().numpy() - gx).max() <= 1e-2 * np.abs(gx).max()
    assert np.abs(Wt.grad.cpu().numpy() - gW).max() <= 1e-2 * np.abs(gW).max()


def test_soft_and_hard_mapping_against_reference_vectors(golden):
    ops = _ops()
    g = golden
    for tau_key, mk, gxk, gWk in [("soft_tau", "soft_m", "soft_gx", "soft_gW"),
                                  ("soft_tau_500", "soft500_m", "soft500_gx", "soft500_gW")]:
        tau = float(g[tau_key][0])
        xt = dev(g["soft_x"]).requires_grad_(); Wt = dev(g["soft_W"]).requires_grad_()
        m = ops.SoftMapFunction.apply(xt, Wt, tau, 0)
        np.testing.assert_allclose(m.detach().cpu().numpy(), g[mk].reshape(5, -1), rtol=1e-5, atol=1e-6)
        m.backward(dev(g["soft_gm"].reshape(5, -1)))
        np.testing.assert_allclose(xt.grad.cpu().numpy(), g[gxk], rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(Wt.grad.cpu().numpy(), g[gWk], rtol=1e-4, atol=1e-5)
    sel = ops.row_argmax(dev(g["soft_W"]))
    assert np.array_equal(sel.cpu().numpy().reshape(7, 3), g["hard_idx"])
    plan = ops.MappingPlan(sel.view(-1, 1), 20)
    xt = dev(g["soft_x"]).requires_grad_()
    hm = ops.HardSelectFunction.apply(xt, sel, plan)
    assert np.array_equal(hm.detach().cpu().numpy(), g["hard_m"].reshape(5, -1))
    gm = np.random.default_rng(1).standard_normal(hm.shape).astype(np.float32)
    hm.backward(dev(gm))
    want = orc.gather_backward(gm[:, :, None], sel.cpu().numpy().reshape(-1, 1), 20)
    np.testing.assert_allclose(xt.grad.cpu().numpy(), want, rtol=1e-6, atol=1e-6)


def test_row_argmax_ties_and_sizes():
    ops = _ops()
    rng = np.random.default_rng(2)
    W = rng.standard_normal((300, 1000)).astype(np.float32)
    W[5, 17] = W[5, 900] = 9.0   # tie: lowest index wins
    W[6, :] = -1.0
    sel = ops.row_argmax(dev(W)).cpu().numpy()
    assert np.array_equal(sel, W.argmax(1)) and sel[5] == 17 and sel[6] == 0
    # widths that are no multiple of four (one value per lane and load), of four but not of 1024 (a tail of 16-byte
    # loads), and a tie that straddles two lanes' pieces
    for M, I in ((9, 1031), (5, 2052), (7, 4096), (3, 12)):
        W = rng.standard_normal((M, I)).astype(np.float32)
        W[1, I - 1] = W[1, 2] = 7.0
        W[2, :] = 0.5
        sel = ops.row_argmax(dev(W)).cpu().numpy()
        assert np.array_equal(sel, W.argmax(1)) and sel[1] == 2 and sel[2] == 0


# ------------------------------------------------------------------------------ encoder / head
def test_thermometer_and_group_sum(golden):
    ops = _ops()
    g = golden
    bits = ops.thermometer_encode(dev(g["thermo_x"]), dev(g["thermo_thr"]))
    assert np.array_equal(bits.cpu().numpy().reshape(9, -1), g["thermo_bits"])
    xt = dev(g["groupsum_x"]).requires_grad_()
    y = ops.GroupSumFunction.apply(xt, 5, 2.0)
    np.testing.assert_allclose(y.detach().cpu().numpy(), g["groupsum_y"], rtol=1e-6, atol=1e-6)
    gy = np.random.default_rng(0).standard_normal((6, 5)).astype(np.float32)
    y.backward(dev(gy))
    np.testing.assert_allclose(xt.grad.cpu().numpy(), np.repeat(gy, 4, 1) / 2.0, rtol=1e-6)
    # rows of bits that are and are not a multiple of four values (16-byte stores or one value at a time), strict compare
    for B, F, nb in ((7, 5, 3), (64, 12, 4), (3, 6, 2), (130, 784, 4), (5, 1, 1)):
        rs = np.random.default_rng(B * F + nb)
        xs = rs.random((B, F)).astype(np.float32)
        th = np.sort(rs.random((F, nb)).astype(np.float32), axis=1)
        xs[0, 0] = th[0, 0]  # equal to a threshold: not above it
        got = ops.thermometer_encode(dev(xs), dev(th)).cpu().numpy().reshape(B, F, nb)
        assert np.array_equal(got, (xs[:, :, None] > th[None]).astype(np.float32))
    x = np.random.default_rng(1).standard_normal((3, 10)).astype(np.float32)  # 10 features, 4 groups: padded
    y = ops.GroupSumFunction.apply(dev(x), 4, 1.0)
    np.testing.assert_allclose(y.cpu().numpy(), orc.group_sum(x, 4, 1.0), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(8192, 10), (1, 3), (257, 1), (1000, 64), (33, 300)])
def test_cross_entropy_against_torch(shape):
    """Fused mean cross-entropy and its gradient against torch's own (float64 on the CPU): loss to rtol 1e-6,
    gradient to rtol 1e-5 with a floor of 1e-9 (entries are (softmax - onehot) / B); large logits do not overflow;
    a row with a label outside the classes adds nothing."""
    from difflut_amd.utils import cross_entropy
    B, C = shape
    rng = np.random.default_rng(B + C)
    z = (rng.standard_normal((B, C)) * 4).astype(np.float32)
    z[0, 0] = 90.0                                        # exp(90) overflows fp32 without the max shift
    y = rng.integers(0, C, (B,))
    zt = dev(z).requires_grad_()
    loss = cross_entropy(zt, torch.as_tensor(y, device=DEV))
    (loss * 3.0).backward()
    zr = torch.tensor(z, dtype=torch.float64, requires_grad=True)
    want = torch.nn.functional.cross_entropy(zr, torch.as_tensor(y))
    (want * 3.0).backward()
    np.testing.assert_allclose(loss.item(), want.item(), rtol=1e-6)
    np.testing.assert_allclose(zt.grad.cpu().numpy(), zr.grad.numpy(), rtol=1e-5, atol=1e-9)
    if B > 1:
        y2 = y.copy()
        y2[1] = C + 5
        l2 = cross_entropy(dev(z), torch.as_tensor(y2, device=DEV))
        keep = np.ones(B, bool); keep[1] = False
        ref = torch.nn.functional.cross_entropy(torch.tensor(z[keep], dtype=torch.float64), torch.as_tensor(y[keep]), reduction="sum") / B
        np.testing.assert_allclose(l2.item(), ref.item(), rtol=1e-6)


# ------------------------------------------------------------------------------ error paths
def test_argument_errors_are_reported_not_launched():
    from difflut_amd import _native as nat
    lib = nat.lib()
    assert lib.dl_dwn_layer_fwd(None, None, None, None, None, None, 0, 1, 1, 1, 1, 1, None) == -1
    t = torch.zeros(64, device=DEV)
    p = t.data_ptr()
    assert lib.dl_dwn_layer_fwd(p, p, p, p, p, p, 0, 4, 4, 4, 2, 1, None) == -4   # workspace too small
    assert lib.dl_dwn_layer_fwd(p, p, p, p, p, p, 1 << 20, 4, 4, 4, 17, 1, None) == -3  # k beyond DL_MAX_K
    assert lib.dl_gather_fwd(p, p, 8, p, 1, 1, 1, 1, None) == -3
    assert lib.dl_prob_layer_fwd(p, p, p, 1.0, p, p, 256, 0, 1, 1, 1, 1, None) == -2
    with pytest.raises(RuntimeError, match="ROCm devices only"):
        _ops().DWNLayerFunction.apply(torch.zeros(2, 2), torch.zeros(1, 1, 4), None, 0.1, 0.1)
    with pytest.raises(IndexError):
        _ops().MappingPlan(torch.tensor([[0, 7]], device=DEV, dtype=torch.int32), 4)


def test_row_counts_beyond_one_grid_dimension():
    """B > 65535 rows for the gathers (RandomLayer.get_mapping, LearnableLayer eval) and more than 2^20 rows for the
    bit-plane packing (patch matrices of large image batches): the kernels walk the rows a grid dimension cannot hold."""
    from difflut_amd import _native as nat
    lib = nat.lib()
    rng = np.random.default_rng(5)
    B, I, N, k = 70001, 9, 5, 2
    x = rng.random((B, I)).astype(np.float32)
    idx = rng.integers(0, I, (N, k)).astype(np.int16)
    xd, idd = dev(x), torch.as_tensor(idx).to(DEV)
    m = torch.empty(B, N * k, device=DEV)
    nat.check(lib.dl_gather_fwd(xd.data_ptr(), idd.data_ptr(), 16, m.data_ptr(), B, I, N, k, nat.stream()))
    assert np.array_equal(m.cpu().numpy(), x[:, idx.reshape(-1).astype(np.int64)])
    plan = _ops().MappingPlan(idd.to(torch.int32), I)
    gm = rng.standard_normal((B, N * k)).astype(np.float32)
    gx = torch.empty(B, I, device=DEV)
    nat.check(lib.dl_gather_bwd(dev(gm).data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), gx.data_ptr(), B, I, N, k,
                                nat.stream()))
    want = np.zeros((B, I), np.float32)
    for p, i in enumerate(idx.reshape(-1)):
        want[:, i] += gm[:, p]
    np.testing.assert_allclose(gx.cpu().numpy(), want, rtol=1e-6, atol=1e-6)
    # bit-planes of 1 050 000 rows x 8 columns: 65 625 pieces of 16 rows
    R, C = 1050000, 8
    v = torch.rand(R, C, device=DEV)
    planes = torch.zeros(lib.dl_dwn_planes_bytes(R, C) // 8, dtype=torch.int64, device=DEV)
    nat.check(lib.dl_dwn_pack_planes(v.data_ptr(), planes.data_ptr(), R, C, nat.stream()))
    BT = (R + 63) // 64
    bits = torch.zeros(BT * 64, C, dtype=torch.int64, device=DEV)
    bits[:R] = (v >= 0.5).long()
    want_planes = (bits.view(BT, 64, C) << torch.arange(64, device=DEV).view(1, 64, 1)).sum(1)  # wraps into the sign bit
    assert torch.equal(planes[:BT * C].view(BT, C), want_planes)


@pytest.mark.parametrize("opts", [dict(lr=0.01), dict(lr=0.003, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.05),
                                  dict(lr=0.01, maximize=True)])
def test_bank_adam_against_torch_adam(opts):
    """`dl_adam_step`: several tensors of ragged sizes (one of them not 16-byte aligned) in one launch, five steps,
    against torch.optim.Adam on the same gradients."""
    from difflut_amd.utils import BankAdam

    torch.manual_seed(11)
    base = torch.randn(5000 + 1, device=DEV)
    ours = [torch.randn(300, 1, 64, device=DEV).requires_grad_(), torch.randn(2049, device=DEV).requires_grad_(),
            None, torch.randn(3, device=DEV).requires_grad_()]
    ours[2] = base[1:].detach().requires_grad_()  # a view that starts 4 bytes into its allocation
    ref = [t.detach().clone().requires_grad_() for t in ours]
    opt, ropt = BankAdam(ours, **opts), torch.optim.Adam(ref, **opts)
    for _ in range(5):
        for x, y in zip(ours, ref):
            g = torch.randn_like(x)
            x.grad, y.grad = g.clone(), g.clone()
        opt.step()
        ropt.step()
    for x, y in zip(ours, ref):
        np.testing.assert_allclose(x.detach().cpu().numpy(), y.detach().cpu().numpy(), rtol=2e-6, atol=1e-7)
    from difflut_amd import _native
    assert _native.lib().dl_adam_step(None, None, None, None, None, 1, 0.1, 0.9, 0.999, 1e-8, 0.0, 1, 0, None) == -1


@pytest.mark.parametrize("per_row", [False, True])
@pytest.mark.parametrize("subtract_mean", [False, True])
def test_grad_stabilize_against_the_reference_formula(per_row, subtract_mean):
    """`dl_grad_stabilize` against the torch operations of base_layer.py:266-339 evaluated in float64."""
    torch.manual_seed(3)
    rows, cols = 37, 5003
    g = (torch.randn(rows, cols, device=DEV) * 0.3 + 0.05)
    out = _ops().grad_stabilize(g, per_row, 0.7, subtract_mean, 1e-8)
    w = g.double()
    if subtract_mean:
        w = w - (w.mean(dim=1, keepdim=True) if per_row else w.mean())
    var = w.pow(2).mean(dim=1, keepdim=True) if per_row else w.pow(2).mean()
    want = w * torch.sqrt(0.7 / (var + 1e-8))
    np.testing.assert_allclose(out.cpu().numpy(), want.cpu().numpy(), rtol=1e-5, atol=1e-6)
    again = _ops().grad_stabilize(g, per_row, 0.7, subtract_mean, 1e-8)
    assert torch.equal(out, again)  # fixed order of additions
