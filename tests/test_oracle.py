"""Pins the CPU oracle: against the reference's own numbers (tests/golden), against the
known-answer tests the reference holds, and against what the mathematics fixes.
Runs without a GPU."""
import itertools

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import difflut_oracle as orc

MAP_TAGS = ["fused_a", "fused_b", "layer_fn", "exact3", "cfg1", "nocover"]


# ------------------------------------------------------------------ a1 mapping
@pytest.mark.parametrize("tag", MAP_TAGS)
def test_mapping_matches_reference_table(golden, tag):
    I, N, k, seed, cover = (int(v) for v in golden[f"map_{tag}_meta"])
    ref = golden[f"map_{tag}_idx"]
    got = orc.random_mapping(I, N, k, seed, ensure_full_input_coverage=bool(cover))
    assert got.dtype == torch.int16 and ref.dtype == np.int16
    assert np.array_equal(got.numpy(), ref)


def test_mapping_invariants_and_rng_restore():
    torch.manual_seed(99)
    before = torch.get_rng_state().clone()
    t = orc.random_mapping(50, 30, 4, seed=3).numpy().reshape(-1).astype(np.int64)
    assert torch.equal(before, torch.get_rng_state())  # random_layer.py:208,256
    full, rem = divmod(30 * 4, 50)
    for c in range(full):  # every full cycle is a permutation of all inputs
        assert np.array_equal(np.sort(t[c * 50:(c + 1) * 50]), np.arange(50))
    tail = t[full * 50:]
    assert len(tail) == rem and len(np.unique(tail)) == rem  # distinct draws
    assert orc.random_mapping(40000, 4, 2, seed=1).dtype == torch.int32  # random_layer.py:214
    given = torch.tensor([[1, 2], [3, 0]])
    assert np.array_equal(orc.random_mapping(4, 2, 2, mapping_indices=given).numpy(), given.numpy())


# ------------------------------------------------------------------ a2/a3 gather
def test_gather_brute_force():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 11)).astype(np.float32)
    idx = rng.integers(0, 11, (7, 3))
    m = orc.gather_forward(x, idx)
    gm = rng.standard_normal(m.shape)
    gx = orc.gather_backward(gm, idx, 11)
    for b in range(5):
        want = np.zeros(11)
        for n in range(7):
            for j in range(3):
                assert m[b, n, j] == x[b, idx[n, j]]
                want[idx[n, j]] += gm[b, n, j]
        assert np.allclose(gx[b], want, atol=1e-12)
    xt = torch.tensor(x)
    tm = torch.gather(xt.unsqueeze(1).expand(-1, 7, -1), 2, torch.tensor(idx).unsqueeze(0).expand(5, -1, -1))
    assert np.array_equal(tm.numpy(), m)  # random_layer.py:301-302


# ------------------------------------------------------------------ a6..a9 DWN
@pytest.mark.parametrize("tag", ["k6o2", "k4o1", "k2o3"])
def test_dwn_matches_reference(golden, tag):
    g = golden
    x, luts, gy = g[f"dwn_{tag}_x"], g[f"dwn_{tag}_luts"], g[f"dwn_{tag}_gy"]
    alpha, beta = g[f"dwn_{tag}_ab"]
    assert np.array_equal(orc.dwn_forward(x, luts), g[f"dwn_{tag}_y"])  # bit exact
    gx, gl = orc.efd_backward(x, luts, gy, alpha, beta)
    np.testing.assert_allclose(gx, g[f"dwn_{tag}_gx"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gl, g[f"dwn_{tag}_gl"], rtol=1e-6, atol=1e-6)
    gx2, gl2 = orc.efd_backward_literal(x, luts, gy, float(alpha), float(beta))
    assert np.array_equal(gx2, g[f"dwn_{tag}_gx"])  # same loop, same doubles -> identical
    np.testing.assert_allclose(gl2, g[f"dwn_{tag}_gl"], rtol=0, atol=1e-6)
    assert np.array_equal(orc.dwn_eval_forward(g[f"dwn_{tag}_eval_x"], luts), g[f"dwn_{tag}_eval_y"])


def test_dwn_default_alpha_beta(golden):
    a, b = golden["dwn_k6o2_ab"]  # dwn_node.py:410-415
    assert a == pytest.approx(0.5 * 0.75 ** 5, rel=1e-7) and b == pytest.approx(1 / 3, rel=1e-7)


def test_dwn_nondefault_alpha_beta(golden):
    g = golden
    gx, gl = orc.efd_backward(g["dwn_ab_x"], g["dwn_ab_luts"], g["dwn_ab_gy"], 0.7, 0.9)
    np.testing.assert_allclose(gx, g["dwn_ab_gx"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gl, g["dwn_ab_gl"], rtol=1e-6, atol=1e-6)


def test_dwn_address_is_lsb_first_all_corners():
    k = 6
    corners = np.array(list(itertools.product([0.0, 1.0], repeat=k)), dtype=np.float32)
    want = (corners * 2 ** np.arange(k)).sum(1).astype(np.int64)
    assert np.array_equal(orc.dwn_address(corners), want)
    assert orc.dwn_address(np.array([[0.5, 0.49999997, 0.50000006]], dtype=np.float32))[0] == 0b101  # >=


def test_residual_known_answer(golden):
    """reference tests/test_nodes/test_residual_initialization.py:56-105: eval passes input bit 0 through."""
    luts = golden["dwn_residual_luts"]
    corners = np.array(list(itertools.product([0, 1], repeat=6)), dtype=np.float32)
    assert np.array_equal(orc.dwn_eval_forward(corners, luts)[:, 0], corners[:, 0])
    want = np.where(np.arange(64) & 1, 5.0, -5.0).astype(np.float32)[None]
    assert np.array_equal(luts, want)


def test_efd_closed_form_special_cases():
    rng = np.random.default_rng(1)
    k, O, B = 4, 2, 9
    L = 1 << k
    x = rng.random((B, k)).astype(np.float32)
    luts = rng.uniform(-1, 1, (O, L)).astype(np.float32)
    gy = rng.standard_normal((B, O)).astype(np.float32)
    addr = orc.dwn_address(x)
    # beta = 0: plain finite difference  alpha * gy * (lut[a | bit] - lut[a & ~bit])   (0**0 == 1)
    gx, _ = orc.efd_backward(x, luts, gy, 0.3, 0.0)
    for l in range(k):
        hi, lo = addr | (1 << l), addr & ~(1 << l)
        l64 = luts.astype(np.float64)
        want = 0.3 * (gy.astype(np.float64) * (l64[:, hi] - l64[:, lo]).T).sum(1)
        np.testing.assert_allclose(gx[:, l], want, atol=1e-12)
    # beta = 1: alpha * gy * (sum of entries with bit l set - sum with it clear), same for every address
    gx, _ = orc.efd_backward(x, luts, gy, 0.3, 1.0)
    for l in range(k):
        sel = ((np.arange(L) >> l) & 1).astype(bool)
        diff = luts[:, sel].astype(np.float64).sum(1) - luts[:, ~sel].astype(np.float64).sum(1)
        np.testing.assert_allclose(gx[:, l], 0.3 * gy.astype(np.float64) @ diff, atol=1e-12)
    # constant table: no input gradient
    gx, _ = orc.efd_backward(x, np.full((O, L), 0.37, np.float32), gy, 0.3, 1 / 3)
    assert np.abs(gx).max() < 1e-12
    # literal loops agree with the closed form, and the table gradient conserves gy
    gxl, gll = orc.efd_backward_literal(x, luts, gy, 0.3, 1 / 3)
    gx, gl = orc.efd_backward(x, luts, gy, 0.3, 1 / 3)
    np.testing.assert_allclose(gxl, gx, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(gll, gl, atol=1e-6)
    np.testing.assert_allclose(gl.sum(1), gy.astype(np.float64).sum(0), atol=1e-12)


def test_dwn_layer_equals_per_node_loop_and_c_restatement():
    rng = np.random.default_rng(2)
    B, I, N, k, O = 6, 20, 9, 3, 2
    x = rng.random((B, I)).astype(np.float32)
    idx = orc.random_mapping(I, N, k, seed=5).numpy()
    luts = rng.uniform(-1, 1, (N, O, 1 << k)).astype(np.float32)
    gy = rng.standard_normal((B, N, O)).astype(np.float32)
    y = orc.dwn_layer_forward(x, idx, luts)
    gx, gl = orc.dwn_layer_backward(x, idx, luts, gy, 0.2, 1 / 3)
    m = orc.gather_forward(x, idx)
    gm = np.zeros((B, N, k))
    for n in range(N):  # random_layer.py:331-335
        assert np.array_equal(y[:, n], orc.dwn_forward(m[:, n], luts[n]))
        gm[:, n], gln = orc.efd_backward(m[:, n], luts[n], gy[:, n], 0.2, 1 / 3)
        np.testing.assert_allclose(gl[n], gln, atol=1e-12)
    np.testing.assert_allclose(gx, orc.gather_backward(gm, idx, I), atol=1e-12)
    assert np.array_equal(c_oracle.dwn_layer_forward(x, idx, luts), y)
    cgx, cgl = c_oracle.dwn_layer_backward(x, idx, luts, gy, 0.2, 1 / 3)
    np.testing.assert_allclose(cgx, gx, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(cgl, gl, rtol=1e-6, atol=1e-6)


def test_end_to_end_smallest_configuration(golden):
    """thermometer -> RandomLayer+DWN -> GroupSum -> cross-entropy, every gradient (reduced cfg)."""
    g = golden
    thr = orc.thermometer_fit(g["e2e_x"], 4)
    bits = orc.thermometer_encode(g["e2e_x"], thr)
    assert np.array_equal(bits, g["e2e_bits"])
    idx = orc.random_mapping(80, 30, 6, seed=42).numpy()
    assert np.array_equal(idx, g["e2e_idx"])
    y = orc.dwn_layer_forward(bits, idx, g["e2e_luts"])[:, :, 0]
    logits = orc.group_sum(y, 10, 1.0)
    np.testing.assert_allclose(logits, g["e2e_logits"], rtol=1e-6, atol=1e-6)
    lt = torch.tensor(logits, requires_grad=True)
    loss = torch.nn.functional.cross_entropy(lt, torch.tensor(g["e2e_labels"]))
    assert float(loss) == pytest.approx(float(g["e2e_loss"]), rel=1e-6)
    loss.backward()
    gy = np.repeat(lt.grad.numpy(), 3, axis=1)[:, :, None]  # adjoint of the group sum (30 nodes / 10)
    gx, gl = orc.dwn_layer_backward(bits, idx, g["e2e_luts"], gy, 0.5 * 0.75 ** 5, 1 / 3)
    np.testing.assert_allclose(gx, g["e2e_gbits"], rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(gl, g["e2e_gluts"], rtol=1e-5, atol=1e-7)


# ------------------------------------------------------------------ a11..a13 probabilistic
@pytest.mark.parametrize("tag", ["k4o2", "k6o1"])
def test_probabilistic_matches_reference(golden, tag):
    g = golden
    x, w, gy, T = g[f"prob_{tag}_x"], g[f"prob_{tag}_w"], g[f"prob_{tag}_gy"], float(g[f"prob_{tag}_T"][0])
    np.testing.assert_allclose(orc.prob_forward(x, w, T), g[f"prob_{tag}_y"], rtol=1e-6, atol=1e-7)
    gx, gw = orc.prob_backward(x, w, gy, T)
    np.testing.assert_allclose(gx, g[f"prob_{tag}_gx"], rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(gw, g[f"prob_{tag}_gw"], rtol=1e-4, atol=1e-6)
    assert np.array_equal(orc.prob_eval_forward(g[f"prob_{tag}_eval_x"], w, T), g[f"prob_{tag}_eval_y"])


def test_probabilistic_closed_forms():
    rng = np.random.default_rng(3)
    k, O = 4, 2
    w = rng.standard_normal((1 << k, O))
    corners = np.array(list(itertools.product([0.0, 1.0], repeat=k)))
    addr = (corners * 2 ** np.arange(k)).sum(1).astype(int)
    y = orc.prob_forward(corners, w, 0.7, dtype=torch.float64)
    np.testing.assert_allclose(y, 1 / (1 + np.exp(-w[addr] / 0.7)), atol=1e-12)  # corners hit the table
    x = rng.random((7, k))
    const = np.full((1 << k, O), 0.3)
    yc = orc.prob_forward(x, const, 1.0, dtype=torch.float64)
    np.testing.assert_allclose(yc, 1 / (1 + np.exp(-0.3)), atol=1e-12)  # probabilities sum to one
    gx, _ = orc.prob_backward(x, const, rng.standard_normal((7, O)), 1.0)
    assert np.abs(gx).max() < 1e-12
    xt = torch.tensor(x, requires_grad=True)
    wt = torch.tensor(w, requires_grad=True)
    assert torch.autograd.gradcheck(lambda a, b: orc._prob_forward_t(a, b, 0.7), (xt, wt), eps=1e-6, atol=1e-6)


def test_probabilistic_residual_known_answer():
    """reference test_residual_initialization.py:118-173: all-zero input -> sigmoid(-5), all-one -> sigmoid(5)."""
    w = np.where(np.arange(64) & 1, 5.0, -5.0)[:, None]
    lo = orc.prob_forward(np.zeros((3, 6)), w, 1.0)
    hi = orc.prob_forward(np.ones((3, 6)), w, 1.0)
    assert abs(lo.mean() - 1 / (1 + np.exp(5.0))) < 1e-6 and abs(hi.mean() - 1 / (1 + np.exp(-5.0))) < 1e-6
    a = np.zeros((1, 6)); b = np.zeros((1, 6)); b[0, 1:] = 1.0  # :185-232 independent of bits 1..5
    assert abs(orc.prob_forward(a, w)[0, 0] - orc.prob_forward(b, w)[0, 0]) < 1e-6


# ------------------------------------------------------------------ a14 learnable mapping
def test_soft_and_hard_mapping_match_reference(golden):
    g = golden
    tau = float(g["soft_tau"][0])
    np.testing.assert_allclose(orc.soft_mapping_forward(g["soft_x"], g["soft_W"], tau), g["soft_m"].reshape(5, -1),
                               rtol=1e-6, atol=1e-7)
    gx, gW = orc.soft_mapping_backward(g["soft_x"], g["soft_W"], g["soft_gm"].reshape(5, -1), tau)
    np.testing.assert_allclose(gx, g["soft_gx"], rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(gW, g["soft_gW"], rtol=1e-4, atol=1e-7)
    m, sel = orc.hard_mapping(g["soft_x"], g["soft_W"])
    assert np.array_equal(m, g["hard_m"].reshape(5, -1)) and np.array_equal(sel.reshape(7, 3), g["hard_idx"])
    t500 = orc.tau_schedule(1.0, 1e-4, 1000.0, 500)
    assert t500 == pytest.approx(float(g["soft_tau_500"][0]), rel=1e-12)
    np.testing.assert_allclose(orc.soft_mapping_forward(g["soft_x"], g["soft_W"], t500),
                               g["soft500_m"].reshape(5, -1), rtol=1e-5, atol=1e-7)
    gx, gW = orc.soft_mapping_backward(g["soft_x"], g["soft_W"], g["soft_gm"].reshape(5, -1), t500)
    np.testing.assert_allclose(gx, g["soft500_gx"], rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(gW, g["soft500_gW"], rtol=1e-4, atol=1e-6)


def test_soft_mapping_limits():
    rng = np.random.default_rng(4)
    x = rng.random((3, 6))
    W = rng.standard_normal((4, 6))
    cold = orc.soft_mapping_forward(x, W, 1e-4, dtype=torch.float64)  # tau -> 0: hard selection
    np.testing.assert_allclose(cold, orc.hard_mapping(x, W)[0], atol=1e-9)
    hot = orc.soft_mapping_forward(x, W, 1e9, dtype=torch.float64)  # tau -> inf: row mean
    np.testing.assert_allclose(hot, np.repeat(x.mean(1, keepdims=True), 4, 1), atol=1e-6)


# ------------------------------------------------------------------ a16 / a17
def test_thermometer(golden):
    thr = orc.thermometer_fit(golden["thermo_x"], 4)
    assert np.array_equal(thr, golden["thermo_thr"])
    assert np.array_equal(orc.thermometer_encode(golden["thermo_x"], thr), golden["thermo_bits"])
    # notebook known answer: 3 bits on linspace(0,1,20) -> thresholds 0.25, 0.5, 0.75
    t = orc.thermometer_fit(np.linspace(0, 1, 20, dtype=np.float32)[:, None], 3)
    np.testing.assert_allclose(t, [[0.25, 0.5, 0.75]], atol=1e-7)
    assert np.array_equal(orc.thermometer_encode(np.array([[0.25], [0.6]], np.float32), t), [[0, 0, 0], [1, 1, 0]])


def test_group_sum(golden):
    np.testing.assert_allclose(orc.group_sum(golden["groupsum_x"], 5, 2.0), golden["groupsum_y"], rtol=1e-6, atol=1e-6)
    ones = np.ones((2, 12), np.float32)  # reference tests/test_utils/test_utils_modules.py: ones -> group size / tau
    assert np.array_equal(orc.group_sum(ones, 3, 1.0), np.full((2, 3), 4.0))
    assert np.array_equal(orc.group_sum(ones, 3, 2.0), np.full((2, 3), 2.0))
    assert np.array_equal(orc.group_sum(np.ones((1, 10), np.float32), 4, 1.0), [[3, 3, 3, 1]])  # zero padded


# ------------------------------------------------------------------ gradient-stabilised DWN node
def _stable_literal(xk, luts, gy, scale):
    """Per-thread loop of the device kernel (dwn_stable_cuda_kernel.cu:84-172), accumulating in Python floats."""
    B, k = xk.shape
    O, L = luts.shape
    gx = np.zeros((B, k))
    gl = np.zeros((O, L))
    for b in range(B):
        addr = sum(1 << i for i in range(k) if xk[b, i] >= 0.5)
        for d in range(O):
            gl[d, addr] += float(gy[b, d]) * scale
        for l in range(k):
            mask = (L - 1) & ~(1 << l)
            for d in range(O):
                tot = 0.0
                for kap in range(L):
                    h = bin((addr & mask) ^ (kap & mask)).count("1")
                    tot += (1.0 if (kap >> l) & 1 else -1.0) * float(luts[d, kap]) / (h + 1.0)
                gx[b, l] += tot * float(gy[b, d]) * scale
    return gx, gl


def test_stable_coefficients_are_the_beta_integral_of_the_efd_coefficients():
    """1/(h+1) = integral of beta^h over [0,1]: the stabilised weights are the pinned EFD weights
    (alpha = 1) integrated over beta; Gauss-Legendre with 4 nodes is exact up to degree 7 > k-1."""
    rng = np.random.default_rng(5)
    nodes, weights = np.polynomial.legendre.leggauss(4)
    for k in (1, 2, 4, 6):
        luts = rng.random((3, 1 << k))
        want = sum(w / 2 * orc.efd_coefficients(luts, 1.0, (t + 1) / 2) for t, w in zip(nodes, weights))
        assert np.allclose(orc.stable_coefficients(luts, 1.7), 1.7 * want, rtol=1e-12, atol=1e-13)


def test_stable_backward_special_cases_and_literal_loop():
    rng = np.random.default_rng(6)
    for B, k, O in [(7, 3, 2), (5, 1, 1), (4, 4, 1)]:
        xk = rng.random((B, k)).astype(np.float32)
        luts = rng.random((O, 1 << k)).astype(np.float32)
        gy = rng.standard_normal((B, O)).astype(np.float32)
        gx, gl = orc.stable_backward(xk, luts, gy, 1.25)
        lx, ll = _stable_literal(xk, luts, gy, 1.25)
        assert np.allclose(gx, lx, rtol=1e-12, atol=1e-12) and np.allclose(gl, ll, rtol=1e-12, atol=1e-12)
        assert np.allclose(gl.sum(1), 1.25 * gy.astype(np.float64).sum(0))  # every sample lands in one bin
        assert np.allclose(orc.stable_backward(xk, np.full_like(luts, 0.3), gy, 1.25)[0], 0.0, atol=1e-15)
        if k == 1:  # no other input: the plain difference of the two entries
            assert np.allclose(gx[:, 0], 1.25 * gy[:, 0].astype(np.float64) * (float(luts[0, 1]) - float(luts[0, 0])))
    # k = 2 by hand: same other bit weighs 1, flipped other bit weighs 1/2
    luts = np.array([[0.1, 0.4, 0.8, 0.3]])
    gx, _ = orc.stable_backward(np.array([[0.9, 0.2]], dtype=np.float32), luts, np.array([[2.0]]), 1.0)
    assert np.allclose(gx, [[2.0 * ((0.4 - 0.1) + (0.3 - 0.8) / 2), 2.0 * ((0.3 - 0.4) + (0.8 - 0.1) / 2)]])


def test_stable_layer_equals_per_node_loop_with_sigmoid_chain():
    rng = np.random.default_rng(7)
    B, I, N, k, O = 9, 11, 6, 3, 2
    x = rng.random((B, I)).astype(np.float32)
    idx = rng.integers(0, I, (N, k))
    raw = rng.standard_normal((N, O, 1 << k)).astype(np.float32)
    gy = rng.standard_normal((B, N, O)).astype(np.float32)
    scale = rng.random(N) + 0.5
    gx, graw = orc.stable_layer_backward(x, idx, raw, gy, scale)
    wx = np.zeros((B, I))
    for n in range(N):
        s = torch.sigmoid(torch.tensor(raw[n], dtype=torch.float64)).requires_grad_()
        gxn, gln = orc.stable_backward(x[:, idx[n]], s.detach().numpy(), gy[:, n], scale[n])
        np.add.at(wx, (slice(None), idx[n]), gxn)
        t = torch.tensor(raw[n], dtype=torch.float64, requires_grad=True)
        torch.sigmoid(t).backward(torch.tensor(gln))  # the sigmoid autograd applies outside the Function
        assert np.allclose(graw[n], t.grad.numpy(), rtol=1e-12, atol=1e-14)
    assert np.allclose(gx, wx, rtol=1e-12, atol=1e-13)


# ------------------------------------------------------------------ hybrid node
def _hybrid_literal(xk, luts, gy):
    """Per-thread loops of hybrid_backward_input_kernel / hybrid_backward_lut_kernel
    (hybrid_cuda_kernel.cu:38-126) in Python floats."""
    B, k = xk.shape
    O, L = luts.shape
    gx = np.zeros((B, k))
    gl = np.zeros((O, L))
    for b in range(B):
        xs = [float(v) for v in xk[b]]
        for a in range(L):
            p = 1.0
            for i in range(k):
                ai = (a >> i) & 1
                p *= xs[i] * ai + (1.0 - xs[i]) * (1.0 - ai)
            for d in range(O):
                gl[d, a] += p * float(gy[b, d])
                for l in range(k):
                    al = (a >> l) & 1
                    gx[b, l] += p * (al - xs[l]) / (xs[l] * (1.0 - xs[l]) + 1e-8) * float(luts[d, a]) * float(gy[b, d])
    return gx, gl


def test_hybrid_backward_is_the_gradient_of_the_multilinear_interpolation():
    rng = np.random.default_rng(8)
    for B, k, O in [(6, 3, 2), (5, 6, 1), (4, 1, 3)]:
        xk = (0.05 + 0.9 * rng.random((B, k)))
        luts = rng.random((O, 1 << k))
        gy = rng.standard_normal((B, O))
        gx, gl = orc.hybrid_backward(xk, luts, gy)
        lx, ll = _hybrid_literal(xk, luts, gy)
        assert np.allclose(gx, lx, rtol=1e-11, atol=1e-12) and np.allclose(gl, ll, rtol=1e-11, atol=1e-12)
        # interior points: eps only perturbs by <= 1e-8 / (x (1 - x)) relative
        x = torch.tensor(xk, requires_grad=True)
        t = torch.tensor(luts, requires_grad=True)
        combos = torch.tensor([[(a >> j) & 1 for j in range(k)] for a in range(1 << k)], dtype=torch.float64)
        p = torch.prod(x[:, None, :] * combos + (1 - x[:, None, :]) * (1 - combos), dim=2)
        (p @ t.T).backward(torch.tensor(gy))
        assert np.allclose(gx, x.grad.numpy(), rtol=1e-6, atol=1e-9)
        assert np.allclose(gl, t.grad.numpy(), rtol=1e-12, atol=1e-13)
        assert np.allclose(gl.sum(1), gy.sum(0))  # the product weights of a sample sum to one


def test_hybrid_backward_is_zero_at_binary_inputs():
    rng = np.random.default_rng(9)
    xk = rng.integers(0, 2, (8, 4)).astype(np.float32)
    luts = rng.random((2, 16)).astype(np.float32)
    gy = rng.standard_normal((8, 2)).astype(np.float32)
    gx, gl = orc.hybrid_backward(xk, luts, gy)
    assert np.all(gx == 0.0)  # p * (a_l - x_l) vanishes term by term and the denominator is eps, not 0
    addr = orc.dwn_address(xk)
    want = np.zeros((2, 16))
    np.add.at(want, (slice(None), addr), gy.astype(np.float64).T)
    assert np.allclose(gl, want)  # at a corner the weights are the indicator of the address
    mixed = xk.copy()
    mixed[:, 1] = 0.3
    gm, _ = orc.hybrid_backward(mixed, luts, gy)
    assert np.all(gm[:, [0, 2, 3]] == 0.0) and np.all(gm[:, 1] != 0.0)


# ------------------------------------------------------------------ convolutional layer
def test_conv_unfold_ordering_and_fold_adjoint():
    """Patch columns are (channel, dy, dx), rows are (image, output position) row-major; fold is the
    adjoint (<unfold(x), g> = <x, fold(g)>)."""
    rng = np.random.default_rng(10)
    x = rng.random((2, 3, 5, 6)).astype(np.float32)
    p = orc.conv_unfold(x, (3, 2), (1, 2), (1, 0))
    out_h, out_w = (5 + 2 - 3) // 1 + 1, (6 - 2) // 2 + 1
    assert p.shape == (2 * out_h * out_w, 3 * 3 * 2)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (0, 0)))
    for b, oy, ox, c, dy, dx in [(0, 0, 0, 0, 0, 0), (1, 4, 2, 2, 2, 1), (0, 2, 1, 1, 1, 0)]:
        assert p[(b * out_h + oy) * out_w + ox, (c * 3 + dy) * 2 + dx] == xp[b, c, oy + dy, ox * 2 + dx]
    g = rng.standard_normal(p.shape).astype(np.float32)
    back = orc.conv_fold(g, x.shape, (3, 2), (1, 2), (1, 0))
    assert np.isclose((p.astype(np.float64) * g).sum(), (x.astype(np.float64) * back).sum(), rtol=1e-6)


def test_conv_tree_loops_on_a_hand_built_case():
    """Two trees of depth 1 with n = 2 in one chunk: tree t reads first-layer columns 2t, 2t+1 only."""
    rng = np.random.default_rng(11)
    patches = rng.random((7, 4)).astype(np.float32)
    idx0 = np.array([[0, 1], [2, 3], [1, 2], [3, 0]])
    tab0 = rng.random((4, 1, 4)).astype(np.float32)
    idx1 = np.array([[0, 1]])
    t1a, t1b = rng.random((1, 1, 4)).astype(np.float32), rng.random((1, 1, 4)).astype(np.float32)
    fwd = lambda x, idx, tab: orc.dwn_layer_forward(x, idx, tab)[:, :, 0]
    out, acts = orc.conv_trees_forward(patches, [(idx0, tab0)], [[(idx1, t1a)], [(idx1, t1b)]], 2, fwd)
    first = fwd(patches, idx0, tab0)
    assert np.array_equal(out[:, 0], fwd(first[:, 0:2], idx1, t1a)[:, 0])
    assert np.array_equal(out[:, 1], fwd(first[:, 2:4], idx1, t1b)[:, 0])
    gout = rng.standard_normal((7, 2)).astype(np.float32)
    bwd = lambda x, idx, tab, gy: orc.dwn_layer_backward(x, idx, tab, gy[:, :, None], 0.3, 0.4)
    gp, gch, gtr = orc.conv_trees_backward(patches, [(idx0, tab0)], [[(idx1, t1a)], [(idx1, t1b)]], 2, acts, gout, bwd)
    ga, gta = bwd(first[:, 0:2], idx1, t1a, gout[:, 0:1])
    gb, gtb = bwd(first[:, 2:4], idx1, t1b, gout[:, 1:2])
    wp, wt0 = bwd(patches, idx0, tab0, np.concatenate([ga, gb], 1))
    assert np.allclose(gp, wp) and np.allclose(gch[0], wt0) and np.allclose(gtr[0][0], gta) and np.allclose(gtr[1][0], gtb)


# ------------------------------------------------------------------ reference numbers for the later node types
@pytest.mark.parametrize("kind", ["stable", "hybrid"])
@pytest.mark.parametrize("tag", ["k6o1", "k3o2"])
def test_stable_and_hybrid_match_reference(golden_next, kind, tag):
    g = golden_next
    x, raw, gy = g[f"{kind}_{tag}_x"], g[f"{kind}_{tag}_raw"], g[f"{kind}_{tag}_gy"]
    luts = orc.table_sigmoid(raw)
    assert np.allclose(orc.dwn_forward(x, luts.astype(np.float32)), g[f"{kind}_{tag}_y"], rtol=1e-6, atol=1e-7)
    idx = np.arange(x.shape[1])[None]
    if kind == "stable":
        gx, graw = orc.stable_layer_backward(x, idx, raw[None], gy[:, None, :], 1.6)
    else:
        gx, graw = orc.hybrid_layer_backward(x, idx, raw[None], gy[:, None, :])
    assert np.allclose(gx, g[f"{kind}_{tag}_gx"], rtol=2e-5, atol=2e-6)      # the reference accumulates in fp32
    assert np.allclose(graw[0], g[f"{kind}_{tag}_graw"], rtol=2e-5, atol=2e-6)
    ev = orc.dwn_eval_forward(g[f"{kind}_{tag}_eval_x"], luts.astype(np.float32))
    assert np.array_equal(ev, g[f"{kind}_{tag}_eval_y"])


def test_conv_loops_match_reference_layer(golden_next):
    """The oracle's chunk / tree loops on the reference layer's own tables and index tables."""
    g = golden_next
    state = {k[len("conv_state."):]: v for k, v in g.items() if k.startswith("conv_state.")}
    def sub(prefix):
        n = 1 + max(int(k.split(".")[len(prefix.split(".")) + 1]) for k in state if k.startswith(prefix + ".nodes."))
        return state[prefix + "._mapping_indices"].astype(np.int64), np.stack([state[f"{prefix}.nodes.{i}.luts"] for i in range(n)])
    chunks = [sub(f"first_layer_chunks.{c}") for c in range(2)]
    trees = [[sub(f"trees.{t}.{l}") for l in range(2)] for t in range(3)]
    alpha, beta = float(state["trees.0.0.nodes.0.alpha"]), float(state["trees.0.0.nodes.0.beta"])
    x = g["conv_x"]
    patches = orc.conv_unfold(x, (2, 2), (1, 1), (0, 0))
    fwd = lambda m, i, t: orc.dwn_layer_forward(m, i, t)[:, :, 0]
    out, acts = orc.conv_trees_forward(patches, chunks, trees, 4, fwd)
    y = out.reshape(2, 9, 3).transpose(0, 2, 1).reshape(2, 3, 3, 3)
    assert np.array_equal(y, g["conv_y"])
    gout = g["conv_gy"].reshape(2, 3, 9).transpose(0, 2, 1).reshape(-1, 3)
    bwd = lambda m, i, t, gy: orc.dwn_layer_backward(m, i, t, gy[:, :, None], alpha, beta)
    gp, gch, gtr = orc.conv_trees_backward(patches, chunks, trees, 4, acts, gout, bwd)
    assert np.allclose(orc.conv_fold(gp, x.shape, (2, 2), (1, 1), (0, 0)), g["conv_gx"], rtol=1e-5, atol=1e-6)
    assert np.allclose(gch[1][3], g["conv_grad.first_layer_chunks.1.nodes.3.luts"], rtol=1e-5, atol=1e-6)
    assert np.allclose(gtr[2][1][0], g["conv_grad.trees.2.1.nodes.0.luts"], rtol=1e-5, atol=1e-6)
    assert np.allclose(gtr[0][0][1], g["conv_grad.trees.0.0.nodes.1.luts"], rtol=1e-5, atol=1e-6)
