"""CPU restatement of the DiffLUT hot path.  TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; nothing under difflut_amd/ does.  Every function restates one piece
of the reference (paths relative to the reference checkout) and is pinned by
tests/test_oracle.py against tests/golden/reference_vectors.npz (numbers written
by the reference's own CPU path) and against closed forms / brute force.

Pin status (see tests/test_oracle.py for the checks):
  random_mapping ............ golden index tables for 6 (I,N,k,seed) cases + permutation invariants
  gather_forward/backward ... brute force, torch.gather
  dwn_address/forward ....... golden y, all-2^k corner brute force, residual-init known answer
  dwn_eval_forward .......... golden, residual-init pass-through of input bit 0
  efd_backward .............. golden gx/gl, literal-loop restatement, beta=0/beta=1/constant-table cases
  prob_forward/backward ..... golden y/gx/gw, corner values, partition of unity, float64 gradcheck
  prob_eval_forward ......... golden
  soft_mapping_* ............ golden m/gx/gW at two temperatures, torch autograd
  hard_mapping .............. golden
  thermometer_* ............. golden thresholds/bits, notebook known answer [0.25,0.5,0.75]
  group_sum ................. golden, reference unit-test values
  stable_coefficients/backward  integral of the pinned EFD coefficients over beta in [0,1] (1/(h+1) =
                              int beta^h), literal-loop restatement, k=1 and constant-table cases, histogram sum
  conv_unfold/fold .......... torch.nn.functional.unfold/fold (library routines); conv_trees_* are loops over the
                              pinned layer functions, checked against a hand-built two-tree case
  hybrid_backward ........... autograd of the multilinear interpolation for interior x, per-thread loop form
                              of the device kernels, exact zeros at x in {0,1}, partition of unity
No function is left "parity unpinned".
"""
from __future__ import annotations

import numpy as np
import torch

# ----------------------------------------------------------------------------
# a1  RandomLayer._init_mapping          difflut/layers/random_layer.py:195-256
# ----------------------------------------------------------------------------


def random_mapping(input_size, output_size, n, seed=42, ensure_full_input_coverage=True,
                   mapping_indices=None):
    """Seeded [output_size, n] index table; int16 below 32768 inputs else int32.

    Same torch CPU-generator calls in the same order as random_layer.py:208-256:
    save state, manual_seed, floor(N*n/I) randperm(I) draws, one
    multinomial(ones(I), rem, replacement=False) for the tail, restore state.
    """
    state = torch.get_rng_state()
    torch.manual_seed(seed)
    dtype = torch.int16 if input_size < 32768 else torch.int32  # random_layer.py:214
    if mapping_indices is not None:
        table = torch.as_tensor(mapping_indices).to(dtype)  # :216-217
    elif not ensure_full_input_coverage:  # :219-224
        table = torch.multinomial(torch.ones((output_size, input_size)), n,
                                  replacement=n > input_size).to(dtype)
    else:  # :226-246
        total = output_size * n
        chunks = [torch.randperm(input_size) for _ in range(total // input_size)]
        rem = total % input_size
        if rem > 0:
            chunks.append(torch.multinomial(torch.ones(input_size), rem, replacement=False))
        table = torch.cat(chunks).reshape(output_size, n).to(dtype)
    torch.set_rng_state(state)
    return table


# ----------------------------------------------------------------------------
# a2/a3  gather and its adjoint          random_layer.py:284-304, mapping_cuda_kernel.cu:30-56,136-162
# ----------------------------------------------------------------------------


def gather_forward(x, idx):
    """m[b,n,j] = x[b, idx[n,j]]"""
    x = np.asarray(x)
    return x[:, np.asarray(idx, dtype=np.int64)]


def gather_backward(gm, idx, input_size):
    """gx[b,i] = sum over (n,j) with idx[n,j]==i of gm[b,n,j]; float64 accumulation."""
    gm = np.asarray(gm, dtype=np.float64)
    flat = np.asarray(idx, dtype=np.int64).reshape(-1)
    gx = np.zeros((gm.shape[0], input_size), dtype=np.float64)
    np.add.at(gx, (slice(None), flat), gm.reshape(gm.shape[0], -1))
    return gx


# ----------------------------------------------------------------------------
# a6  DWN training forward               dwn_node.py:137-165, efd_cuda_kernel.cu:12-43
# ----------------------------------------------------------------------------


def dwn_address(xk):
    """addr[...] = sum_j [xk[..., j] >= 0.5] << j   (input 0 is the LSB)."""
    xk = np.asarray(xk)
    k = xk.shape[-1]
    bits = (xk >= np.float32(0.5)).astype(np.int64)
    return (bits << np.arange(k, dtype=np.int64)).sum(-1)


def dwn_forward(xk, luts):
    """One node: xk [B,k], luts [O,2^k] -> y [B,O] = luts[:, addr].T"""
    luts = np.asarray(luts)
    return luts[:, dwn_address(xk)].T.copy()


def dwn_layer_forward(x, idx, luts):
    """Whole layer: x [B,I], idx [N,k], luts [N,O,2^k] -> y [B,N,O] (random_layer.py:306-340)."""
    luts = np.asarray(luts)
    addr = dwn_address(gather_forward(x, idx))  # [B,N]
    n_ar = np.arange(luts.shape[0])[None, :]
    return luts[n_ar, :, addr]  # [B,N,O]


# ----------------------------------------------------------------------------
# a7  DWN eval forward                   dwn_node.py:457-483
# ----------------------------------------------------------------------------


def dwn_eval_forward(xk, luts):
    """addr = floor(sum_j x_j 2^j) with NO thresholding of x; y = (luts[:,addr] >= 0.5)."""
    xk = np.asarray(xk, dtype=np.float32)
    k = xk.shape[-1]
    powers = (2.0 ** np.arange(k)).astype(np.float32)
    addr = (xk * powers).sum(-1, dtype=np.float32).astype(np.int64)
    return (np.asarray(luts)[:, addr].T >= np.float32(0.5)).astype(np.float32)


# ----------------------------------------------------------------------------
# a8/a9  Extended-finite-difference backward     dwn_node.py:167-229, efd_cuda_kernel.cu:79-189
# ----------------------------------------------------------------------------


def efd_backward_literal(xk, luts, gy, alpha, beta):
    """Loop-for-loop restatement of EFDFunctionCPU.backward (dwn_node.py:183-227).

    Python floats (doubles) accumulate the input gradient exactly as the
    reference does; tiny shapes only.
    """
    xk = np.asarray(xk); luts = np.asarray(luts); gy = np.asarray(gy)
    B, k = xk.shape
    O, L = luts.shape
    gx = np.zeros((B, k), dtype=np.float32)
    gl = np.zeros((O, L), dtype=np.float32)
    for b in range(B):
        addr = 0
        for i in range(k):
            if float(xk[b, i]) >= 0.5:
                addr |= 1 << i
        for d in range(O):
            gl[d, addr] += gy[b, d]
        for l in range(k):
            mask = ((1 << k) - 1) & ~(1 << l)
            am = addr & mask
            total = 0.0
            for kk in range(L):
                h = bin(am ^ (kk & mask)).count("1")
                sgn = -1.0 if ((kk >> l) & 1) == 0 else 1.0
                for d in range(O):
                    total += alpha * sgn * float(luts[d, kk]) * (beta ** h) * float(gy[b, d])
            gx[b, l] = total
    return gx, gl


def efd_coefficients(luts, alpha, beta):
    """D[..., l, a] = alpha * sum_kappa s(kappa_l) luts[..., kappa] beta^popc((a^kappa)&~(1<<l)).

    luts [..., 2^k] -> D [..., k, 2^k] in float64.  The value does not depend on
    bit l of a; both copies are stored so callers can index with the full address.
    """
    luts = np.asarray(luts, dtype=np.float64)
    L = luts.shape[-1]
    k = L.bit_length() - 1
    a = np.arange(L)[:, None]
    kap = np.arange(L)[None, :]
    D = np.empty(luts.shape[:-1] + (k, L), dtype=np.float64)
    for l in range(k):
        mask = (L - 1) & ~(1 << l)
        ham = np.vectorize(lambda v: bin(v).count("1"))((a ^ kap) & mask)
        sgn = np.where((kap >> l) & 1, 1.0, -1.0)
        M = alpha * sgn * np.power(float(beta), ham)  # [a, kappa]; 0**0 == 1 like the reference
        D[..., l, :] = luts @ M.T
    return D


def efd_backward(xk, luts, gy, alpha, beta):
    """Vectorised float64 form of the same sums: returns (gx [B,k], gl [O,2^k])."""
    xk = np.asarray(xk); gy64 = np.asarray(gy, dtype=np.float64)
    O, L = np.asarray(luts).shape
    addr = dwn_address(xk)
    D = efd_coefficients(luts, alpha, beta)  # [O,k,L]
    gx = np.einsum("bd,dlb->bl", gy64, D[:, :, addr])
    gl = np.zeros((O, L), dtype=np.float64)
    np.add.at(gl, (slice(None), addr), gy64.T)
    return gx, gl


def dwn_layer_backward(x, idx, luts, gy, alpha, beta):
    """Layer adjoint: x [B,I], idx [N,k], luts [N,O,L], gy [B,N,O] -> gx [B,I], gl [N,O,L] (float64)."""
    x = np.asarray(x); luts = np.asarray(luts)
    gy64 = np.asarray(gy, dtype=np.float64)
    B, I = x.shape
    N, O, L = luts.shape
    k = np.asarray(idx).shape[1]
    addr = dwn_address(gather_forward(x, idx))  # [B,N]
    D = efd_coefficients(luts, alpha, beta)  # [N,O,k,L]
    n_ar = np.arange(N)[None, :]
    Dsel = D[n_ar, :, :, addr]  # [B,N,O,k]
    gm = np.einsum("bnd,bndl->bnl", gy64, Dsel)  # [B,N,k]
    gx = gather_backward(gm, idx, I)
    gl = np.zeros((N, O, L), dtype=np.float64)
    b_ar = np.arange(B)[:, None]
    for d in range(O):
        np.add.at(gl[:, d, :], (np.broadcast_to(n_ar, addr.shape), addr), gy64[b_ar, n_ar, d])
    return gx, gl


# ----------------------------------------------------------------------------
# f1  Gradient-stabilised DWN node       dwn_stable_node.py:113-206, dwn_stable_cuda_kernel.cu:84-172
# ----------------------------------------------------------------------------


def table_sigmoid(raw):
    """luts = sigmoid(raw_luts) (dwn_stable_node.py:289-295, hybrid_node.py:309-315), float64."""
    return 1.0 / (1.0 + np.exp(-np.asarray(raw, dtype=np.float64)))


def stable_coefficients(luts, scale=1.0):
    """D[..., l, a] = scale * sum_kappa s(kappa_l) luts[..., kappa] / (popc((a^kappa)&~(1<<l)) + 1).

    The EFD sum with the weight beta^h replaced by 1/(h+1) (dwn_stable_node.py:176-201).
    `scale` broadcasts against luts.shape[:-1].  luts [..., 2^k] -> D [..., k, 2^k], float64.
    """
    luts = np.asarray(luts, dtype=np.float64)
    L = luts.shape[-1]
    k = L.bit_length() - 1
    a = np.arange(L)[:, None]
    kap = np.arange(L)[None, :]
    D = np.empty(luts.shape[:-1] + (k, L), dtype=np.float64)
    for l in range(k):
        mask = (L - 1) & ~(1 << l)
        ham = np.vectorize(lambda v: bin(v).count("1"))((a ^ kap) & mask)
        sgn = np.where((kap >> l) & 1, 1.0, -1.0)
        D[..., l, :] = luts @ (sgn / (ham + 1.0)).T
    return D * np.asarray(scale, dtype=np.float64)[..., None, None]


def stable_backward(xk, luts, gy, scale):
    """One node: xk [B,k], luts [O,2^k] (already sigmoid-ed), gy [B,O] -> (gx [B,k], gl [O,2^k]).
    gl[d, addr_b] += gy[b,d] * scale (dwn_stable_node.py:170-172)."""
    gy64 = np.asarray(gy, dtype=np.float64)
    O, L = np.asarray(luts).shape
    addr = dwn_address(xk)
    D = stable_coefficients(luts, scale)
    gx = np.einsum("bd,dlb->bl", gy64, D[:, :, addr])
    gl = np.zeros((O, L), dtype=np.float64)
    np.add.at(gl, (slice(None), addr), gy64.T * float(scale))
    return gx, gl


def stable_layer_backward(x, idx, raw_luts, gy, scale):
    """Layer adjoint down to the raw tables: x [B,I], idx [N,k], raw_luts [N,O,L], gy [B,N,O],
    scale [N] -> gx [B,I], graw [N,O,L] (float64).  graw = gl * s (1 - s), the sigmoid applied by
    forward_train outside the autograd Function (dwn_stable_node.py:309-316)."""
    x = np.asarray(x)
    luts = table_sigmoid(raw_luts)
    gy64 = np.asarray(gy, dtype=np.float64)
    scale = np.broadcast_to(np.asarray(scale, dtype=np.float64), (luts.shape[0],))
    B, I = x.shape
    N, O, L = luts.shape
    addr = dwn_address(gather_forward(x, idx))
    D = stable_coefficients(luts, scale[:, None])  # [N,O,k,L]
    n_ar = np.arange(N)[None, :]
    gm = np.einsum("bnd,bndl->bnl", gy64, D[n_ar, :, :, addr])
    gx = gather_backward(gm, idx, I)
    gl = np.zeros((N, O, L), dtype=np.float64)
    b_ar = np.arange(B)[:, None]
    for d in range(O):
        np.add.at(gl[:, d, :], (np.broadcast_to(n_ar, addr.shape), addr), gy64[b_ar, n_ar, d] * scale[None, :])
    return gx, gl * luts * (1.0 - luts)


# ----------------------------------------------------------------------------
# f1  Hybrid node                        hybrid_node.py:137-204, hybrid_cuda_kernel.cu:38-126
# ----------------------------------------------------------------------------

HYBRID_EPS = 1e-8  # hybrid_node.py:166


def hybrid_backward(xk, luts, gy, dtype=np.float64):
    """Probabilistic gradients of a thresholded lookup: xk [B,k], luts [O,2^k], gy [B,O] ->
    (gx [B,k], gl [O,2^k]).  Vectorised form of HybridFunctionCPU.backward: p[b,a] = prod_j
    (x_j a_j + (1-x_j)(1-a_j)); gl = (p^T gy)^T; gx[b,l] = sum_d gy[b,d] sum_a luts[d,a] p[b,a]
    (a_l - x_l) / (x_l (1 - x_l) + eps).  Because of eps an input that is exactly 0 or 1 gets a zero
    gradient, not the one-sided derivative."""
    x = np.asarray(xk, dtype=dtype)
    luts = np.asarray(luts, dtype=dtype)
    gy = np.asarray(gy, dtype=dtype)
    k = x.shape[1]
    L = luts.shape[1]
    combos = np.array([[(a >> j) & 1 for j in range(k)] for a in range(L)], dtype=dtype)
    xe = x[:, None, :]
    ae = combos[None, :, :]
    p = np.prod(xe * ae + (1 - xe) * (1 - ae), axis=2)  # [B,L]
    gl = (p.T @ gy).T
    deriv = (ae - xe) / (xe * (1 - xe) + dtype(HYBRID_EPS))  # [B,L,k]
    weighted = p[:, :, None] * deriv
    gx = np.einsum("bd,da,bal->bl", gy, luts, weighted)
    return gx, gl


def hybrid_layer_backward(x, idx, raw_luts, gy):
    """x [B,I], idx [N,k], raw_luts [N,O,L], gy [B,N,O] -> gx [B,I], graw [N,O,L] (float64);
    graw carries the sigmoid of forward_train (hybrid_node.py:327-332)."""
    x = np.asarray(x)
    luts = table_sigmoid(raw_luts)
    gy = np.asarray(gy, dtype=np.float64)
    m = gather_forward(x, idx)
    gm = np.zeros(m.shape, dtype=np.float64)
    gl = np.zeros(luts.shape, dtype=np.float64)
    for n in range(luts.shape[0]):
        gm[:, n], gl[n] = hybrid_backward(m[:, n], luts[n], gy[:, n])
    return gather_backward(gm, idx, x.shape[1]), gl * luts * (1.0 - luts)


# ----------------------------------------------------------------------------
# a11/a12/a13  Probabilistic node        probabilistic_node.py:236-328
# ----------------------------------------------------------------------------


def _prob_forward_t(x, raw_w, temperature):
    """torch form of forward_train's CPU branch (probabilistic_node.py:284-300)."""
    k = x.shape[-1]
    L = raw_w.shape[0]
    combos = torch.tensor([[(a >> j) & 1 for j in range(k)] for a in range(L)], dtype=x.dtype)
    w = torch.sigmoid(raw_w / torch.clamp(torch.tensor(float(temperature), dtype=x.dtype), min=1e-6))
    xe = x.unsqueeze(1)
    ae = combos.unsqueeze(0)
    probs = torch.prod(xe * ae + (1 - xe) * (1 - ae), dim=-1)
    return probs @ w


def prob_forward(xk, raw_w, temperature=1.0, dtype=torch.float32):
    """xk [B,k], raw_w [2^k,O] -> y [B,O]."""
    return _prob_forward_t(torch.as_tensor(np.asarray(xk)).to(dtype),
                           torch.as_tensor(np.asarray(raw_w)).to(dtype), temperature).numpy()


def prob_backward(xk, raw_w, gy, temperature=1.0, dtype=torch.float64):
    """Autograd of prob_forward (the reference's CPU backward is plain autograd): (gx, gw)."""
    x = torch.as_tensor(np.asarray(xk)).to(dtype).requires_grad_()
    w = torch.as_tensor(np.asarray(raw_w)).to(dtype).requires_grad_()
    y = _prob_forward_t(x, w, temperature)
    y.backward(torch.as_tensor(np.asarray(gy)).to(dtype))
    return x.grad.numpy(), w.grad.numpy()


def prob_eval_forward(xk, raw_w, temperature=1.0):
    """addr = floor(sum x_j 2^j); y = (sigmoid(w[addr]/T) >= 0.5)  (probabilistic_node.py:302-328)."""
    xk = torch.as_tensor(np.asarray(xk), dtype=torch.float32)
    w = torch.sigmoid(torch.as_tensor(np.asarray(raw_w), dtype=torch.float32)
                      / torch.clamp(torch.tensor(float(temperature)), min=1e-6))
    powers = 2 ** torch.arange(xk.shape[-1], dtype=torch.float32)
    addr = (xk * powers).sum(-1).long()
    return (w[addr] >= 0.5).float().numpy()


def prob_layer_forward(x, idx, raw_w, temperature=1.0, dtype=torch.float32):
    """x [B,I], idx [N,k], raw_w [N,2^k,O] -> y [B,N,O]."""
    m = gather_forward(x, idx)
    return np.stack([prob_forward(m[:, n], raw_w[n], temperature, dtype) for n in range(len(raw_w))], 1)


def prob_layer_backward(x, idx, raw_w, gy, temperature=1.0):
    """-> gx [B,I], gw [N,2^k,O] in float64."""
    x = np.asarray(x); raw_w = np.asarray(raw_w); gy = np.asarray(gy)
    m = gather_forward(x, idx)
    gm = np.zeros(m.shape, dtype=np.float64)
    gw = np.zeros(raw_w.shape, dtype=np.float64)
    for n in range(raw_w.shape[0]):
        gm[:, n], gw[n] = prob_backward(m[:, n], raw_w[n], gy[:, n], temperature)
    return gather_backward(gm, idx, x.shape[1]), gw


# ----------------------------------------------------------------------------
# a14  LearnableMappingModule            learnable_layer.py:216-278
# ----------------------------------------------------------------------------


def soft_mapping_forward(x, W, tau, dtype=torch.float32):
    """m = x @ softmax(W / tau, dim=-1).T      (learnable_layer.py:254-255)"""
    x = torch.as_tensor(np.asarray(x)).to(dtype)
    W = torch.as_tensor(np.asarray(W)).to(dtype)
    return (x @ torch.softmax(W / tau, dim=-1).t()).numpy()


def soft_mapping_backward(x, W, gm, tau, dtype=torch.float64):
    """Autograd of soft_mapping_forward: (gx, gW)."""
    x = torch.as_tensor(np.asarray(x)).to(dtype).requires_grad_()
    W = torch.as_tensor(np.asarray(W)).to(dtype).requires_grad_()
    m = x @ torch.softmax(W / tau, dim=-1).t()
    m.backward(torch.as_tensor(np.asarray(gm)).to(dtype))
    return x.grad.numpy(), W.grad.numpy()


def hard_mapping(x, W):
    """Eval mode: m[b,o] = x[b, argmax_i W[o,i]]   (learnable_layer.py:216-236, 257-276)."""
    sel = torch.argmax(torch.as_tensor(np.asarray(W)), dim=-1).numpy()
    return np.asarray(x)[:, sel], sel


def tau_schedule(tau_start, tau_min, tau_decay_iters, iteration):
    """learnable_layer.py:458-468"""
    return max(tau_start * 10.0 ** (-iteration / tau_decay_iters), tau_min)


# ----------------------------------------------------------------------------
# a16  ThermometerEncoder                encoder/thermometer.py:38-116
# ----------------------------------------------------------------------------


def thermometer_fit(x, num_bits):
    """thr[f,j] = min_f + (j+1) * (max_f - min_f) / (num_bits + 1), fp32 like the reference."""
    x = torch.as_tensor(np.asarray(x), dtype=torch.float32)
    lo = x.min(dim=0)[0]
    hi = x.max(dim=0)[0]
    steps = torch.arange(1, num_bits + 1)
    return (lo.unsqueeze(-1) + steps.unsqueeze(0) * ((hi - lo) / (num_bits + 1)).unsqueeze(-1)).numpy()


def thermometer_encode(x, thr):
    """bits[b, f*num_bits + j] = (x[b,f] > thr[f,j])  - strict compare, feature-major flatten."""
    x = np.asarray(x, dtype=np.float32)
    return (x[:, :, None] > np.asarray(thr)[None]).astype(np.float32).reshape(x.shape[0], -1)


# ----------------------------------------------------------------------------
# a17  GroupSum                          utils/modules.py:116-163
# ----------------------------------------------------------------------------


def group_sum(x, k, tau=1.0):
    """zero-pad the feature axis to a multiple of k, view [B,k,F/k], sum, divide by tau."""
    x = np.asarray(x, dtype=np.float32)
    F = x.shape[1]
    if F % k:
        x = np.pad(x, ((0, 0), (0, k - F % k)))
    return x.reshape(x.shape[0], k, -1).sum(-1, dtype=np.float32) / np.float32(tau)


# ----------------------------------------------------------------------------
# f4  Convolutional layer                layers/convolutional.py:194-267
# ----------------------------------------------------------------------------


def conv_unfold(x, receptive_field, stride, padding):
    """x [B,C,H,W] -> patches [B*positions, C*kh*kw] (nn.Unfold, then transpose/flatten, convolutional.py:199-205)."""
    p = torch.nn.functional.unfold(torch.as_tensor(np.asarray(x)), kernel_size=receptive_field, padding=padding, stride=stride)
    return p.transpose(1, 2).reshape(-1, p.shape[1]).numpy()


def conv_fold(gpatches, shape, receptive_field, stride, padding):
    """Adjoint of conv_unfold: gpatches [B*positions, C*kh*kw] -> gx [B,C,H,W] (what autograd does for nn.Unfold)."""
    B, C, H, W = shape
    g = torch.as_tensor(np.asarray(gpatches))
    g = g.reshape(B, -1, g.shape[1]).transpose(1, 2)
    return torch.nn.functional.fold(g, (H, W), kernel_size=receptive_field, padding=padding, stride=stride).numpy()


def conv_trees_forward(patches, chunks, trees, hidden0, layer_forward):
    """The chunk / tree loops of ConvolutionalLayer.forward (convolutional.py:214-242).

    chunks: [(idx, tables)] of the first-layer chunks; trees: per tree [(idx, tables)] of its later layers;
    layer_forward(x, idx, tables) -> [rows, nodes].  Returns (out [rows, trees], the activations kept for the
    backward)."""
    rows = patches.shape[0]
    out = np.zeros((rows, len(trees)), dtype=np.float32)
    acts, t = [], 0
    for idx, tab in chunks:
        first = layer_forward(patches, idx, tab)
        count = first.shape[1] // hidden0
        first = first.reshape(rows, count, hidden0)
        for local in range(count):
            h = first[:, local, :]
            kept = [h]
            for idx_l, tab_l in trees[t]:
                h = layer_forward(h, idx_l, tab_l)
                kept.append(h)
            out[:, t] = h[:, 0]
            acts.append(kept)
            t += 1
    return out, acts


def conv_trees_backward(patches, chunks, trees, hidden0, acts, gout, layer_backward):
    """Adjoint of conv_trees_forward.  layer_backward(x, idx, tables, gy [rows, nodes]) -> (gx, gtables).
    Returns (gpatches, chunk table gradients, per-tree table gradients)."""
    rows = patches.shape[0]
    gpatches = np.zeros(patches.shape, dtype=np.float64)
    gchunks, gtrees, t = [], [], 0
    for idx, tab in chunks:
        count = np.asarray(tab).shape[0] // hidden0
        gfirst = np.zeros((rows, count, hidden0), dtype=np.float64)
        for local in range(count):
            g = np.asarray(gout)[:, t:t + 1].astype(np.float64)
            grads = []
            for (idx_l, tab_l), x_l in zip(reversed(trees[t]), reversed(acts[t][:-1])):
                g, gt = layer_backward(x_l, idx_l, tab_l, g)
                grads.append(gt)
            gtrees.append(list(reversed(grads)))
            gfirst[:, local, :] = g
            t += 1
        gx, gt = layer_backward(patches, idx, tab, gfirst.reshape(rows, -1))
        gpatches += gx
        gchunks.append(gt)
    return gpatches, gchunks, gtrees
