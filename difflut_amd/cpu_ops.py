"""CPU branch of the layer-level operators, in plain torch.

The reference dispatches every operator on `x.is_cuda` and runs Python / torch code on CPU tensors
(difflut/layers/random_layer.py:272-304, difflut/nodes/dwn_node.py:130-229, 319-338,
difflut/nodes/probabilistic_node.py:277-328, difflut/nodes/hybrid_node.py:108-226,
difflut/nodes/dwn_stable_node.py:36-206, difflut/layers/learnable_layer.py:224-276).  These are the same
operators for a module that lives on the CPU (the reference's own CI runs there): whole-layer calls with the
argument conventions of `ops.py`, vectorised over batch, nodes and the 2^k table entries instead of the
reference's interpreter loops.  Like the reference's CPU path the EFD sums are accumulated in float64 and
rounded once.  Nothing here touches the HIP library, and nothing of the device path comes through here.
"""
import torch

_NODE_CHUNK = 256  # nodes per pass of the per-node weight tensors [chunk, k, L, L]


def _mapped(x, plan):
    """x [B, I] -> [B, N, k]: column idx[n, j] of x for every node input."""
    return x[:, plan.idx32.long()]


def _addresses(mapped):
    """Thresholded addresses [B, N]: bit j = (input j >= 0.5), input 0 the least significant bit."""
    k = mapped.shape[-1]
    weights = (1 << torch.arange(k, device=mapped.device)).long()
    return ((mapped >= 0.5).long() * weights).sum(-1)


def _float_addresses(mapped, L):
    """Eval-mode addresses floor(sum x_j 2^j) [B, N], clamped into the table (dwn_node.py:469-473)."""
    k = mapped.shape[-1]
    powers = (2.0 ** torch.arange(k, device=mapped.device, dtype=torch.float32))
    return (mapped.float() * powers).sum(-1).long().clamp_(0, L - 1)


def _lookup(tables, addr):
    """tables [N, O, L], addr [B, N] -> [B, N, O]."""
    N = tables.shape[0]
    return tables[torch.arange(N, device=tables.device).unsqueeze(0), :, addr]


def _hamming_tables(k, device):
    """H[l, a, kappa] = popcount((a ^ kappa) & ~(1 << l)) and sign[l, kappa] = +1 where bit l of kappa is set, else -1."""
    L = 1 << k
    a = torch.arange(L, device=device)
    xor = a.view(L, 1) ^ a.view(1, L)
    bits = torch.arange(k, device=device)
    masked = xor.unsqueeze(0) & ~(1 << bits).view(k, 1, 1)
    H = torch.zeros_like(masked)
    for b in range(k):
        H += (masked >> b) & 1
    sign = (((a.view(1, L) >> bits.view(k, 1)) & 1) * 2 - 1).double()
    return H, sign


def _scatter_inputs(gm, plan, B):
    """Adjoint of `_mapped`: gm [B, N, k] -> gx [B, I]."""
    gx = torch.zeros((B, plan.I), dtype=gm.dtype, device=gm.device)
    gx.index_add_(1, plan.idx32.reshape(-1).long(), gm.reshape(B, -1))
    return gx


def _table_histogram(gy, addr, L):
    """gl[n, d, e] = sum over the rows b with addr[b, n] = e of gy[b, n, d]."""
    B, N, O = gy.shape
    gl = torch.zeros((N, O, L), dtype=gy.dtype, device=gy.device)
    index = addr.t().unsqueeze(1).expand(N, O, B)
    gl.scatter_add_(2, index, gy.permute(1, 2, 0))
    return gl


def _weighted_input_grad(luts, gy, addr, weight_of_h, scale_of_node, k):
    """gm[b, n, l] = scale[n] * sum_d gy[b, n, d] * sum_kappa sign(kappa_l) luts[n, d, kappa] * w(h),
    h = popcount((addr ^ kappa) & ~bit_l); accumulated in float64.  `weight_of_h(H, nodes)` returns the weights as
    [k, L, L] (one set for the layer) or [chunk, k, L, L] (per node)."""
    B, N, O = gy.shape
    H, sign = _hamming_tables(k, luts.device)
    gm = torch.empty((B, N, k), dtype=torch.float32, device=luts.device)
    for n0 in range(0, N, _NODE_CHUNK):
        n1 = min(N, n0 + _NODE_CHUNK)
        W = weight_of_h(H, slice(n0, n1)) * sign.unsqueeze(1)  # [.., k, L(a), L(kappa)]
        t = luts[n0:n1].double()
        if W.dim() == 3:
            D = torch.einsum("ndq,laq->ndla", t, W)
        else:
            D = torch.einsum("ndq,nlaq->ndla", t, W)
        D = D * scale_of_node(slice(n0, n1)).view(-1, 1, 1, 1)
        nodes = torch.arange(n1 - n0, device=luts.device).unsqueeze(0)
        picked = D[nodes, :, :, addr[:, n0:n1]]  # [B, chunk, O, k]
        gm[:, n0:n1] = (gy[:, n0:n1].double().unsqueeze(-1) * picked).sum(2).float()
    return gm


# ----------------------------------------------------------------------------- gather
def gather(x, idx):
    """m[b, n, j] = x[b, idx[n, j]] with autograd (RandomLayer.get_mapping, random_layer.py:284-304)."""
    return x.float()[:, idx.long()]


# ----------------------------------------------------------------------------- DWN
class DWNLayerCPU(torch.autograd.Function):
    """Thresholded lookup with the extended-finite-difference backward for a whole layer
    (EFDFunctionCPU, dwn_node.py:130-229, applied to every node's mapped inputs)."""

    @staticmethod
    def forward(ctx, x, luts, plan, alpha, beta):
        x, luts = x.contiguous().float(), luts.contiguous().float()
        addr = _addresses(_mapped(x, plan))
        ctx.save_for_backward(luts, addr)
        ctx.plan, ctx.ab = plan, (alpha, beta)
        return _lookup(luts, addr).reshape(x.shape[0], -1)

    @staticmethod
    def backward(ctx, gy):
        luts, addr = ctx.saved_tensors
        plan = ctx.plan
        N, O, L = luts.shape
        B = addr.shape[0]
        gy = gy.contiguous().float().view(B, N, O)
        alpha, beta = ctx.ab
        alpha_n = torch.as_tensor(alpha, dtype=torch.float64, device=luts.device).expand(N)
        gx = None
        if ctx.needs_input_grad[0]:
            if torch.is_tensor(beta) and beta.numel() > 1:
                beta_n = beta.double().reshape(N)
                weights = lambda H, nodes: beta_n[nodes].view(-1, 1, 1, 1) ** H.unsqueeze(0)  # noqa: E731
            else:
                b = float(beta)
                weights = lambda H, nodes: torch.full((), b, dtype=torch.float64) ** H  # noqa: E731
            gm = _weighted_input_grad(luts, gy, addr, weights, lambda nodes: alpha_n[nodes], plan.k)
            gx = _scatter_inputs(gm, plan, B)
        return gx, _table_histogram(gy, addr, L), None, None, None


def dwn_layer(x, luts, plan, alpha, beta, beta_abs_max=None):
    return DWNLayerCPU.apply(x, luts, plan, alpha, beta)


def dwn_layer_eval(x, luts, plan):
    """DWNNode.forward_eval for a whole layer: no thresholding of the inputs, output (entry >= 0.5) as 0/1."""
    luts = luts.float()
    addr = _float_addresses(_mapped(x, plan), luts.shape[-1])
    return (_lookup(luts, addr) >= 0.5).float().reshape(x.shape[0], -1)


class DWNStableLayerCPU(torch.autograd.Function):
    """Thresholded lookup; backward with the weight scale / (h + 1), the table gradient scaled as well
    (dwn_stable_node.py:36-206)."""

    @staticmethod
    def forward(ctx, x, luts, scale, plan):
        x, luts = x.contiguous().float(), luts.contiguous().float()
        addr = _addresses(_mapped(x, plan))
        ctx.save_for_backward(luts, addr, scale.detach().double().reshape(-1))
        ctx.plan = plan
        return _lookup(luts, addr).reshape(x.shape[0], -1)

    @staticmethod
    def backward(ctx, gy):
        luts, addr, scale = ctx.saved_tensors
        plan = ctx.plan
        N, O, L = luts.shape
        B = addr.shape[0]
        gy = gy.contiguous().float().view(B, N, O)
        gx = None
        if ctx.needs_input_grad[0]:
            gm = _weighted_input_grad(luts, gy, addr, lambda H, nodes: 1.0 / (H.double() + 1.0),
                                      lambda nodes: scale[nodes], plan.k)
            gx = _scatter_inputs(gm, plan, B)
        gl = _table_histogram(gy, addr, L) * scale.float().view(N, 1, 1)
        return gx, gl, None, None


def dwn_stable_layer(x, luts, scale, plan):
    return DWNStableLayerCPU.apply(x, luts, scale, plan)


def _corner_probabilities(mapped):
    """p[b, n, a] = prod_j (x_j if bit j of a else 1 - x_j) for the 2^k corners, input 0 the least significant bit."""
    B, N, k = mapped.shape
    p = torch.ones((B, N, 1), dtype=mapped.dtype, device=mapped.device)
    for j in range(k):  # corner index gains bit j: [.., 2^j] -> [.., 2^(j+1)]
        xj = mapped[:, :, j:j + 1]
        p = torch.cat([p * (1.0 - xj), p * xj], dim=-1)
    return p


class HybridLayerCPU(torch.autograd.Function):
    """Thresholded lookup forward, probabilistic backward on the real-valued inputs
    (HybridFunctionCPU, hybrid_node.py:108-226)."""

    @staticmethod
    def forward(ctx, x, luts, plan):
        x, luts = x.contiguous().float(), luts.contiguous().float()
        mapped = _mapped(x, plan)
        ctx.save_for_backward(mapped, luts)
        ctx.plan = plan
        return _lookup(luts, _addresses(mapped)).reshape(x.shape[0], -1)

    @staticmethod
    def backward(ctx, gy):
        mapped, luts = ctx.saved_tensors
        plan = ctx.plan
        B, N, k = mapped.shape
        O, L = luts.shape[1], luts.shape[2]
        gy = gy.contiguous().float().view(B, N, O)
        p = _corner_probabilities(mapped)  # [B, N, L]
        gl = torch.einsum("bna,bnd->nda", p, gy)
        gx = None
        if ctx.needs_input_grad[0]:
            corners = ((torch.arange(L, device=luts.device).view(L, 1) >> torch.arange(k, device=luts.device)) & 1).float()
            xe = mapped.unsqueeze(2)  # [B, N, 1, k]
            factors = (corners.view(1, 1, L, k) - xe) / (xe * (1.0 - xe) + 1e-8)
            weighted = p.unsqueeze(-1) * factors  # [B, N, L, k]
            # sum over table entries of lut * p_a * (a_j - x_j) / (x_j (1 - x_j) + eps), then over the outputs with gy
            per_output = torch.einsum("bnaj,nda->bndj", weighted, luts)
            gm = (per_output * gy.unsqueeze(-1)).sum(2)
            gx = _scatter_inputs(gm, plan, B)
        return gx, gl, None


def hybrid_layer(x, luts, plan):
    return HybridLayerCPU.apply(x, luts, plan)


# ----------------------------------------------------------------------------- Probabilistic
def prob_layer(x, raw, plan, temperature):
    """y[b, n*O+d] = sum_a sigmoid(raw[n, a, d] / T) prod_j (x_j a_j + (1 - x_j)(1 - a_j)); torch autograd supplies the
    backward, as on the reference's CPU path (probabilistic_node.py:284-300).  `temperature`: a number or [N]."""
    x, raw = x.float(), raw.float()
    N = raw.shape[0]
    T = torch.as_tensor(temperature, dtype=torch.float32, device=raw.device).reshape(-1).clamp(min=1e-6)
    weights = torch.sigmoid(raw / T.expand(N).view(N, 1, 1))  # [N, L, O]
    p = _corner_probabilities(_mapped(x, plan))  # [B, N, L]
    return torch.einsum("bna,nad->bnd", p, weights).reshape(x.shape[0], -1)


def prob_layer_eval(x, raw, plan, temperature):
    """addr = floor(sum x_j 2^j), output (sigmoid(raw[addr] / T) >= 0.5) as 0/1 (probabilistic_node.py:302-328)."""
    raw = raw.float()
    N, L, O = raw.shape
    T = torch.as_tensor(temperature, dtype=torch.float32, device=raw.device).reshape(-1).clamp(min=1e-6)
    weights = torch.sigmoid(raw / T.expand(N).view(N, 1, 1)).permute(0, 2, 1)  # [N, O, L]
    addr = _float_addresses(_mapped(x, plan), L)
    return (_lookup(weights, addr) >= 0.5).float().reshape(x.shape[0], -1)


# ----------------------------------------------------------------------------- learnable mapping
def soft_map(x, W, tau, precision=0):
    """m = x @ softmax(W / tau, dim=-1).T (learnable_layer.py:254-255); always fp32 on the CPU."""
    return torch.matmul(x.float(), torch.softmax(W.float() / tau, dim=-1).t())


def row_argmax(W):
    return torch.argmax(W.float(), dim=-1).to(torch.int32)


def hard_select(x, sel):
    """m[b, o] = x[b, sel[o]] with the scatter-add backward of indexing."""
    return x.float()[:, sel.long()]


# ----------------------------------------------------------------------------- encoder / head
def thermometer_encode(x, thresholds):
    """bits[b, f, j] = (x[b, f] > thresholds[f, j]) as fp32."""
    return (x.float().unsqueeze(-1) > thresholds.float().unsqueeze(0)).float()


def group_sum(x, groups, tau):
    """Features zero-padded to a multiple of `groups`, summed per contiguous group, divided by tau."""
    B, F = x.shape
    pad = (-F) % groups
    if pad:
        x = torch.nn.functional.pad(x, (0, pad))
    return x.float().view(B, groups, -1).sum(-1) / tau
