"""Layer-level operators: torch.autograd.Functions over the C ABI of libdifflut_hip.so.

These are the callers of the drop-in boundary.  They keep the conventions of the
reference's autograd wrappers (difflut/layers/random_layer.py:34-100,
difflut/nodes/dwn_node.py:58-128, difflut/nodes/probabilistic_node.py:39-129,
difflut/layers/learnable_layer.py:58-123): inputs are made contiguous fp32, outputs
are new tensors, non-tensor arguments get no gradient.  Unlike the reference, one
call covers a whole layer, kernels go to torch's current stream and nothing
synchronises the device.
"""
import torch

from . import _native as nat
from . import cpu_ops

FAST_K = 6


def _f32(t):
    return t.contiguous().float()


def _bytes(n, device):
    return torch.empty(max(int(n), 256), dtype=torch.uint8, device=device)


class MappingPlan:
    """Device-side form of an index table idx [N,k] over I inputs.

    idx32   int32 [N,k]         the table widened (the reference registers int16 below 32768 inputs)
    inv_ptr int32 [I+1]         CSR row pointers of the inverse mapping
    inv_pos int32 [N*k]         flat positions n*k+j, grouped by input, ascending inside a group
    Built once per table with torch ops (sort + bincount); the kernels only read it.
    """

    def __init__(self, idx, input_size):
        if idx.dim() != 2:
            raise ValueError(f"mapping indices must be 2D (nodes, inputs per node), got {tuple(idx.shape)}")
        if idx.dtype not in (torch.int16, torch.int32, torch.int64):
            raise TypeError(f"mapping indices must be int16, int32 or int64, got {idx.dtype}")
        self.N, self.k = idx.shape
        self.I = int(input_size)
        flat = idx.reshape(-1).long()
        if flat.numel() and (int(flat.min()) < 0 or int(flat.max()) >= self.I):
            raise IndexError(f"mapping index outside [0, {self.I})")
        self.idx32 = idx.to(torch.int32).contiguous()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=self.I)
        self.inv_ptr = torch.cat([counts.new_zeros(1), counts.cumsum(0)]).to(torch.int32).contiguous()
        self.inv_pos = order.to(torch.int32).contiguous()
        self.device = idx.device
        self.source_ptr = idx.data_ptr()
        self.source_version = idx._version

    def matches(self, idx):
        return (idx.device == self.device and idx.data_ptr() == self.source_ptr
                and idx._version == self.source_version and tuple(idx.shape) == (self.N, self.k))

    @staticmethod
    def identity(k, device):
        return MappingPlan(torch.arange(k, dtype=torch.int32, device=device).view(1, k), k)


# ----------------------------------------------------------------------------- gather
class GatherFunction(torch.autograd.Function):
    """m[b,n,j] = x[b, idx[n,j]]  (RandomLayer.get_mapping)."""

    @staticmethod
    def forward(ctx, x, idx, plan):
        nat.require_device(x, idx)
        x = _f32(x)
        B, I = x.shape
        N, k = idx.shape
        bits = {torch.int16: 16, torch.int32: 32}.get(idx.dtype)
        if bits is None:
            raise TypeError("Unsupported index type for mapping kernel. Use int16 or int32.")
        m = torch.empty((B, N, k), dtype=torch.float32, device=x.device)
        nat.check(nat.lib().dl_gather_fwd(nat.ptr(x), nat.ptr(idx.contiguous()), bits, nat.ptr(m), B, I, N, k,
                                          nat.stream()))
        ctx.plan = plan
        ctx.shape = (B, I, N, k)
        return m

    @staticmethod
    def backward(ctx, gm):
        B, I, N, k = ctx.shape
        gm = _f32(gm)
        gx = torch.empty((B, I), dtype=torch.float32, device=gm.device)
        p = ctx.plan
        nat.check(nat.lib().dl_gather_bwd(nat.ptr(gm), nat.ptr(p.inv_ptr), nat.ptr(p.inv_pos), nat.ptr(gx), B, I, N, k,
                                          nat.stream()))
        return gx, None, None


# ----------------------------------------------------------------------------- patches of the convolutional layer
def _flip_bytes(flip, shape):
    """A flip mask as the contiguous byte matrix the kernels read (None stays None)."""
    if flip is None:
        return None
    if tuple(flip.shape) != tuple(shape):
        raise RuntimeError(f"flip mask {tuple(flip.shape)} does not match the patch matrix {tuple(shape)}")
    flip = flip.contiguous()
    return flip.view(torch.uint8) if flip.dtype == torch.bool else flip.to(torch.uint8)


class UnfoldFunction(torch.autograd.Function):
    """x [B,C,H,W] -> patches [B*OH*OW, C*KH*KW] (nn.Unfold, transposed and flattened as
    difflut/layers/convolutional.py:199-205 does); backward folds the patch gradients back.
    `geom` = (KH, KW, SH, SW, PH, PW).  `flip` (optional bool/uint8 [rows, C*KH*KW]): entries of the patch matrix that
    the bit-flip augmentation turns into 1 - value; noise, so the backward ignores it."""

    @staticmethod
    def forward(ctx, x, geom, flip=None):
        nat.require_device(x, flip)
        x = _f32(x)
        B, C, H, W = x.shape
        lib = nat.lib()
        rows = lib.dl_unfold_rows(B, H, W, *geom)
        if rows <= 0:
            raise RuntimeError(f"receptive field {geom[:2]} with stride {geom[2:4]}, padding {geom[4:]} does not fit a "
                               f"{H}x{W} image")
        patches = torch.empty((rows, C * geom[0] * geom[1]), dtype=torch.float32, device=x.device)
        flip = _flip_bytes(flip, patches.shape)
        nat.check(lib.dl_unfold_flip(nat.ptr(x), nat.ptr(flip), nat.ptr(patches), None, B, C, H, W, *geom, nat.stream()))
        ctx.shape, ctx.geom = (B, C, H, W), geom
        return patches

    @staticmethod
    def backward(ctx, gp):
        gp = _f32(gp)
        gx = torch.empty(ctx.shape, dtype=torch.float32, device=gp.device)
        nat.check(nat.lib().dl_fold(nat.ptr(gp), 0, nat.ptr(gx), *ctx.shape, *ctx.geom, nat.stream()))
        return gx, None, None


# ----------------------------------------------------------------------------- DWN
class DWNLayerFunction(torch.autograd.Function):
    """y[b, n*O+d] = luts[n,d,addr(b,n)] with the extended-finite-difference backward."""

    @staticmethod
    def forward(ctx, x, luts, plan, alpha, beta, beta_abs_max=None):
        """alpha, beta: Python floats for the whole layer, or device tensors [N] with every node's own values
        (then beta_abs_max = max |beta|, a host value)."""
        nat.require_device(x, luts)
        x, luts = _f32(x), _f32(luts)
        B, I = x.shape
        N, O, L = luts.shape
        k = plan.k
        if (N, 1 << k, I) != (plan.N, L, plan.I):
            raise RuntimeError(f"shape mismatch: x {tuple(x.shape)}, luts {tuple(luts.shape)}, mapping [{plan.N},{k}] "
                               f"over {plan.I} inputs")
        lib = nat.lib()
        dims = (B, I, N, k, O)
        y = torch.empty((B, N * O), dtype=torch.float32, device=x.device)
        saved = _bytes(lib.dl_dwn_saved_bytes(*dims), x.device)
        ws = _bytes(lib.dl_dwn_fwd_workspace_bytes(*dims), x.device)
        nat.check(lib.dl_dwn_layer_fwd(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(luts), nat.ptr(y), nat.ptr(saved),
                                       nat.ptr(ws), ws.numel(), *dims, nat.stream()))
        if torch.is_tensor(alpha) or torch.is_tensor(beta):
            alpha = torch.as_tensor(alpha, dtype=torch.float32, device=x.device).expand(N).contiguous()
            beta = torch.as_tensor(beta, dtype=torch.float32, device=x.device).expand(N).contiguous()
            if beta_abs_max is None:
                beta_abs_max = float(beta.abs().max())
            ctx.ab = (alpha, beta, float(beta_abs_max))
        else:
            ctx.ab = (float(alpha), float(beta))
        ctx.save_for_backward(luts, saved, x if k > FAST_K else None)
        ctx.plan, ctx.dims = plan, dims
        return y

    @staticmethod
    def backward(ctx, gy):
        luts, saved, x = ctx.saved_tensors
        B, I, N, k, O = ctx.dims
        plan = ctx.plan
        gy = _f32(gy)
        lib = nat.lib()
        gx = torch.empty((B, I), dtype=torch.float32, device=gy.device) if ctx.needs_input_grad[0] else None
        gl = torch.empty_like(luts)
        ws = _bytes(lib.dl_dwn_bwd_workspace_bytes(*ctx.dims), gy.device)
        if len(ctx.ab) == 3:
            nat.check(lib.dl_dwn_layer_bwd_nodes(nat.ptr(x), nat.ptr(saved), nat.ptr(plan.idx32), nat.ptr(plan.inv_ptr),
                                                 nat.ptr(plan.inv_pos), nat.ptr(luts), nat.ptr(gy), nat.ptr(ctx.ab[0]),
                                                 nat.ptr(ctx.ab[1]), ctx.ab[2], nat.ptr(gx), nat.ptr(gl), nat.ptr(ws),
                                                 ws.numel(), *ctx.dims, nat.stream()))
        else:
            nat.check(lib.dl_dwn_layer_bwd(nat.ptr(x), nat.ptr(saved), nat.ptr(plan.idx32), nat.ptr(plan.inv_ptr),
                                           nat.ptr(plan.inv_pos), nat.ptr(luts), nat.ptr(gy), ctx.ab[0], ctx.ab[1],
                                           nat.ptr(gx), nat.ptr(gl), nat.ptr(ws), ws.numel(), *ctx.dims, nat.stream()))
        return gx, gl, None, None, None, None


class DWNStackFunction(torch.autograd.Function):
    """A chain of RandomLayer + DWN layers in one autograd node.  A following DWN layer only thresholds
    what it is given, so between layers the activations stay bit-planes and the gradients stay
    tile-major: no [B, N] fp32 tensor is written or read except the last layer's output (and the
    first layer's input gradient, if asked for).  Same arithmetic as calling the layers one by one."""

    @staticmethod
    def forward(ctx, x, source, plans, scalars, head, *luts):
        """`scalars`: per layer (alpha, beta) as numbers, or (alpha [N], beta [N], max |beta|) with every node's own.
        `head`: None, or (groups, tau) of a GroupSum that follows the last layer: the function then returns
        the [B, groups] sums and neither the last layer's [B, N] output nor its gradient is ever written.
        `source` says what the first layer reads:
        None                  x [B, I] itself;
        a tensor [F, nbits]   thermometer thresholds: x is raw data [B, F], its code is produced directly
                              as bit-planes and x gets no gradient (the code is a step function of it);
        a tuple (KH, KW, SH, SW, PH, PW[, flip])   x is an image batch [B, C, H, W]: the first layer reads its patch
                              matrix (rows = output positions), again produced directly as bit-planes; the
                              input gradient is folded back from the tile-major patch gradient.  `flip`
                              (bool [rows, C*KH*KW], optional): patch entries the bit-flip augmentation inverts."""
        thresholds = source if torch.is_tensor(source) else None
        geom = tuple(source[:6]) if isinstance(source, tuple) else None
        flip = source[6] if isinstance(source, tuple) and len(source) > 6 else None
        nat.require_device(x, thresholds, *luts)
        x = _f32(x)
        luts = tuple(_f32(t) for t in luts)
        lib = nat.lib()
        ctx.image = None
        if geom is not None:
            Bi, C, H, W = x.shape
            B = int(lib.dl_unfold_rows(Bi, H, W, *geom))
            if B <= 0:
                raise RuntimeError(f"receptive field {geom[:2]} with stride {geom[2:4]}, padding {geom[4:]} does not fit "
                                   f"a {H}x{W} image")
            width = C * geom[0] * geom[1]
            planes = _bytes(lib.dl_dwn_planes_bytes(B, width), x.device)
            flip = _flip_bytes(flip, (B, width))
            nat.check(lib.dl_unfold_flip(nat.ptr(x), nat.ptr(flip), None, nat.ptr(planes), Bi, C, H, W, *geom, nat.stream()))
            ctx.image = ((Bi, C, H, W), geom)
        elif thresholds is None:
            B, width = x.shape
            planes = _bytes(lib.dl_dwn_planes_bytes(B, width), x.device)
            nat.check(lib.dl_dwn_pack_planes(nat.ptr(x), nat.ptr(planes), B, width, nat.stream()))
        else:
            B, width = x.shape
            thr = _f32(thresholds)
            if thr.dim() != 2 or thr.shape[0] != width:
                raise RuntimeError(f"thresholds {tuple(thr.shape)} do not match {width} features")
            nbits = thr.shape[1]
            planes = _bytes(lib.dl_dwn_planes_bytes(B, width * nbits), x.device)
            nat.check(lib.dl_thermometer_planes(nat.ptr(x), nat.ptr(thr), nat.ptr(planes), B, width, nbits, nat.stream()))
            width *= nbits
        saved, dims_all, y = [], [], None
        for l, (plan, lut) in enumerate(zip(plans, luts)):
            N, O, L = lut.shape
            k = plan.k
            if k > FAST_K or (N, 1 << k, width) != (plan.N, L, plan.I):
                raise RuntimeError(f"layer {l}: cannot chain (k={k}, tables {tuple(lut.shape)}, mapping [{plan.N},{k}] over "
                                   f"{plan.I} inputs, incoming width {width})")
            dims = (B, width, N, k, O)
            last = l == len(plans) - 1
            keep = _bytes(lib.dl_dwn_saved_bytes(*dims), x.device)
            nxt = None if last else _bytes(lib.dl_dwn_planes_bytes(B, N * O), x.device)
            if last and head is not None:
                groups, tau = head
                y = torch.empty((B, groups), dtype=torch.float32, device=x.device)
                ws = _bytes(lib.dl_dwn_groups_workspace_bytes(B, N, O, groups), x.device)
                nat.check(lib.dl_dwn_layer_fwd_planes_groups(nat.ptr(planes), nat.ptr(plan.idx32), nat.ptr(lut), nat.ptr(y),
                                                             nat.ptr(keep), nat.ptr(ws), ws.numel(), *dims, int(groups),
                                                             float(tau), nat.stream()))
            else:
                y = torch.empty((B, N * O), dtype=torch.float32, device=x.device) if last else None
                nat.check(lib.dl_dwn_layer_fwd_planes(nat.ptr(planes), nat.ptr(plan.idx32), nat.ptr(lut), nat.ptr(y),
                                                      nat.ptr(nxt), nat.ptr(keep), *dims, nat.stream()))
            saved.append(keep)
            dims_all.append(dims)
            planes, width = nxt, N * O
        ctx.save_for_backward(*luts, *saved)
        ctx.plans, ctx.scalars, ctx.dims_all = plans, scalars, dims_all
        ctx.encoded = thresholds is not None
        ctx.head = head
        return y

    @staticmethod
    def backward(ctx, gy):
        n = len(ctx.plans)
        luts, saved = ctx.saved_tensors[:n], ctx.saved_tensors[n:]
        lib = nat.lib()
        g, tiled = _f32(gy), 0
        device = g.device
        grads = [None] * n
        have_tables = [False] * n  # table gradient already produced by the call for the layer behind
        for l in range(n - 1, -1, -1):
            B, I, N, k, O = dims = ctx.dims_all[l]
            plan = ctx.plans[l]
            first_wants_input_grad = ctx.needs_input_grad[0] and not ctx.encoded
            if l > 0:
                gx = torch.empty(lib.dl_dwn_tiled_bytes(B, I) // 4, dtype=torch.float32, device=device)
                gx_tiled = 1
            else:
                want = ctx.needs_input_grad[0] and not ctx.encoded
                gx_tiled = 1 if ctx.image is not None else 0
                if not want:
                    gx = None
                elif gx_tiled:
                    gx = torch.empty(lib.dl_dwn_tiled_bytes(B, I) // 4, dtype=torch.float32, device=device)
                else:
                    gx = torch.empty((B, I), dtype=torch.float32, device=device)
            if have_tables[l] and gx is None:  # nothing left to compute for this layer
                g = None
                continue
            if not have_tables[l]:
                grads[l] = torch.empty_like(luts[l])
            ws = _bytes(lib.dl_dwn_bwd_workspace_bytes(*dims), device)
            headed = l == n - 1 and ctx.head is not None
            groups, tau = ctx.head if headed else (1, 1.0)
            if len(ctx.scalars[l]) == 3:  # every node's own alpha and beta
                alpha_n, beta_n, beta_max = ctx.scalars[l]
                alpha_n = _f32(alpha_n.detach()).reshape(-1).expand(N).contiguous()
                beta_n = _f32(beta_n.detach()).reshape(-1).expand(N).contiguous()
                # the gather of this layer can fill the table gradient of the layer in front as it goes: that layer's
                # own pass over its [B, N] output gradient is then left out
                k_prev = ctx.dims_all[l - 1][3] if l > 0 else 0
                fuse = (l > 0 and gx_tiled == 1 and ctx.dims_all[l - 1][4] == 1
                        and lib.dl_dwn_chain_fusable(*dims, k_prev, float(beta_max)) == 1)
                if fuse:
                    grads[l - 1] = torch.empty_like(luts[l - 1])
                    have_tables[l - 1] = True
                    ws = _bytes(lib.dl_dwn_bwd_fused_workspace_bytes(*dims, k_prev), device)
                    if l == 1 and not first_wants_input_grad:
                        gx = None  # the first layer's table gradient is all that is left: nobody reads this gradient
                nat.check(lib.dl_dwn_layer_bwd_chain_fused(
                    nat.ptr(saved[l]), nat.ptr(plan.inv_ptr), nat.ptr(plan.inv_pos), nat.ptr(luts[l]), nat.ptr(g),
                    2 if headed else tiled, int(groups), float(tau), nat.ptr(alpha_n), nat.ptr(beta_n), float(beta_max),
                    nat.ptr(gx), gx_tiled, None if have_tables[l] else nat.ptr(grads[l]),
                    nat.ptr(saved[l - 1]) if fuse else None, k_prev, nat.ptr(grads[l - 1]) if fuse else None,
                    nat.ptr(ws), ws.numel(), *dims, nat.stream()))
                g, tiled = gx, gx_tiled
                continue
            alpha, beta = ctx.scalars[l]
            if headed:
                nat.check(lib.dl_dwn_layer_bwd_groups(nat.ptr(saved[l]), nat.ptr(plan.inv_ptr), nat.ptr(plan.inv_pos),
                                                      nat.ptr(luts[l]), nat.ptr(g), int(groups), float(tau), float(alpha),
                                                      float(beta), nat.ptr(gx), gx_tiled, nat.ptr(grads[l]), nat.ptr(ws),
                                                      ws.numel(), *dims, nat.stream()))
            else:
                nat.check(lib.dl_dwn_layer_bwd_tiled(nat.ptr(saved[l]), nat.ptr(plan.inv_ptr), nat.ptr(plan.inv_pos),
                                                     nat.ptr(luts[l]), nat.ptr(g), tiled, float(alpha), float(beta),
                                                     nat.ptr(gx), gx_tiled, nat.ptr(grads[l]), nat.ptr(ws), ws.numel(), *dims,
                                                     nat.stream()))
            g, tiled = gx, gx_tiled
        if ctx.image is not None and g is not None:
            shape, geom = ctx.image
            gimg = torch.empty(shape, dtype=torch.float32, device=device)
            nat.check(lib.dl_fold(nat.ptr(g), 1, nat.ptr(gimg), *shape, *geom, nat.stream()))
            g = gimg
        return (g, None, None, None, None, *grads)


def dwn_stack_eval(x, thresholds, plans, luts, head=None):
    """Inference through a chain of RandomLayer + DWN layers whose first input is binary: `thresholds` [F, nbits]
    (x is raw data, its thermometer code feeds the first layer) or None (x [B, I] holds exact 0/1 values).
    Activations stay bit-planes between the layers; returns the last layer's 0/1 output [B, N], or with
    `head` = (groups, tau) its GroupSum [B, groups].  Equals calling the layers' eval forward one by one."""
    nat.require_device(x, thresholds, *luts)
    x = _f32(x)
    lib = nat.lib()
    B, width = x.shape
    if thresholds is None:
        planes = _bytes(lib.dl_dwn_planes_bytes(B, width), x.device)
        nat.check(lib.dl_dwn_pack_planes(nat.ptr(x), nat.ptr(planes), B, width, nat.stream()))
    else:
        thr = _f32(thresholds)
        if thr.dim() != 2 or thr.shape[0] != width:
            raise RuntimeError(f"thresholds {tuple(thr.shape)} do not match {width} features")
        nbits = thr.shape[1]
        planes = _bytes(lib.dl_dwn_planes_bytes(B, width * nbits), x.device)
        nat.check(lib.dl_thermometer_planes(nat.ptr(x), nat.ptr(thr), nat.ptr(planes), B, width, nbits, nat.stream()))
        width *= nbits
    y = None
    for l, (plan, lut) in enumerate(zip(plans, luts)):
        lut = _f32(lut)
        N, O, L = lut.shape
        k = plan.k
        if k > FAST_K or (N, 1 << k, width) != (plan.N, L, plan.I):
            raise RuntimeError(f"layer {l}: cannot chain (k={k}, tables {tuple(lut.shape)}, mapping [{plan.N},{k}] over "
                               f"{plan.I} inputs, incoming width {width})")
        dims = (B, width, N, k, O)
        last = l == len(plans) - 1
        if last and head is not None:
            groups, tau = head
            y = torch.empty((B, groups), dtype=torch.float32, device=x.device)
            ws = _bytes(lib.dl_dwn_groups_workspace_bytes(B, N, O, groups), x.device)
            nat.check(lib.dl_dwn_layer_eval_planes_groups(nat.ptr(planes), nat.ptr(plan.idx32), nat.ptr(lut), nat.ptr(y),
                                                          nat.ptr(ws), ws.numel(), *dims, int(groups), float(tau),
                                                          nat.stream()))
        else:
            y = torch.empty((B, N * O), dtype=torch.float32, device=x.device) if last else None
            nxt = None if last else _bytes(lib.dl_dwn_planes_bytes(B, N * O), x.device)
            nat.check(lib.dl_dwn_layer_eval_planes(nat.ptr(planes), nat.ptr(plan.idx32), nat.ptr(lut), nat.ptr(y),
                                                   nat.ptr(nxt), *dims, nat.stream()))
            planes = nxt
        width = N * O
    return y


def dwn_layer_eval(x, luts, plan):
    if not x.is_cuda:
        return cpu_ops.dwn_layer_eval(x, luts, plan)
    nat.require_device(x, luts)
    x, luts = _f32(x), _f32(luts)
    B, I = x.shape
    N, O, _ = luts.shape
    y = torch.empty((B, N * O), dtype=torch.float32, device=x.device)
    lib = nat.lib()
    dims = (B, I, N, plan.k, O)
    ws = _bytes(lib.dl_dwn_eval_workspace_bytes(*dims), x.device)
    nat.check(lib.dl_dwn_layer_eval_ws(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(luts), nat.ptr(y), nat.ptr(ws), ws.numel(),
                                       *dims, nat.stream()))
    return y


# ----------------------------------------------------------------------------- DWN-stable and hybrid nodes
class TableSigmoidFunction(torch.autograd.Function):
    """luts = sigmoid(raw_luts), elementwise, for a whole bank of tables at once
    (`_get_luts`, dwn_stable_node.py:289-295, hybrid_node.py:309-315)."""

    @staticmethod
    def forward(ctx, raw):
        nat.require_device(raw)
        raw = _f32(raw)
        luts = torch.empty_like(raw)
        nat.check(nat.lib().dl_table_sigmoid_fwd(nat.ptr(raw), nat.ptr(luts), raw.numel(), nat.stream()))
        ctx.save_for_backward(luts)
        return luts

    @staticmethod
    def backward(ctx, gl):
        (luts,) = ctx.saved_tensors
        gl = _f32(gl)
        graw = torch.empty_like(luts)
        nat.check(nat.lib().dl_table_sigmoid_bwd(nat.ptr(gl), nat.ptr(luts), nat.ptr(graw), luts.numel(), nat.stream()))
        return graw


def _dwn_lookup(x, luts, plan):
    """Training forward shared by the DWN-type nodes: (y, saved, dims)."""
    B, I = x.shape
    N, O, L = luts.shape
    k = plan.k
    if (N, 1 << k, I) != (plan.N, L, plan.I):
        raise RuntimeError(f"shape mismatch: x {tuple(x.shape)}, luts {tuple(luts.shape)}, mapping [{plan.N},{k}] "
                           f"over {plan.I} inputs")
    lib = nat.lib()
    dims = (B, I, N, k, O)
    y = torch.empty((B, N * O), dtype=torch.float32, device=x.device)
    saved = _bytes(lib.dl_dwn_saved_bytes(*dims), x.device)
    ws = _bytes(lib.dl_dwn_fwd_workspace_bytes(*dims), x.device)
    nat.check(lib.dl_dwn_layer_fwd(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(luts), nat.ptr(y), nat.ptr(saved),
                                   nat.ptr(ws), ws.numel(), *dims, nat.stream()))
    return y, saved, dims


class DWNStableLayerFunction(torch.autograd.Function):
    """Thresholded lookup with the gradient-stabilised backward: the EFD sum weighted 1/(h+1) and
    multiplied, like the table gradient, by the node's gradient scale (dwn_stable_node.py:36-206).
    `scale` is a device tensor [N] (one value per node); it gets no gradient, as in the reference."""

    @staticmethod
    def forward(ctx, x, luts, scale, plan):
        nat.require_device(x, luts, scale)
        x, luts = _f32(x), _f32(luts)
        scale = _f32(scale.detach()).reshape(-1)
        if scale.numel() != luts.shape[0]:
            raise RuntimeError(f"gradient_scale has {scale.numel()} entries for {luts.shape[0]} nodes")
        y, saved, dims = _dwn_lookup(x, luts, plan)
        ctx.save_for_backward(luts, saved, scale, x if plan.k > FAST_K else None)
        ctx.plan, ctx.dims = plan, dims
        return y

    @staticmethod
    def backward(ctx, gy):
        luts, saved, scale, x = ctx.saved_tensors
        B, I, N, k, O = ctx.dims
        plan = ctx.plan
        gy = _f32(gy)
        lib = nat.lib()
        gx = torch.empty((B, I), dtype=torch.float32, device=gy.device) if ctx.needs_input_grad[0] else None
        gl = torch.empty_like(luts)
        ws = _bytes(lib.dl_dwn_bwd_workspace_bytes(*ctx.dims), gy.device)
        nat.check(lib.dl_dwn_stable_layer_bwd(nat.ptr(x), nat.ptr(saved), nat.ptr(plan.idx32), nat.ptr(plan.inv_ptr),
                                              nat.ptr(plan.inv_pos), nat.ptr(luts), nat.ptr(gy), nat.ptr(scale),
                                              nat.ptr(gx), nat.ptr(gl), nat.ptr(ws), ws.numel(), *ctx.dims,
                                              nat.stream()))
        return gx, gl, None, None


class HybridLayerFunction(torch.autograd.Function):
    """Thresholded lookup forward, probabilistic backward on the real-valued inputs (hybrid_node.py:33-204)."""

    @staticmethod
    def forward(ctx, x, luts, plan):
        nat.require_device(x, luts)
        x, luts = _f32(x), _f32(luts)
        y, _, dims = _dwn_lookup(x, luts, plan)
        ctx.save_for_backward(x, luts)
        ctx.plan, ctx.dims = plan, dims
        return y

    @staticmethod
    def backward(ctx, gy):
        x, luts = ctx.saved_tensors
        B, I, N, k, O = ctx.dims
        plan = ctx.plan
        gy = _f32(gy)
        lib = nat.lib()
        gx = torch.empty((B, I), dtype=torch.float32, device=gy.device) if ctx.needs_input_grad[0] else None
        gl = torch.empty_like(luts)
        ws = _bytes(lib.dl_hybrid_bwd_workspace_bytes(*ctx.dims), gy.device)
        nat.check(lib.dl_hybrid_layer_bwd(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(plan.inv_ptr), nat.ptr(plan.inv_pos),
                                          nat.ptr(luts), nat.ptr(gy), nat.ptr(gx), nat.ptr(gl), nat.ptr(ws), ws.numel(),
                                          *ctx.dims, nat.stream()))
        return gx, gl, None


# ----------------------------------------------------------------------------- Probabilistic
def _node_temperatures(temperature, N, device):
    """None for one temperature (a number), else the nodes' own values as a float32 device array [N]."""
    if not torch.is_tensor(temperature):
        return None
    return temperature.detach().to(device=device, dtype=torch.float32).reshape(-1).expand(N).contiguous()


class ProbLayerFunction(torch.autograd.Function):
    """y[b, n*O+d] = sum_a sigmoid(raw[n,a,d]/T) prod_j (x_j a_j + (1-x_j)(1-a_j)); `temperature` is a number for the
    whole layer or a tensor [N] with every node's own value."""

    @staticmethod
    def forward(ctx, x, raw, plan, temperature):
        nat.require_device(x, raw)
        x, raw = _f32(x), _f32(raw)
        B, I = x.shape
        N, L, O = raw.shape
        k = plan.k
        if (N, 1 << k, I) != (plan.N, L, plan.I):
            raise RuntimeError(f"shape mismatch: x {tuple(x.shape)}, raw_weights {tuple(raw.shape)}, mapping "
                               f"[{plan.N},{k}] over {plan.I} inputs")
        y = torch.empty((B, N * O), dtype=torch.float32, device=x.device)
        dims = (B, I, N, k, O)
        saved = _bytes(nat.lib().dl_prob_saved_bytes(*dims), x.device)
        T = _node_temperatures(temperature, N, x.device)
        if T is None:
            nat.check(nat.lib().dl_prob_layer_fwd(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(raw), float(temperature),
                                                  nat.ptr(y), nat.ptr(saved), saved.numel(), *dims, nat.stream()))
        else:
            nat.check(nat.lib().dl_prob_layer_fwd_nodes(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(raw), nat.ptr(T),
                                                        nat.ptr(y), nat.ptr(saved), saved.numel(), *dims, nat.stream()))
        ctx.save_for_backward(x, raw, saved, T)
        ctx.plan, ctx.T, ctx.dims = plan, None if T is not None else float(temperature), dims
        return y

    @staticmethod
    def backward(ctx, gy):
        x, raw, saved, T = ctx.saved_tensors
        plan = ctx.plan
        gy = _f32(gy)
        lib = nat.lib()
        B, I = x.shape
        gx = torch.empty((B, I), dtype=torch.float32, device=gy.device) if ctx.needs_input_grad[0] else None
        graw = torch.empty_like(raw)
        ws = _bytes(lib.dl_prob_bwd_workspace_bytes(*ctx.dims), gy.device)
        if T is None:
            nat.check(lib.dl_prob_layer_bwd(nat.ptr(x), nat.ptr(saved), nat.ptr(plan.idx32), nat.ptr(plan.inv_ptr),
                                            nat.ptr(plan.inv_pos),
                                            nat.ptr(raw), ctx.T, nat.ptr(gy), nat.ptr(gx), nat.ptr(graw), nat.ptr(ws),
                                            ws.numel(), *ctx.dims, nat.stream()))
        else:
            nat.check(lib.dl_prob_layer_bwd_nodes(nat.ptr(x), nat.ptr(saved), nat.ptr(plan.idx32), nat.ptr(plan.inv_ptr),
                                                  nat.ptr(plan.inv_pos), nat.ptr(raw), nat.ptr(T), nat.ptr(gy), nat.ptr(gx),
                                                  nat.ptr(graw), nat.ptr(ws), ws.numel(), *ctx.dims, nat.stream()))
        return gx, graw, None, None


def prob_layer_eval(x, raw, plan, temperature):
    if not x.is_cuda:
        return cpu_ops.prob_layer_eval(x, raw, plan, temperature)
    nat.require_device(x, raw)
    x, raw = _f32(x), _f32(raw)
    B, I = x.shape
    N, _, O = raw.shape
    y = torch.empty((B, N * O), dtype=torch.float32, device=x.device)
    lib = nat.lib()
    dims = (B, I, N, plan.k, O)
    ws = _bytes(lib.dl_prob_eval_workspace_bytes(*dims), x.device)
    T = _node_temperatures(temperature, N, x.device)
    if T is None:
        nat.check(lib.dl_prob_layer_eval_ws(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(raw), float(temperature), nat.ptr(y),
                                            nat.ptr(ws), ws.numel(), *dims, nat.stream()))
    else:
        nat.check(lib.dl_prob_layer_eval_ws_nodes(nat.ptr(x), nat.ptr(plan.idx32), nat.ptr(raw), nat.ptr(T), nat.ptr(y),
                                                  nat.ptr(ws), ws.numel(), *dims, nat.stream()))
    return y


# ----------------------------------------------------------------------------- Learnable mapping
class SoftMapFunction(torch.autograd.Function):
    """m = x @ softmax(W / tau, dim=-1).T without materialising the softmax."""

    @staticmethod
    def forward(ctx, x, W, tau, precision):
        nat.require_device(x, W)
        x, W = _f32(x), _f32(W)
        B, I = x.shape
        M = W.shape[0]
        if W.shape[1] != I:
            raise RuntimeError(f"shape mismatch: x {tuple(x.shape)} vs W {tuple(W.shape)}")
        lib = nat.lib()
        m = torch.empty((B, M), dtype=torch.float32, device=x.device)
        stats = _bytes(lib.dl_soft_map_saved_bytes(B, I, M, precision), x.device)
        ws = _bytes(lib.dl_soft_map_workspace_bytes(B, I, M, precision), x.device)
        nat.check(lib.dl_soft_map_fwd(nat.ptr(x), nat.ptr(W), float(tau), nat.ptr(m), nat.ptr(stats), nat.ptr(ws),
                                      ws.numel(), B, I, M, precision, nat.stream()))
        ctx.save_for_backward(x, W, m, stats)
        ctx.tau, ctx.precision = float(tau), precision
        return m

    @staticmethod
    def backward(ctx, gm):
        x, W, m, stats = ctx.saved_tensors
        gm = _f32(gm)
        B, I = x.shape
        M = W.shape[0]
        lib = nat.lib()
        gx = torch.empty_like(x)
        gW = torch.empty_like(W)
        ws = _bytes(lib.dl_soft_map_workspace_bytes(B, I, M, ctx.precision), x.device)
        nat.check(lib.dl_soft_map_bwd(nat.ptr(x), nat.ptr(W), ctx.tau, nat.ptr(m), nat.ptr(stats), nat.ptr(gm),
                                      nat.ptr(gx), nat.ptr(gW), nat.ptr(ws), ws.numel(), B, I, M, ctx.precision,
                                      nat.stream()))
        return gx, gW, None, None


def row_argmax(W):
    if not W.is_cuda:
        return cpu_ops.row_argmax(W)
    nat.require_device(W)
    W = _f32(W)
    sel = torch.empty((W.shape[0],), dtype=torch.int32, device=W.device)
    nat.check(nat.lib().dl_row_argmax(nat.ptr(W), nat.ptr(sel), W.shape[0], W.shape[1], nat.stream()))
    return sel


class HardSelectFunction(torch.autograd.Function):
    """m[b,o] = x[b, sel[o]] with the straight scatter-add backward."""

    @staticmethod
    def forward(ctx, x, sel, plan):
        nat.require_device(x, sel)
        x = _f32(x)
        B, I = x.shape
        M = sel.numel()
        m = torch.empty((B, M), dtype=torch.float32, device=x.device)
        nat.check(nat.lib().dl_hard_select_fwd(nat.ptr(x), nat.ptr(sel.contiguous().int()), nat.ptr(m), B, I, M,
                                               nat.stream()))
        ctx.plan, ctx.shape = plan, (B, I, M)
        return m

    @staticmethod
    def backward(ctx, gm):
        B, I, M = ctx.shape
        gm = _f32(gm)
        gx = torch.empty((B, I), dtype=torch.float32, device=gm.device)
        p = ctx.plan
        nat.check(nat.lib().dl_hard_select_bwd(nat.ptr(gm), nat.ptr(p.inv_ptr), nat.ptr(p.inv_pos), nat.ptr(gx), B, I, M,
                                               nat.stream()))
        return gx, None, None


# ----------------------------------------------------------------------------- encoder / head
def thermometer_encode(x, thresholds):
    if not x.is_cuda:
        return cpu_ops.thermometer_encode(x, thresholds)
    nat.require_device(x, thresholds)
    x, thr = _f32(x), _f32(thresholds)
    B, F = x.shape
    nbits = thr.shape[1]
    bits = torch.empty((B, F, nbits), dtype=torch.float32, device=x.device)
    nat.check(nat.lib().dl_thermometer_encode(nat.ptr(x), nat.ptr(thr), nat.ptr(bits), B, F, nbits, nat.stream()))
    return bits


class CrossEntropyFunction(torch.autograd.Function):
    """Mean cross-entropy of [B, C] logits against int64 class labels: loss and its gradient from one pass
    (what torch.nn.functional.cross_entropy and its backward compute for the logits GroupSum returns)."""

    @staticmethod
    def forward(ctx, logits, labels):
        nat.require_device(logits, labels)
        logits = _f32(logits)
        if logits.dim() != 2 or labels.shape != (logits.shape[0],):
            raise RuntimeError(f"expected logits [B, C] and labels [B], got {tuple(logits.shape)} and {tuple(labels.shape)}")
        labels = labels.to(torch.int64).contiguous()
        B, C = logits.shape
        lib = nat.lib()
        loss = torch.empty((), dtype=torch.float32, device=logits.device)
        glogits = torch.empty_like(logits)
        ws = _bytes(lib.dl_cross_entropy_workspace_bytes(B), logits.device)
        nat.check(lib.dl_cross_entropy(nat.ptr(logits), nat.ptr(labels), nat.ptr(loss), nat.ptr(glogits), nat.ptr(ws),
                                       ws.numel(), B, C, nat.stream()))
        ctx.save_for_backward(glogits)
        return loss

    @staticmethod
    def backward(ctx, gloss):
        (glogits,) = ctx.saved_tensors
        return glogits * gloss, None


class GroupSumFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, groups, tau):
        nat.require_device(x)
        x = _f32(x)
        B, F = x.shape
        y = torch.empty((B, groups), dtype=torch.float32, device=x.device)
        nat.check(nat.lib().dl_group_sum_fwd(nat.ptr(x), nat.ptr(y), B, F, groups, float(tau), nat.stream()))
        ctx.args = (B, F, groups, float(tau))
        return y

    @staticmethod
    def backward(ctx, gy):
        B, F, groups, tau = ctx.args
        gy = _f32(gy)
        gx = torch.empty((B, F), dtype=torch.float32, device=gy.device)
        nat.check(nat.lib().dl_group_sum_bwd(nat.ptr(gy), nat.ptr(gx), B, F, groups, tau, nat.stream()))
        return gx, None, None


# ----------------------------------------------------------------------------- dispatch
# The reference's rule (random_layer.py:272, dwn_node.py:334, probabilistic_node.py:277): the extension runs iff the
# input is a device tensor, otherwise the CPU code does.  Layers, nodes, the encoder and the head call these.
def gather(x, idx, plan):
    return GatherFunction.apply(x, idx, plan) if x.is_cuda else cpu_ops.gather(x, idx)


def dwn_layer(x, luts, plan, alpha, beta, beta_abs_max=None):
    if x.is_cuda:
        return DWNLayerFunction.apply(x, luts, plan, alpha, beta, beta_abs_max)
    return cpu_ops.dwn_layer(x, luts, plan, alpha, beta)


def dwn_stable_layer(x, luts, scale, plan):
    return DWNStableLayerFunction.apply(x, luts, scale, plan) if x.is_cuda else cpu_ops.dwn_stable_layer(x, luts, scale, plan)


def hybrid_layer(x, luts, plan):
    return HybridLayerFunction.apply(x, luts, plan) if x.is_cuda else cpu_ops.hybrid_layer(x, luts, plan)


def table_sigmoid(raw):
    return TableSigmoidFunction.apply(raw) if raw.is_cuda else torch.sigmoid(raw.float())


def prob_layer(x, raw, plan, temperature):
    return ProbLayerFunction.apply(x, raw, plan, temperature) if x.is_cuda else cpu_ops.prob_layer(x, raw, plan, temperature)


def soft_map(x, W, tau, precision=0):
    return SoftMapFunction.apply(x, W, tau, precision) if x.is_cuda else cpu_ops.soft_map(x, W, tau, precision)


def hard_select(x, sel, plan):
    return HardSelectFunction.apply(x, sel, plan) if x.is_cuda else cpu_ops.hard_select(x, sel)


def unfold(x, geom, flip=None):
    """Patch matrix [B*OH*OW, C*KH*KW] of an image batch; on the CPU nn.functional.unfold, transposed and flattened
    as convolutional.py:199-205 does, with the flip applied to the patches."""
    if x.is_cuda:
        return UnfoldFunction.apply(x, geom, flip)
    kh, kw, sh, sw, ph, pw = geom
    cols = torch.nn.functional.unfold(x.float(), (kh, kw), padding=(ph, pw), stride=(sh, sw))
    patches = cols.transpose(1, 2).reshape(-1, cols.shape[1])
    if flip is not None:
        patches = patches + torch.where(flip.bool(), 1.0 - 2.0 * patches.detach(), torch.zeros_like(patches))
    return patches


def grad_stabilize(grad, per_row, target_std, subtract_mean, eps):
    """(grad - mean) * sqrt(target_std / (mean((grad - mean)^2) + eps)) for a [rows, cols] gradient on the device, over
    the whole tensor or per row (base_layer.py:266-339); a new tensor."""
    nat.require_device(grad)
    g = _f32(grad)
    rows, cols = g.shape
    out = torch.empty_like(g)
    lib = nat.lib()
    ws = _bytes(lib.dl_grad_stabilize_workspace_bytes(rows, cols, int(per_row)), g.device)
    nat.check(lib.dl_grad_stabilize(nat.ptr(g), nat.ptr(out), rows, cols, int(per_row), float(target_std),
                                    int(bool(subtract_mean)), float(eps), nat.ptr(ws), ws.numel(), nat.stream()))
    return out


def group_sum(x, groups, tau):
    return GroupSumFunction.apply(x, groups, tau) if x.is_cuda else cpu_ops.group_sum(x, groups, tau)


def cross_entropy(logits, labels):
    if logits.is_cuda:
        return CrossEntropyFunction.apply(logits, labels)
    return torch.nn.functional.cross_entropy(logits.float(), labels.long())
