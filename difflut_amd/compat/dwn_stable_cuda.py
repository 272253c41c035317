"""dwn_stable_cuda.forward/backward (difflut/nodes/cuda/dwn_stable_cuda.cpp:19-43): one node,
input [B,k], luts [O,L] already in [0,1], gradient_scale a Python float."""
import efd_cuda
from _common import check_cuda_contiguous, nat, ops, torch
from probabilistic_cuda import _plan


def forward(input, luts):
    return efd_cuda.forward(input, luts)


def backward(input, luts, grad_output, gradient_scale):
    check_cuda_contiguous(input, luts, grad_output)
    B, k = input.shape
    O = luts.shape[0]
    dims = (B, k, 1, k, O)
    plan = _plan(k, input.device)
    lib = nat.lib()
    saved = torch.empty(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device=input.device)
    ws = torch.empty(max(lib.dl_dwn_fwd_workspace_bytes(*dims), lib.dl_dwn_bwd_workspace_bytes(*dims)), dtype=torch.uint8,
                     device=input.device)
    y = torch.empty((B, O), dtype=torch.float32, device=input.device)
    # the legacy signature hands over x, not the addresses the forward saved: look them up again
    nat.check(lib.dl_dwn_layer_fwd(input.data_ptr(), plan.idx32.data_ptr(), luts.data_ptr(), y.data_ptr(),
                                   saved.data_ptr(), ws.data_ptr(), ws.numel(), *dims, nat.stream()))
    scale = torch.full((1,), float(gradient_scale), dtype=torch.float32, device=input.device)
    gx = torch.empty_like(input)
    gl = torch.empty_like(luts)
    nat.check(lib.dl_dwn_stable_layer_bwd(input.data_ptr(), saved.data_ptr(), plan.idx32.data_ptr(),
                                          plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(), luts.data_ptr(),
                                          grad_output.data_ptr(), scale.data_ptr(), gx.data_ptr(), gl.data_ptr(),
                                          ws.data_ptr(), ws.numel(), *dims, nat.stream()))
    return [gx, gl]
