"""hybrid_cuda.forward/backward (difflut/nodes/cuda/hybrid_cuda.cpp:19-44): one node, input [B,k],
luts [O,L]; binary_combinations [L,k] is accepted and not read (the kernels enumerate the corners,
input 0 = least significant bit, which is the table the reference builds)."""
import efd_cuda
from _common import check_cuda_contiguous, nat, torch
from probabilistic_cuda import _plan


def forward(input, luts):
    return efd_cuda.forward(input, luts)


def backward(input, luts, binary_combinations, grad_output):
    check_cuda_contiguous(input, luts, grad_output)
    B, k = input.shape
    O = luts.shape[0]
    dims = (B, k, 1, k, O)
    plan = _plan(k, input.device)
    lib = nat.lib()
    ws = torch.empty(lib.dl_hybrid_bwd_workspace_bytes(*dims), dtype=torch.uint8, device=input.device)
    gx = torch.empty_like(input)
    gl = torch.empty_like(luts)
    nat.check(lib.dl_hybrid_layer_bwd(input.data_ptr(), plan.idx32.data_ptr(), plan.inv_ptr.data_ptr(),
                                      plan.inv_pos.data_ptr(), luts.data_ptr(), grad_output.data_ptr(), gx.data_ptr(),
                                      gl.data_ptr(), ws.data_ptr(), ws.numel(), *dims, nat.stream()))
    return [gx, gl]
