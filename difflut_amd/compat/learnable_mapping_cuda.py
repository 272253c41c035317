"""learnable_mapping_cuda.forward/soft_forward/backward
(difflut/layers/cuda/learnable_mapping_cuda.cpp:30-99)."""
from _common import check_cuda_contiguous, nat, ops, plan_for, torch


def forward(input, indices):
    check_cuda_contiguous(input, indices)
    B, I = input.shape
    M = indices.numel()
    out = torch.empty((B, M), dtype=torch.float32, device=input.device)
    nat.check(nat.lib().dl_hard_select_fwd(input.data_ptr(), indices.data_ptr(), out.data_ptr(), B, I, M, nat.stream()))
    return out


def soft_forward(input, weights, tau):
    return ops.SoftMapFunction.apply(input, weights.detach(), float(tau), 0)


def backward(grad_output, indices, input_size):
    check_cuda_contiguous(grad_output, indices)
    plan = plan_for(indices.view(-1, 1), input_size)
    B, M = grad_output.shape
    gx = torch.empty((B, input_size), dtype=torch.float32, device=grad_output.device)
    nat.check(nat.lib().dl_hard_select_bwd(grad_output.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(),
                                           gx.data_ptr(), B, input_size, M, nat.stream()))
    return gx
