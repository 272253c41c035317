"""mapping_cuda.forward/backward (difflut/layers/cuda/mapping_cuda.cpp:25-74)."""
from _common import check_cuda_contiguous, nat, plan_for, torch


def forward(input, indices):
    check_cuda_contiguous(input, indices)
    if input.dim() != 2 or indices.dim() != 2:
        raise RuntimeError("Input must be 2D (batch_size, input_size); Indices must be 2D (output_size, n)")
    if input.dtype != torch.float32:
        raise RuntimeError("Input must be float32")
    bits = {torch.int16: 16, torch.int32: 32}.get(indices.dtype)
    if bits is None:
        raise RuntimeError("Indices must be int16 or int32")
    B, I = input.shape
    N, k = indices.shape
    out = torch.empty((B, N, k), dtype=torch.float32, device=input.device)
    nat.check(nat.lib().dl_gather_fwd(input.data_ptr(), indices.data_ptr(), bits, out.data_ptr(), B, I, N, k,
                                      nat.stream()))
    return out


def backward(grad_output, indices, input_size):
    check_cuda_contiguous(grad_output, indices)
    if grad_output.dim() != 3:
        raise RuntimeError("Grad output must be 3D (batch_size, output_size, n)")
    plan = plan_for(indices, input_size)
    B, N, k = grad_output.shape
    gx = torch.empty((B, input_size), dtype=torch.float32, device=grad_output.device)
    nat.check(nat.lib().dl_gather_bwd(grad_output.data_ptr(), plan.inv_ptr.data_ptr(), plan.inv_pos.data_ptr(),
                                      gx.data_ptr(), B, input_size, N, k, nat.stream()))
    return gx
