"""probabilistic_cuda.forward/backward (difflut/nodes/cuda/probabilistic_cuda.cpp:22-49): one node,
input [B,k], raw_weights [L,O], temperature as a 0-d tensor."""
from _common import check_cuda_contiguous, nat, ops, torch

_identity = {}


def _plan(k, device):
    key = (k, str(device))
    if key not in _identity:
        _identity[key] = ops.MappingPlan.identity(k, device)
    return _identity[key]


def forward(input, raw_weights, temperature):
    check_cuda_contiguous(input, raw_weights)
    B, k = input.shape
    L, O = raw_weights.shape
    y = torch.empty((B, O), dtype=torch.float32, device=input.device)
    plan = _plan(k, input.device)
    lib = nat.lib()
    ws = torch.empty(max(lib.dl_prob_saved_bytes(B, k, 1, k, O), 256), dtype=torch.uint8, device=input.device)
    nat.check(lib.dl_prob_layer_fwd(input.data_ptr(), plan.idx32.data_ptr(), raw_weights.data_ptr(),
                                    float(temperature), y.data_ptr(), ws.data_ptr(), ws.numel(), B, k, 1, k, O,
                                    nat.stream()))
    return y


def backward(input, raw_weights, temperature, grad_output):
    check_cuda_contiguous(input, raw_weights, grad_output)
    B, k = input.shape
    L, O = raw_weights.shape
    plan = _plan(k, input.device)
    lib = nat.lib()
    gx = torch.empty_like(input)
    gw = torch.empty_like(raw_weights)
    ws = torch.empty(max(lib.dl_prob_bwd_workspace_bytes(B, k, 1, k, O), 256), dtype=torch.uint8, device=input.device)
    nat.check(lib.dl_prob_layer_bwd(input.data_ptr(), None, plan.idx32.data_ptr(), plan.inv_ptr.data_ptr(),
                                    plan.inv_pos.data_ptr(), raw_weights.data_ptr(), float(temperature),
                                    grad_output.data_ptr(), gx.data_ptr(), gw.data_ptr(), ws.data_ptr(), ws.numel(),
                                    B, k, 1, k, O, nat.stream()))
    return [gx, gw]
