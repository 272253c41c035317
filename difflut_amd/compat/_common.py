import torch

from difflut_amd import _native as nat
from difflut_amd import ops

_plans = {}


def plan_for(indices, input_size):
    """MappingPlan cached on the identity of the index tensor."""
    key = (indices.data_ptr(), indices._version, tuple(indices.shape), int(input_size), str(indices.device))
    plan = _plans.get(key)
    if plan is None:
        if len(_plans) > 64:
            _plans.clear()
        plan = _plans[key] = ops.MappingPlan(indices, input_size)
    return plan


def check_cuda_contiguous(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("input must be a CUDA tensor")
        if not t.is_contiguous():
            raise RuntimeError("input must be contiguous")


__all__ = ["torch", "nat", "ops", "plan_for", "check_cuda_contiguous"]
