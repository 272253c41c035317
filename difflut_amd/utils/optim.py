"""Adam over a model's parameter banks in one device launch.

The reference trains with `torch.optim.Adam(model.parameters(), ...)` over N small per-node Parameters.  Here the
nodes' parameters of a layer live in one tensor (`layer.bank_parameters()`), and `BankAdam` updates all such tensors of a
model with ONE kernel launch per step (`dl_adam_step`): the same arithmetic as torch.optim.Adam without amsgrad
(bias-corrected first and second moments, optional L2 weight decay, `maximize`).  CPU tensors, other dtypes and sparse
cases take plain torch operations with the same formula.
"""
import ctypes
import math

import torch


class BankAdam(torch.optim.Optimizer):
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, maximize=False):
        if lr < 0.0 or eps < 0.0 or weight_decay < 0.0 or not (0.0 <= betas[0] < 1.0 and 0.0 <= betas[1] < 1.0):
            raise ValueError("invalid Adam hyper-parameters")
        super().__init__(params, dict(lr=lr, betas=tuple(betas), eps=eps, weight_decay=weight_decay, maximize=maximize))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            device_batch = []
            group["_step"] = step = group.get("_step", 0) + 1
            beta1, beta2 = group["betas"]
            for p in group["params"]:
                g = p.grad
                if g is None:
                    continue
                state = self.state[p]
                if not state:
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                m, v = state["exp_avg"], state["exp_avg_sq"]
                if (p.is_cuda and p.dtype == torch.float32 and g.dtype == torch.float32 and p.is_contiguous()
                        and g.is_contiguous() and not g.is_sparse):
                    device_batch.append((p, g, m, v))
                    continue
                if group["maximize"]:
                    g = -g
                if group["weight_decay"] != 0.0:
                    g = g.add(p, alpha=group["weight_decay"])
                m.lerp_(g, 1.0 - beta1)
                v.mul_(beta2).addcmul_(g, g, value=1.0 - beta2)
                bc1, bc2 = 1.0 - beta1 ** step, 1.0 - beta2 ** step
                denom = (v.sqrt() / math.sqrt(bc2)).add_(group["eps"])
                p.addcdiv_(m, denom, value=-group["lr"] / bc1)
            if device_batch:
                self._device_step(device_batch, group, step)
        return loss

    @staticmethod
    def _device_step(batch, group, step):
        from .. import _native as nat

        by_device = {}
        for item in batch:
            by_device.setdefault(item[0].device, []).append(item)
        for device, items in by_device.items():
            count = len(items)
            ptrs = [(ctypes.c_void_p * count)(*[t[i].data_ptr() for t in items]) for i in range(4)]
            numel = (ctypes.c_longlong * count)(*[t[0].numel() for t in items])
            with torch.cuda.device(device):
                nat.check(nat.lib().dl_adam_step(ptrs[0], ptrs[1], ptrs[2], ptrs[3], numel, count, float(group["lr"]),
                                                 float(group["betas"][0]), float(group["betas"][1]), float(group["eps"]),
                                                 float(group["weight_decay"]), int(step), int(bool(group["maximize"])),
                                                 nat.stream()))
