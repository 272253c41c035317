"""Parameter initialisers that the hot-path configurations and known-answer tests use
(difflut/nodes/utils/initializers.py:40-113 and :553-631, :788-1000 for the LUT branch of
residual_init).  All are host-side, one-shot and modify the tensor in place."""
import torch

from ...registry import register_initializer
from ...utils.warnings import warn_default_value


@register_initializer("zeros")
def zeros_init(param, **kwargs):
    with torch.no_grad():
        param.zero_()


@register_initializer("ones")
def ones_init(param, **kwargs):
    with torch.no_grad():
        param.fill_(1.0)


@register_initializer("normal")
def normal_init(param, mean=0.0, std=1.0, **kwargs):
    with torch.no_grad():
        param.normal_(mean, std)


@register_initializer("uniform")
def uniform_init(param, a=-1.0, b=1.0, **kwargs):
    with torch.no_grad():
        param.uniform_(a, b)


def _residual_lut(param, input_dim, noise_factor, logit_clarity):
    """Truth table of 'output = input 0': +clarity where address bit 0 is set, -clarity elsewhere,
    plus N(0, noise^2) drawn per table entry in address order (one randn(output_dim) per entry)."""
    size = 2 ** input_dim
    with torch.no_grad():
        if param.shape[0] == size:
            entries = lambda a: param[a, :]  # noqa: E731  [2^k, O] (probabilistic)
            out_dim = param.shape[1]
        elif param.dim() > 1 and param.shape[1] == size:
            entries = lambda a: param[:, a]  # noqa: E731  [O, 2^k] (dwn)
            out_dim = param.shape[0]
        else:  # unknown orientation
            param.normal_(0, noise_factor) if noise_factor > 0 else param.zero_()
            return
        for a in range(size):
            base = logit_clarity if a & 1 else -logit_clarity
            if noise_factor > 0:
                entries(a).copy_(base + torch.randn(out_dim, device=param.device, dtype=param.dtype) * noise_factor)
            else:
                entries(a).fill_(base)


@register_initializer("residual")
def residual_init(param, node_type=None, param_name=None, input_dim=None, output_dim=None, noise_factor=0.0,
                  logit_clarity=5.0, **kwargs):
    if noise_factor == 0.0:
        warn_default_value("noise_factor (residual_init)", noise_factor, stacklevel=3)
    if logit_clarity == 5.0:
        warn_default_value("logit_clarity (residual_init)", logit_clarity, stacklevel=3)
    if node_type is None:
        raise ValueError("residual_init requires 'node_type' to determine initialization strategy.")
    kind = node_type.lower()
    if kind in ("dwn", "dwn_stable", "probabilistic", "hybrid"):
        if input_dim is None:
            raise ValueError(f"residual_init for {kind} nodes requires 'input_dim' to determine truth table size")
        _residual_lut(param, input_dim, noise_factor, logit_clarity)
    else:
        raise ValueError(f"Unknown node_type '{node_type}' for residual initialization in this build; "
                         "the table-based node types are 'dwn', 'dwn_stable', 'probabilistic', 'hybrid'.")
