"""RandomLayer: LUT layer with a seeded, fixed random input mapping.

Constructor, buffer name (`_mapping_indices`, int16 below 32768 inputs else int32), seeding
rule and `get_mapping`/`get_mapping_matrix` follow difflut/layers/random_layer.py:123-356.
forward() differs in how it gets there: for DWN / Probabilistic nodes the gather, all N nodes
and (in backward) the scatter run as one fused device call and the [batch, N, n] tensor is
never written; other node types take the gather kernel plus a per-node loop.  CPU tensors take
the plain-torch branch of the same operators (the reference's rule: the extension iff `x.is_cuda`).
"""
import torch

from .. import _native, ops
from ..registry import register_layer
from .base_layer import BaseLUTLayer

DEFAULT_RANDOM_LAYER_SEED = 42
_MAPPING_CUDA_AVAILABLE = _native.is_built()


def draw_mapping(input_size, output_size, n, seed, ensure_full_input_coverage=True, mapping_indices=None):
    """Index table [output_size, n].  With full coverage every input is used once before any is
    reused: floor(N*n/I) permutations of all inputs followed by N*n mod I distinct draws, taken from
    torch's CPU generator seeded with `seed`; the caller's generator state is restored afterwards."""
    saved = torch.get_rng_state()
    torch.manual_seed(seed)
    dtype = torch.int16 if input_size < 32768 else torch.int32
    if mapping_indices is not None:
        table = mapping_indices.to(dtype=dtype)
    elif not ensure_full_input_coverage:
        table = torch.multinomial(torch.ones((output_size, input_size)), num_samples=n,
                                  replacement=n > input_size).to(dtype=dtype)
    else:
        cycles, rest = divmod(output_size * n, input_size)
        parts = [torch.randperm(input_size) for _ in range(cycles)]
        if rest > 0:
            parts.append(torch.multinomial(torch.ones(input_size), num_samples=rest, replacement=False))
        table = torch.cat(parts).reshape(output_size, n).to(dtype=dtype)
    torch.set_rng_state(saved)
    return table


def mapping_forward_cuda(input, indices, input_size):
    """Gather with autograd on a device tensor, None otherwise (random_layer.py:103-120)."""
    if _MAPPING_CUDA_AVAILABLE and input.is_cuda:
        return ops.GatherFunction.apply(input, indices, ops.MappingPlan(indices, input_size))
    return None


@register_layer("random")
class RandomLayer(BaseLUTLayer):
    def __init__(self, input_size, output_size, node_type, node_kwargs, seed=DEFAULT_RANDOM_LAYER_SEED,
                 layer_config=None, flip_probability=None, grad_stabilization=None, grad_target_std=None,
                 grad_subtract_mean=None, grad_epsilon=None, ensure_full_input_coverage=True, mapping_indices=None):
        self.seed = seed
        super().__init__(input_size=input_size, output_size=output_size, node_type=node_type, node_kwargs=node_kwargs,
                         layer_config=layer_config, flip_probability=flip_probability,
                         grad_stabilization=grad_stabilization, grad_target_std=grad_target_std,
                         grad_subtract_mean=grad_subtract_mean, grad_epsilon=grad_epsilon)
        self._init_mapping(ensure_full_input_coverage, mapping_indices)

    def _init_mapping(self, ensure_full_input_coverage=True, mapping_indices=None):
        table = draw_mapping(self.input_size, self.output_size, self.n, self.seed, ensure_full_input_coverage,
                             mapping_indices)
        self.register_buffer("_mapping_indices", table)
        self._plan = None

    def mapping_plan(self):
        """Device form of the index table (widened copy + CSR inverse), rebuilt when the buffer changes."""
        if self._plan is None or not self._plan.matches(self._mapping_indices):
            self._plan = ops.MappingPlan(self._mapping_indices, self.input_size)
        return self._plan

    def get_mapping(self, x):
        return ops.gather(x, self._mapping_indices, self.mapping_plan())

    def get_mapping_indices(self):
        return self._mapping_indices.long()

    def forward(self, x):
        self._validate_input_dims(x)
        out = self._run_nodes(x, self.mapping_plan())
        if out is None:
            out = self._loop_nodes(self.get_mapping(x))
        return out

    def get_mapping_matrix(self):
        return self._mapping_indices.long()

    def extra_repr(self):
        flip = f", flip_prob={self.flip_probability}" if self.flip_probability > 0 else ""
        stab = f", grad_stab={self.grad_stabilization}" if self.grad_stabilization != "none" else ""
        return (f"input_size={self.input_size}, output_size={self.output_size}, n={self.n}, seed={self.seed}, "
                f"mapping=random{flip}{stab}")
