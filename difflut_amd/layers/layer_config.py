"""Training options shared by the LUT layers (difflut/layers/layer_config.py:14-137) and the grouped
input mapping of the convolutional layer (layer_config.py:141-220)."""
from dataclasses import dataclass

import torch

GRAD_MODES = ("none", "layerwise", "batchwise")


def validate_layer_options(flip_probability, grad_stabilization, grad_target_std, grad_epsilon):
    if not isinstance(flip_probability, (int, float)) or not 0.0 <= flip_probability <= 1.0:
        raise ValueError(f"flip_probability must be a float in [0, 1], got {flip_probability}.")
    if grad_stabilization not in GRAD_MODES:
        raise ValueError(f"grad_stabilization must be one of {list(GRAD_MODES)}, got '{grad_stabilization}'.")
    if not isinstance(grad_target_std, (int, float)) or grad_target_std <= 0:
        raise ValueError(f"grad_target_std must be a positive number, got {grad_target_std}.")
    if not isinstance(grad_epsilon, (int, float)) or grad_epsilon <= 0:
        raise ValueError(f"grad_epsilon must be a positive number, got {grad_epsilon}.")


@dataclass
class LayerConfig:
    flip_probability: float = 0.0
    grad_stabilization: str = "none"
    grad_target_std: float = 1.0
    grad_subtract_mean: bool = False
    grad_epsilon: float = 1e-8

    def __post_init__(self):
        validate_layer_options(self.flip_probability, self.grad_stabilization, self.grad_target_std, self.grad_epsilon)

    def copy(self):
        return LayerConfig(self.flip_probability, self.grad_stabilization, self.grad_target_std,
                           self.grad_subtract_mean, self.grad_epsilon)


class GroupedInputConfig:
    """Index table in which every node reads from one group (channel) of the inputs only.

    [output_trees * luts_per_tree, bits_per_node] positions inside a group drawn row by row without
    replacement, plus a group offset per node: with full coverage the groups are dealt out as
    floor(nodes / n_groups) permutations followed by distinct draws for the rest, otherwise uniformly.
    All draws come from torch's CPU generator seeded with `seed`, in that order; the caller's
    generator state is restored."""

    def __init__(self, n_groups, input_size, output_trees, luts_per_tree, bits_per_node, seed, ensure_full_coverage=True):
        if n_groups < 1:
            raise ValueError(f"n_groups must be >= 1, got {n_groups}. Example: n_groups=4 for 4 input groups.")
        self.n_groups = n_groups
        self.luts_per_tree = luts_per_tree
        nodes = output_trees * luts_per_tree
        saved = torch.get_rng_state()
        torch.manual_seed(seed)
        group_size = input_size // n_groups
        table = torch.multinomial(torch.ones((nodes, group_size)), num_samples=bits_per_node,
                                  replacement=bits_per_node > group_size)
        if not ensure_full_coverage:
            groups = torch.randint(low=0, high=n_groups, size=(nodes, 1))
        else:
            cycles, rest = divmod(nodes, n_groups)
            parts = [torch.randperm(n_groups) for _ in range(cycles)]
            if rest > 0:
                parts.append(torch.multinomial(torch.ones((n_groups,)), num_samples=rest, replacement=False))
            groups = torch.cat(parts).unsqueeze(1)
        self.mapping_indices = table + groups * group_size
        torch.set_rng_state(saved)

    def get_mapping_indices(self, chunk_start, chunk_end):
        """Rows of the trees chunk_start .. chunk_end - 1."""
        return self.mapping_indices[chunk_start * self.luts_per_tree:chunk_end * self.luts_per_tree, :]
