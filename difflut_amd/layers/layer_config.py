"""Training options shared by the LUT layers (difflut/layers/layer_config.py:14-137)."""
from dataclasses import dataclass

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
