"""Device availability helper kept under the reference's module path (difflut/nodes/cuda/__init__.py)."""
import torch


def is_cuda_available():
    """True when a ROCm device is visible (torch reports it under the 'cuda' name)."""
    return torch.cuda.is_available()


__all__ = ["is_cuda_available"]
