from .initializers import normal_init, ones_init, residual_init, uniform_init, zeros_init

__all__ = ["zeros_init", "ones_init", "normal_init", "uniform_init", "residual_init"]
