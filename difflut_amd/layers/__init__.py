"""Layers on the accelerated path; importing registers them."""
from .base_layer import BaseLUTLayer
from .layer_config import LayerConfig
from .learnable_layer import LearnableLayer
from .random_layer import RandomLayer
from .dwn_stack import DWNStack

__all__ = ["BaseLUTLayer", "RandomLayer", "LearnableLayer", "LayerConfig", "DWNStack"]
