"""Layers on the accelerated path; importing registers them."""
from .base_layer import BaseLUTLayer
from .convolutional import ConvolutionalLayer, ConvolutionConfig
from .layer_config import GroupedInputConfig, LayerConfig
from .learnable_layer import LearnableLayer
from .random_layer import RandomLayer
from .dwn_stack import DWNStack

__all__ = ["BaseLUTLayer", "RandomLayer", "LearnableLayer", "LayerConfig", "GroupedInputConfig", "DWNStack",
           "ConvolutionalLayer", "ConvolutionConfig"]
