from .base_encoder import BaseEncoder
from .thermometer import ThermometerEncoder

__all__ = ["BaseEncoder", "ThermometerEncoder"]
