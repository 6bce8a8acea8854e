"""Fused ops with the reference's names (megalodon/modules/fused_ops/__init__.py:1-14)."""
from .ema_parameters import ema_parameters
from .fftconv import fftconv

__all__ = ["ema_parameters", "fftconv"]
