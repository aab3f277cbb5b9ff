"""v2 simulation model and the helpers that reconfigure its quantizers (aimet_torch/v2/quantsim/__init__.py)."""
from .quantsim import QuantizationSimModel

__all__ = ['QuantizationSimModel']
