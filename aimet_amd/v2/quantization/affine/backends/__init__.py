"""v2 affine quantization functions, dispatched to the current backend
(TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/backends/__init__.py:178-179, 325-370)."""
import math

from .utils import add_backend, get_backend, set_backend, set_global_backend


def quantize(tensor, scale, offset, qmin, qmax, block_size=None):
    return get_backend().quantize(tensor, scale, offset, qmin, qmax, block_size)


def quantize_dequantize(tensor, scale, offset, qmin, qmax, block_size=None):
    return get_backend().quantize_dequantize(tensor, scale, offset, qmin, qmax, block_size)


def dequantize(tensor, scale, offset, block_size=None):
    return get_backend().dequantize(tensor, scale, offset, block_size)


def _derive_qmin_qmax(*, bitwidth: int = None, num_steps: int = None, signed: bool):
    if bitwidth is not None:
        num_steps = 2 ** bitwidth - 1
    if signed:
        return -math.ceil(num_steps / 2), math.floor(num_steps / 2)
    return 0, num_steps


__all__ = ['quantize', 'quantize_dequantize', 'dequantize', 'add_backend', 'get_backend', 'set_backend',
           'set_global_backend']
